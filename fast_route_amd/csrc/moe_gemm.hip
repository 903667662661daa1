// Host side of the grouped expert GEMMs: tile selection, launches, top-k combine.
#include "moe_gemm_tiles.h"
#include "moe_gemv.h"

namespace fr {

// ---- top-k combine: out[m] = sum over splits and slots of partial ------------
// P = float (one fp32 slice per K split) or the operand type (single slice: each pair's row
// rounded once before the sum over its token's slots, as the reference's second GEMM writes it,
// fast_route/fast_route/ops/fused_moe.py:117-123, before torch.sum).
template <typename T, typename P, int V>
__global__ __launch_bounds__(256) void combine_kernel(const P* __restrict__ partial,
                                                      int64_t split_stride, int splits, int topk,
                                                      int64_t M, int H, T* __restrict__ out,
                                                      const int32_t* __restrict__ pair_ids, int E) {
  typedef P pv __attribute__((ext_vector_type(V)));
  typedef T tv __attribute__((ext_vector_type(V)));
  const int64_t idx = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * V;
  if (idx >= M * H) return;
  const int64_t m = idx / H;
  const int h = static_cast<int>(idx % H);
  float s[V];
#pragma unroll
  for (int r = 0; r < V; ++r) s[r] = 0.f;
  for (int j = 0; j < topk; ++j) {
    if (pair_ids) {  // a pair whose expert id lies outside [0, E) got no slot in the routing arrays: no row was written for it
      const int e = pair_ids[m * topk + j];
      if (e < 0 || e >= E) continue;
    }
    for (int sp = 0; sp < splits; ++sp) {
      const pv v = *reinterpret_cast<const pv*>(partial + sp * split_stride + (m * topk + j) * H + h);
#pragma unroll
      for (int r = 0; r < V; ++r) s[r] += static_cast<float>(v[r]);
    }
  }
  tv o;
#pragma unroll
  for (int r = 0; r < V; ++r) o[r] = static_cast<T>(s[r]);
  *reinterpret_cast<tv*>(out + idx) = o;
}

// ---- tile launches: instantiated per (element type, epilogue) in moe_gemm_inst_*.hip ---------
#define FR_DECLARE_TILES(T)                                                                       \
  extern template int dispatch_block<T, EPI_PLAIN>(GemmArgs, int, int, int64_t, hipStream_t);     \
  extern template int dispatch_block<T, EPI_SILU>(GemmArgs, int, int, int64_t, hipStream_t);      \
  extern template int dispatch_block<T, EPI_DOWN>(GemmArgs, int, int, int64_t, hipStream_t);      \
  extern template int prepare_tiles<T, EPI_PLAIN>();                                              \
  extern template int prepare_tiles<T, EPI_SILU>();                                               \
  extern template int prepare_tiles<T, EPI_DOWN>();
FR_DECLARE_TILES(bf16_t)
FR_DECLARE_TILES(f16_t)
FR_DECLARE_TILES(fp8_t)
#undef FR_DECLARE_TILES

template <int EPI>
int dispatch_dtype(const GemmArgs& a, int dtype, int block, int splits, int64_t sorted_len, hipStream_t st) {
  if (dtype == FR_BF16) return dispatch_block<bf16_t, EPI>(a, block, splits, sorted_len, st);
  if (dtype == FR_F16) return dispatch_block<f16_t, EPI>(a, block, splits, sorted_len, st);
  if (dtype == FR_FP8_E4M3) {
    if (!a.x_scale || !a.w_scale) return fail(FR_E_NULL, "fp8 operands need x_scale and w_scale");
    return dispatch_block<fp8_t, EPI>(a, block, splits, sorted_len, st);
  }
  return fail(FR_E_DTYPE, "dtype %d not in {f16, bf16, fp8_e4m3}", dtype);
}

template <typename T, typename P>
void launch_combine_as(const void* partial, int64_t split_stride, int splits, int topk, int64_t M, int H, void* out,
                       const int32_t* pair_ids, int E, hipStream_t st) {
  // 16-byte loads of the 2-byte rows of a single slice when the row length allows, else 4 elements per thread
  if (sizeof(P) == 2 && H % 8 == 0) {
    const unsigned grid = static_cast<unsigned>(ceil_div(M * H / 8, 256));
    hipLaunchKernelGGL((combine_kernel<T, P, 8>), dim3(grid), dim3(256), 0, st, static_cast<const P*>(partial), split_stride,
                       splits, topk, M, H, static_cast<T*>(out), pair_ids, E);
    return;
  }
  const unsigned grid = static_cast<unsigned>(ceil_div(M * H / 4, 256));
  hipLaunchKernelGGL((combine_kernel<T, P, 4>), dim3(grid), dim3(256), 0, st, static_cast<const P*>(partial), split_stride,
                     splits, topk, M, H, static_cast<T*>(out), pair_ids, E);
}

// partial_dtype: FR_F32, or the 2-byte type a single slice was written in
int launch_combine(const void* partial, int partial_dtype, int64_t split_stride, int splits, int topk, int64_t M, int H,
                   int out_dtype, void* out, const int32_t* pair_ids, int E, hipStream_t st) {
  if (M == 0) return FR_OK;
  if (out_dtype != FR_BF16 && out_dtype != FR_F16) return fail(FR_E_DTYPE, "output dtype %d not in {f16, bf16}", out_dtype);
  const bool ob = out_dtype == FR_BF16;
  if (partial_dtype == FR_F32) {
    if (ob) launch_combine_as<bf16_t, float>(partial, split_stride, splits, topk, M, H, out, pair_ids, E, st);
    else launch_combine_as<f16_t, float>(partial, split_stride, splits, topk, M, H, out, pair_ids, E, st);
  } else if (partial_dtype == FR_BF16) {
    if (ob) launch_combine_as<bf16_t, bf16_t>(partial, split_stride, splits, topk, M, H, out, pair_ids, E, st);
    else launch_combine_as<f16_t, bf16_t>(partial, split_stride, splits, topk, M, H, out, pair_ids, E, st);
  } else if (partial_dtype == FR_F16) {
    if (ob) launch_combine_as<bf16_t, f16_t>(partial, split_stride, splits, topk, M, H, out, pair_ids, E, st);
    else launch_combine_as<f16_t, f16_t>(partial, split_stride, splits, topk, M, H, out, pair_ids, E, st);
  } else {
    return fail(FR_E_DTYPE, "partial dtype %d", partial_dtype);
  }
  return check_launch("combine_kernel");
}

__global__ __launch_bounds__(256) void zero_fill_kernel(u32x4* __restrict__ p, int64_t n16) {
  const u32x4 z = {0u, 0u, 0u, 0u};
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < n16; i += static_cast<int64_t>(gridDim.x) * 256) p[i] = z;
}

// a split whose K range is empty would leave its slice unwritten: shrink until every slice has work
int usable_splits(int split_k, int64_t K, int bk) {
  int splits = split_k;
  while (splits > 1 && round_up(ceil_div(K, splits), bk) * (splits - 1) >= K) --splits;
  return splits;
}

int64_t tail_scratch_bytes(int block, int dtype, int64_t K, int64_t N, bool gateup) {
  // The tiles that run persistently: T256 (both GEMMs for 2-byte operands, the down projection for fp8)
  // and T128P (both GEMMs).  Same K bytes per tile and same feature tile in all of them.
  typedef Tiles<bf16_t>::T256 C;
  static_assert(Tiles<bf16_t>::T256S::BF == C::BF && Tiles<bf16_t>::T256S::BT == C::BT && Tiles<bf16_t>::T128P::BF == C::BF && Tiles<bf16_t>::T128P::BKB == C::BKB, "same K tile and feature tile");
  static_assert(Tiles<fp8_t>::T256::BF == C::BF && Tiles<fp8_t>::T256::BKB == C::BKB, "same K tile and feature tile");
  const bool two_byte = dtype == FR_BF16 || dtype == FR_F16;
  if (!two_byte && dtype != FR_FP8_E4M3) return 0;
  if (!((block == 256 && (two_byte || !gateup)) || block == 128 || block == 160)) return 0;
  const int64_t bk = C::BKB / elem_bytes(dtype), cols = gateup ? C::BF / 2 : C::BF;
  if (K / bk < kTailMinTiles || N % cols != 0) return 0;
  return static_cast<int64_t>(kTailUnits) * C::BT * C::BF * 4;  // sized for the larger tile
}

int gateup_impl(const void* x, const float* x_scale, const void* w1, const float* w1_scale,
                const int32_t* sorted, const int32_t* expert_ids, const int32_t* npost, int64_t M, int64_t H,
                int64_t F, int E, int topk, int block, int dtype, void* act, float* tail_ws, hipStream_t st,
                const char* who, int w_tiled = 0) {
  if (M == 0) return FR_OK;
  FR_REQUIRE(!w_tiled || (F % kTileRows == 0 && (H * elem_bytes(dtype)) % kTileBytes == 0), FR_E_SHAPE,
             "%s: prepared weights need F %% %d == 0 and whole %d-byte K tiles", who, kTileRows, kTileBytes);
  FR_REQUIRE(x && w1 && act && sorted && expert_ids && npost, FR_E_NULL, "%s: null pointer", who);
  FR_REQUIRE(valid_block(block), FR_E_SHAPE, "%s: block=%d not in {16,32,64,128,160,256}", who, block);
  FR_REQUIRE(H > 0 && H % k_multiple(dtype, block) == 0, FR_E_SHAPE, "%s: H=%lld must be a multiple of %d for block %d", who, (long long)H, k_multiple(dtype, block), block);
  FR_REQUIRE(F > 0 && F % 8 == 0, FR_E_SHAPE, "%s: F=%lld must be a positive multiple of 8", who, (long long)F);
  FR_REQUIRE(topk >= 1 && E >= 1 && M * topk < (int64_t(1) << 30), FR_E_SHAPE, "%s: M*topk too large", who);
  FR_REQUIRE(aligned16(x) && aligned16(w1) && aligned16(act) && aligned16(tail_ws), FR_E_ALIGN, "%s: operands must be 16-byte aligned", who);
  const int64_t n = M * topk, sorted_len = n + int64_t(E) * (block - 1);
  GemmArgs a = {};
  a.X = x; a.ldx = H; a.W = w1; a.w_expert_stride = 2 * F * H; a.ldw = H; a.out = act; a.ldo = F;
  a.sorted = sorted; a.expert_ids = expert_ids; a.npost = npost;
  a.x_scale = x_scale; a.w_scale = w1_scale; a.w_rows = static_cast<int>(2 * F);
  a.num_valid = (int)n; a.top_k = topk; a.N = (int)F; a.K = (int)H;
  a.num_experts = E;
  a.tail_ws = tail_ws;
  a.w_tiled = w_tiled;
  // batches the routed form of the row kernel takes run the row kernel here too (same kernel, same sums, whoever
  // did the routing); the row kernels read whole weight rows and take the row-major layout only
  const int64_t min_k = gateup_rows_routes(M, E, topk, block) ? kRowsMinKRouted : kRowsMinK;
  if (!w_tiled && gateup_rows_fits(M, H, block, sorted_len, elem_bytes(dtype), min_k)) {
    // a handful of tokens: stream the weight rows past the token rows without tiles
    if (dtype == FR_BF16) return launch_gateup_rows<bf16_t>(a, block, sorted_len / block * block, st);
    return launch_gateup_rows<f16_t>(a, block, sorted_len / block * block, st);
  }
  return dispatch_dtype<EPI_SILU>(a, dtype, block, 1, sorted_len / block * block, st);
}

int gateup_rows_routed(const void* x, const void* w1, const void* logits, int logits_dtype, int64_t M, int64_t H,
                       int64_t F, int E, int topk, int renorm, int block, int dtype, void* act, float* topk_w,
                       int32_t* topk_ids, int32_t* sorted, int32_t* expert_ids, int32_t* npost, hipStream_t st) {
  const int64_t n = M * topk, sorted_len = n + int64_t(E) * (block - 1);
  if ((dtype != FR_BF16 && dtype != FR_F16) || !gateup_rows_fits(M, H, block, sorted_len, 2, kRowsMinKRouted) ||
      !gateup_rows_routes(M, E, topk, block) || F % 8 != 0 ||
      (logits_dtype != FR_F32 && logits_dtype != FR_F16 && logits_dtype != FR_BF16))
    return 1;
  FR_REQUIRE(x && w1 && logits && act && topk_w && topk_ids && sorted && expert_ids && npost, FR_E_NULL, "gate/up with routing: null pointer");
  FR_REQUIRE(aligned16(x) && aligned16(w1) && aligned16(act), FR_E_ALIGN, "gate/up with routing: operands must be 16-byte aligned");
  GemmArgs a = {};
  a.X = x; a.ldx = H; a.W = w1; a.w_expert_stride = 2 * F * H; a.ldw = H; a.out = act; a.ldo = F;
  a.sorted = sorted; a.expert_ids = expert_ids; a.npost = npost;
  a.w_rows = static_cast<int>(2 * F);
  a.num_valid = (int)n; a.top_k = topk; a.N = (int)F; a.K = (int)H;
  a.num_experts = E;
  const RowsRoute rt = {logits, logits_dtype, E, topk, renorm, topk_w, topk_ids, sorted, expert_ids, npost};
  if (dtype == FR_BF16) return launch_gateup_rows<bf16_t>(a, block, sorted_len / block * block, st, rt);
  return launch_gateup_rows<f16_t>(a, block, sorted_len / block * block, st, rt);
}

int down_impl(const void* act, const float* act_scale, const void* w2, const float* w2_scale,
              const float* topk_weights, const int32_t* sorted, const int32_t* expert_ids, const int32_t* npost,
              int64_t M, int64_t H, int64_t F, int E, int topk, int block, int split_k, int dtype, int out_dtype,
              float* partial, void* out, float* tail_ws, hipStream_t st, const char* who, int w_tiled,
              const int32_t* pair_ids) {
  if (M == 0) return FR_OK;
  FR_REQUIRE(!w_tiled || (H % kTileRows == 0 && (F * elem_bytes(dtype)) % kTileBytes == 0), FR_E_SHAPE,
             "%s: prepared weights need H %% %d == 0 and whole %d-byte K tiles", who, kTileRows, kTileBytes);
  FR_REQUIRE(act && w2 && topk_weights && partial && out && sorted && expert_ids && npost, FR_E_NULL, "%s: null pointer", who);
  FR_REQUIRE(valid_block(block), FR_E_SHAPE, "%s: block=%d not in {16,32,64,128,160,256}", who, block);
  FR_REQUIRE(F > 0 && F % k_multiple(dtype, block) == 0, FR_E_SHAPE, "%s: F=%lld must be a multiple of %d for block %d", who, (long long)F, k_multiple(dtype, block), block);
  FR_REQUIRE(H > 0 && H % 4 == 0, FR_E_SHAPE, "%s: H=%lld must be a positive multiple of 4", who, (long long)H);
  FR_REQUIRE(split_k >= 1 && split_k <= 64, FR_E_SHAPE, "%s: split_k=%d outside [1, 64]", who, split_k);
  FR_REQUIRE(topk >= 1 && E >= 1 && M * topk < (int64_t(1) << 30), FR_E_SHAPE, "%s: M*topk too large", who);
  FR_REQUIRE(aligned16(act) && aligned16(w2) && aligned16(partial) && aligned16(out) && aligned16(tail_ws), FR_E_ALIGN, "%s: operands must be 16-byte aligned", who);
  const int64_t n = M * topk, sorted_len = n + int64_t(E) * (block - 1);
  const int splits = usable_splits(split_k, F, k_multiple(dtype, block));
  GemmArgs a = {};
  a.X = act; a.ldx = F; a.W = w2; a.w_expert_stride = H * F; a.ldw = F; a.out = partial; a.ldo = H;
  a.split_stride = n * H;
  a.sorted = sorted; a.expert_ids = expert_ids; a.npost = npost;
  a.x_scale = act_scale; a.w_scale = w2_scale; a.w_rows = static_cast<int>(H);
  a.topk_w = topk_weights; a.num_valid = (int)n; a.top_k = 0; a.N = (int)H; a.K = (int)F;
  a.mul_weight = 1;
  a.num_experts = E;
  a.tail_ws = tail_ws;
  a.long_k = 1;
  a.w_tiled = w_tiled;
  if (!w_tiled && down_rows_fits(n, F, H, sorted_len, elem_bytes(dtype)) && out_dtype == dtype) {
    // a handful of pairs: weight rows streamed past the activated rows, routed weight and top-k sum in the same kernel
    a.out = out;
    if (dtype == FR_BF16) return launch_down_rows<bf16_t>(a, topk, block, sorted_len, st);
    return launch_down_rows<f16_t>(a, topk, block, sorted_len, st);
  }
  if (splits == 1) {
    const int row_dtype = dtype == FR_F16 ? FR_F16 : FR_BF16;  // type a single slice's rows are written in
    if (tunables().epilogue_combine && topk == 2 && out_dtype == row_dtype) {
      // Two pairs per token, on request (measured slower than the combine kernel): the combine happens in the GEMM epilogue.  `out` is zero-filled (by a kernel: the call
      // stays capturable) and every pair's weighted row is added into its token's row with packed atomics - 0 + a
      // is exact and a + b is rounded once, so the result does not depend on which pair arrives first and equals
      // the sum the combine kernel would form from the same two rounded rows.  No partial rows, no combine launch;
      // a pair whose expert id is out of range has no slot and adds nothing.
      const int64_t n16 = M * H * 2 / 16;  // H % 4 == 0 and 16-byte alignment were checked; M * H * 2 % 16: see below
      if ((M * H) % 8 == 0) {
        hipLaunchKernelGGL(zero_fill_kernel, dim3(static_cast<unsigned>(ceil_div(n16, 256) < 4096 ? ceil_div(n16, 256) : 4096)),
                           dim3(256), 0, st, static_cast<u32x4*>(out), n16);
        int rc = check_launch("zero_fill_kernel");
        if (rc != FR_OK) return rc;
        a.out = out;
        a.add_div = topk;
        return dispatch_dtype<EPI_PLAIN>(a, dtype, block, 1, sorted_len / block * block, st);
      }
    }
    // one slice: each pair's row in the operands' 2-byte type (bf16 for fp8 operands), half the partial traffic
    int rc = dispatch_dtype<EPI_PLAIN>(a, dtype, block, 1, sorted_len / block * block, st);
    if (rc != FR_OK) return rc;
    return launch_combine(partial, row_dtype, n * H, 1, topk, M, (int)H, out_dtype, out, pair_ids, E, st);
  }
  int rc = dispatch_dtype<EPI_DOWN>(a, dtype, block, splits, sorted_len / block * block, st);
  if (rc != FR_OK) return rc;
  return launch_combine(partial, FR_F32, n * H, splits, topk, M, (int)H, out_dtype, out, pair_ids, E, st);
}

// ---- prepared weight layout -----------------------------------------------------------------
// One thread per 16-byte chunk of the OUTPUT (consecutive threads write consecutive memory): chunk o is
// chunk c = o % 8 of row r = (o / 8) % 64 of K tile kt of row group g; its source is chunk kt * 8 + c of row
// g * 64 + r of the row-major matrix (row groups never straddle experts: rows per expert are a multiple of 64).
__global__ __launch_bounds__(256) void tile_weights_kernel(const u32x4* __restrict__ in, u32x4* __restrict__ out,
                                                           int64_t chunks, int64_t ktiles) {
  const int64_t o = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (o >= chunks) return;
  constexpr int CPT = kTileBytes / 16;  // chunks per row and K tile
  const int c = static_cast<int>(o % CPT), r = static_cast<int>((o / CPT) % kTileRows);
  const int64_t piece = o / (CPT * kTileRows), kt = piece % ktiles, g = piece / ktiles;
  out[o] = in[(g * kTileRows + r) * (ktiles * CPT) + kt * CPT + c];
}

}  // namespace fr

using namespace fr;

extern "C" int fr_moe_prepare_weights(const void* w, int dtype, int64_t E, int64_t rows, int64_t K, void* out, void* stream) {
  FR_REQUIRE(dtype == FR_F16 || dtype == FR_BF16 || dtype == FR_FP8_E4M3, FR_E_DTYPE, "fr_moe_prepare_weights: dtype %d not in {f16, bf16, fp8_e4m3}", dtype);
  FR_REQUIRE(w && out, FR_E_NULL, "fr_moe_prepare_weights: null pointer");
  FR_REQUIRE(w != out, FR_E_SHAPE, "fr_moe_prepare_weights: not an in-place transform (out must not be w)");
  const int es = elem_bytes(dtype);
  FR_REQUIRE(E >= 1 && rows > 0 && rows % kTileRows == 0 && K > 0 && (K * es) % kTileBytes == 0, FR_E_SHAPE,
             "fr_moe_prepare_weights: rows=%lld must be a multiple of %d and K=%lld a whole number of %d-byte tiles",
             (long long)rows, kTileRows, (long long)K, kTileBytes);
  FR_REQUIRE(aligned16(w) && aligned16(out), FR_E_ALIGN, "fr_moe_prepare_weights: operands must be 16-byte aligned");
  const int64_t chunks = E * rows * K * es / 16;
  FR_REQUIRE(ceil_div(chunks, 256) < (int64_t(1) << 31), FR_E_SHAPE, "fr_moe_prepare_weights: matrix too large");
  hipLaunchKernelGGL(tile_weights_kernel, dim3(static_cast<unsigned>(ceil_div(chunks, 256))), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const u32x4*>(w), static_cast<u32x4*>(out), chunks, K * es / kTileBytes);
  return check_launch("tile_weights_kernel");
}

extern "C" int fr_moe_grouped_gemm(const void* A, int64_t lda, const void* B, void* C,
                                   const float* topk_weights, const int32_t* sorted_token_ids,
                                   const int32_t* expert_ids, const int32_t* num_tokens_post_pad,
                                   int64_t sorted_len, int64_t num_valid, int64_t N, int64_t K, int E,
                                   int block, int top_k, int mul_routed_weight, int dtype, void* stream) {
  const int w_tiled = (dtype & FR_W_TILED) ? 1 : 0;
  dtype &= ~FR_W_TILED;
  if (num_valid == 0) return FR_OK;
  FR_REQUIRE(A && B && C && sorted_token_ids && expert_ids && num_tokens_post_pad, FR_E_NULL, "fr_moe_grouped_gemm: null pointer");
  FR_REQUIRE(!mul_routed_weight || topk_weights, FR_E_NULL, "fr_moe_grouped_gemm: mul_routed_weight without topk_weights");
  FR_REQUIRE(dtype == FR_F16 || dtype == FR_BF16, FR_E_DTYPE, "fr_moe_grouped_gemm: dtype %d not in {f16, bf16}", dtype);
  FR_REQUIRE(valid_block(block), FR_E_SHAPE, "fr_moe_grouped_gemm: block=%d not in {16,32,64,128,160,256}", block);
  FR_REQUIRE(K > 0 && K % k_multiple(dtype, block) == 0, FR_E_SHAPE, "fr_moe_grouped_gemm: K=%lld must be a positive multiple of %d for block %d", (long long)K, k_multiple(dtype, block), block);
  FR_REQUIRE(N > 0 && N % 4 == 0, FR_E_SHAPE, "fr_moe_grouped_gemm: N=%lld must be a positive multiple of 4", (long long)N);
  FR_REQUIRE(top_k >= 1 && E >= 1, FR_E_SHAPE, "fr_moe_grouped_gemm: top_k=%d E=%d", top_k, E);
  FR_REQUIRE(sorted_len >= block && sorted_len < (int64_t(1) << 31) && num_valid < (int64_t(1) << 31), FR_E_SHAPE, "fr_moe_grouped_gemm: sorted_len=%lld", (long long)sorted_len);
  FR_REQUIRE(lda % 8 == 0 && aligned16(A) && aligned16(B) && aligned16(C), FR_E_ALIGN, "fr_moe_grouped_gemm: operands must be 16-byte aligned, lda %% 8 == 0");
  GemmArgs a = {};
  a.X = A; a.ldx = lda; a.W = B; a.w_expert_stride = N * K; a.ldw = K; a.out = C; a.ldo = N;
  a.sorted = sorted_token_ids; a.expert_ids = expert_ids; a.npost = num_tokens_post_pad;
  a.topk_w = topk_weights; a.num_valid = (int)num_valid; a.top_k = top_k; a.N = (int)N; a.K = (int)K;
  a.mul_weight = mul_routed_weight;
  a.num_experts = E;
  FR_REQUIRE(!w_tiled || (N % kTileRows == 0 && (K * 2) % kTileBytes == 0), FR_E_SHAPE, "fr_moe_grouped_gemm: prepared weights need N %% %d == 0", kTileRows);
  a.w_tiled = w_tiled;
  // only whole blocks inside sorted_token_ids are addressable
  return dispatch_dtype<EPI_PLAIN>(a, dtype, block, 1, sorted_len / block * block, static_cast<hipStream_t>(stream));
}

extern "C" int fr_moe_gateup_silu(const void* x, const void* w1, const int32_t* sorted_token_ids,
                                  const int32_t* expert_ids, const int32_t* num_tokens_post_pad,
                                  int64_t M, int64_t H, int64_t F, int E, int topk, int block, int dtype,
                                  void* act, void* tail_ws, void* stream) {
  const int w_tiled = (dtype & FR_W1_TILED) ? 1 : 0;
  dtype &= ~FR_W_TILED;
  FR_REQUIRE(dtype == FR_F16 || dtype == FR_BF16, FR_E_DTYPE, "fr_moe_gateup_silu: dtype %d not in {f16, bf16}", dtype);
  return gateup_impl(x, nullptr, w1, nullptr, sorted_token_ids, expert_ids, num_tokens_post_pad, M, H, F, E, topk,
                     block, dtype, act, static_cast<float*>(tail_ws), static_cast<hipStream_t>(stream), "fr_moe_gateup_silu", w_tiled);
}

extern "C" int fr_moe_gateup_silu_fp8(const void* xq, const float* x_scale, const void* w1q, const float* w1_scale,
                                      const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                      const int32_t* num_tokens_post_pad, int64_t M, int64_t H, int64_t F, int E,
                                      int topk, int block, void* act_bf16, void* stream) {
  FR_REQUIRE(x_scale && w1_scale, FR_E_NULL, "fr_moe_gateup_silu_fp8: null scale pointer");
  return gateup_impl(xq, x_scale, w1q, w1_scale, sorted_token_ids, expert_ids, num_tokens_post_pad, M, H, F, E, topk,
                     block, FR_FP8_E4M3, act_bf16, nullptr, static_cast<hipStream_t>(stream), "fr_moe_gateup_silu_fp8");
}

extern "C" int fr_moe_down_combine(const void* act, const void* w2, const float* topk_weights,
                                   const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                   const int32_t* num_tokens_post_pad, int64_t M, int64_t H, int64_t F,
                                   int E, int topk, int block, int split_k, int dtype, float* partial,
                                   void* out, void* tail_ws, void* stream) {
  const int w_tiled = (dtype & FR_W2_TILED) ? 1 : 0;
  dtype &= ~FR_W_TILED;
  FR_REQUIRE(dtype == FR_F16 || dtype == FR_BF16, FR_E_DTYPE, "fr_moe_down_combine: dtype %d not in {f16, bf16}", dtype);
  return down_impl(act, nullptr, w2, nullptr, topk_weights, sorted_token_ids, expert_ids, num_tokens_post_pad, M, H, F,
                   E, topk, block, split_k, dtype, dtype, partial, out, static_cast<float*>(tail_ws),
                   static_cast<hipStream_t>(stream), "fr_moe_down_combine", w_tiled, nullptr);
}

extern "C" int fr_moe_down_combine_fp8(const void* actq, const float* act_scale, const void* w2q, const float* w2_scale,
                                       const float* topk_weights, const int32_t* sorted_token_ids,
                                       const int32_t* expert_ids, const int32_t* num_tokens_post_pad, int64_t M,
                                       int64_t H, int64_t F, int E, int topk, int block, int split_k, int out_dtype,
                                       float* partial, void* out, void* tail_ws, void* stream) {
  const int w_tiled = (out_dtype & FR_W2_TILED) ? 1 : 0;
  out_dtype &= ~FR_W_TILED;
  FR_REQUIRE(act_scale && w2_scale, FR_E_NULL, "fr_moe_down_combine_fp8: null scale pointer");
  return down_impl(actq, act_scale, w2q, w2_scale, topk_weights, sorted_token_ids, expert_ids, num_tokens_post_pad, M,
                   H, F, E, topk, block, split_k, FR_FP8_E4M3, out_dtype, partial, out, static_cast<float*>(tail_ws),
                   static_cast<hipStream_t>(stream), "fr_moe_down_combine_fp8", w_tiled, nullptr);
}

// Every kernel the grouped GEMM entry points can launch for `dtype`, set up on the current device.
extern "C" int fr_moe_prepare(int dtype) {
  int rc;
  if (dtype == FR_BF16) {
    rc = prepare_tiles<bf16_t, EPI_PLAIN>();
    if (rc == FR_OK) rc = prepare_tiles<bf16_t, EPI_SILU>();
    if (rc == FR_OK) rc = prepare_tiles<bf16_t, EPI_DOWN>();
  } else if (dtype == FR_F16) {
    rc = prepare_tiles<f16_t, EPI_PLAIN>();
    if (rc == FR_OK) rc = prepare_tiles<f16_t, EPI_SILU>();
    if (rc == FR_OK) rc = prepare_tiles<f16_t, EPI_DOWN>();
  } else if (dtype == FR_FP8_E4M3) {
    rc = prepare_tiles<fp8_t, EPI_PLAIN>();
    if (rc == FR_OK) rc = prepare_tiles<fp8_t, EPI_SILU>();
    if (rc == FR_OK) rc = prepare_tiles<fp8_t, EPI_DOWN>();
  } else {
    return fail(FR_E_DTYPE, "fr_moe_prepare: dtype %d not in {f16, bf16, fp8_e4m3}", dtype);
  }
  if (rc == FR_OK) rc = prepare_static_scratch();  // fr_fused_moe_noalloc then has no set-up left either
  return rc;
}

#ifdef FR_PROF
// measurement builds only: device buffer of 4 x int64 per workgroup the persistent kernels leave their cycle counts in
extern "C" void fr_debug_set_prof(long long* p) { fr::fr_prof_host() = p; }
#endif
