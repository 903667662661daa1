// Host side of the grouped expert GEMMs: tile selection, launches, top-k combine.
#include "moe_gemm_kernel.h"

namespace fr {

// ---- top-k combine: out[m] = sum over splits and slots of partial ------------
template <typename T>
__global__ __launch_bounds__(256) void combine_kernel(const float* __restrict__ partial,
                                                      int64_t split_stride, int splits, int topk,
                                                      int64_t M, int H, T* __restrict__ out) {
  const int64_t idx = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 4;
  if (idx >= M * H) return;
  const int64_t m = idx / H;
  const int h = static_cast<int>(idx % H);
  f32x4 s = {0.f, 0.f, 0.f, 0.f};
  for (int j = 0; j < topk; ++j)
    for (int sp = 0; sp < splits; ++sp) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(partial + sp * split_stride + (m * topk + j) * H + h);
      s += v;
    }
  typename Mfma<T>::vec4 o;
#pragma unroll
  for (int r = 0; r < 4; ++r) o[r] = static_cast<T>(s[r]);
  *reinterpret_cast<typename Mfma<T>::vec4*>(out + idx) = o;
}

// ---- host side ----------------------------------------------------------------
// Token-block sizes and their tile shapes.
//   256 / 128 rows: 8 wavefronts, 32x32x16 MFMA, tiles streamed HBM -> LDS directly
//                   through a 2- or 3-slot ring (compute-bound regime);
//   64 rows:        8 wavefronts, register-staged double buffer;
//   32 / 16 rows:   decode regime, 4 wavefronts side by side along the features,
//                   16x16x32 MFMA, up to 4 workgroups per CU to keep weight bytes in flight.
typedef Cfg<256, 256, 64, 4, 2, 32, 1, 2> CfgT256;
typedef Cfg<128, 256, 64, 2, 4, 32, 1, 3> CfgT128;
typedef Cfg<64, 256, 64, 2, 4, 32, 1, 0> CfgT64;
typedef Cfg<32, 128, 64, 1, 4, 16, 4, 0> CfgT32;
typedef Cfg<16, 128, 64, 1, 4, 16, 4, 0> CfgT16;
constexpr int kGemmKMultiple = 64;  // every configuration uses BK = 64

bool valid_block(int block) { return block == 16 || block == 32 || block == 64 || block == 128 || block == 256; }

template <typename T, int EPI>
int dispatch_block(GemmArgs a, int block, int splits, int64_t sorted_len, hipStream_t st) {
  auto fill = [&](int BT, int BF, int BK) {
    a.num_t_blocks = static_cast<int>(ceil_div(sorted_len, BT));
    const int fper = (EPI == EPI_SILU) ? BF / 2 : BF;
    a.num_f_tiles = static_cast<int>(ceil_div(a.N, fper));
    a.group_t = BT >= 64 ? 4 : 8;
    a.k_per_split = static_cast<int>(round_up(ceil_div(a.K, splits), BK));
  };
  switch (block) {
    case 256: fill(256, 256, 64); return launch_gemm<T, CfgT256, EPI>(a, splits, st);
    case 128: fill(128, 256, 64); return launch_gemm<T, CfgT128, EPI>(a, splits, st);
    case 64: fill(64, 256, 64); return launch_gemm<T, CfgT64, EPI>(a, splits, st);
    case 32: fill(32, 128, 64); return launch_gemm<T, CfgT32, EPI>(a, splits, st);
    case 16: fill(16, 128, 64); return launch_gemm<T, CfgT16, EPI>(a, splits, st);
    default: return fail(FR_E_SHAPE, "routing block %d not in {16, 32, 64, 128, 256}", block);
  }
}

int k_multiple_for_block(int) { return kGemmKMultiple; }

template <int EPI>
int dispatch_dtype(const GemmArgs& a, int dtype, int block, int splits, int64_t sorted_len, hipStream_t st) {
  if (dtype == FR_BF16) return dispatch_block<bf16_t, EPI>(a, block, splits, sorted_len, st);
  if (dtype == FR_F16) return dispatch_block<f16_t, EPI>(a, block, splits, sorted_len, st);
  return fail(FR_E_DTYPE, "dtype %d not in {f16, bf16}", dtype);
}

int launch_combine(const float* partial, int64_t split_stride, int splits, int topk, int64_t M, int H,
                   int dtype, void* out, hipStream_t st) {
  if (M == 0) return FR_OK;
  const unsigned grid = static_cast<unsigned>(ceil_div(M * H / 4, 256));
  if (dtype == FR_BF16)
    hipLaunchKernelGGL(combine_kernel<bf16_t>, dim3(grid), dim3(256), 0, st, partial, split_stride, splits, topk, M, H, static_cast<bf16_t*>(out));
  else
    hipLaunchKernelGGL(combine_kernel<f16_t>, dim3(grid), dim3(256), 0, st, partial, split_stride, splits, topk, M, H, static_cast<f16_t*>(out));
  return check_launch("combine_kernel");
}

}  // namespace fr

using namespace fr;

extern "C" int fr_moe_grouped_gemm(const void* A, int64_t lda, const void* B, void* C,
                                   const float* topk_weights, const int32_t* sorted_token_ids,
                                   const int32_t* expert_ids, const int32_t* num_tokens_post_pad,
                                   int64_t sorted_len, int64_t num_valid, int64_t N, int64_t K, int E,
                                   int block, int top_k, int mul_routed_weight, int dtype, void* stream) {
  if (num_valid == 0) return FR_OK;
  FR_REQUIRE(A && B && C && sorted_token_ids && expert_ids && num_tokens_post_pad, FR_E_NULL, "fr_moe_grouped_gemm: null pointer");
  FR_REQUIRE(!mul_routed_weight || topk_weights, FR_E_NULL, "fr_moe_grouped_gemm: mul_routed_weight without topk_weights");
  FR_REQUIRE(valid_block(block), FR_E_SHAPE, "fr_moe_grouped_gemm: block=%d not in {16,32,64,128,256}", block);
  FR_REQUIRE(K > 0 && K % k_multiple_for_block(block) == 0, FR_E_SHAPE, "fr_moe_grouped_gemm: K=%lld must be a positive multiple of %d for block %d", (long long)K, k_multiple_for_block(block), block);
  FR_REQUIRE(N > 0 && N % 4 == 0, FR_E_SHAPE, "fr_moe_grouped_gemm: N=%lld must be a positive multiple of 4", (long long)N);
  FR_REQUIRE(top_k >= 1 && E >= 1, FR_E_SHAPE, "fr_moe_grouped_gemm: top_k=%d E=%d", top_k, E);
  FR_REQUIRE(sorted_len >= block && sorted_len < (int64_t(1) << 31) && num_valid < (int64_t(1) << 31), FR_E_SHAPE, "fr_moe_grouped_gemm: sorted_len=%lld", (long long)sorted_len);
  FR_REQUIRE(lda % 8 == 0 && aligned16(A) && aligned16(B) && aligned16(C), FR_E_ALIGN, "fr_moe_grouped_gemm: operands must be 16-byte aligned, lda %% 8 == 0");
  GemmArgs a = {};
  a.X = A; a.ldx = lda; a.W = B; a.w_expert_stride = N * K; a.ldw = K; a.out = C; a.ldo = N;
  a.sorted = sorted_token_ids; a.expert_ids = expert_ids; a.npost = num_tokens_post_pad;
  a.topk_w = topk_weights; a.num_valid = (int)num_valid; a.top_k = top_k; a.N = (int)N; a.K = (int)K;
  a.mul_weight = mul_routed_weight;
  // only whole blocks inside sorted_token_ids are addressable
  return dispatch_dtype<EPI_PLAIN>(a, dtype, block, 1, sorted_len / block * block, static_cast<hipStream_t>(stream));
}

extern "C" int fr_moe_gateup_silu(const void* x, const void* w1, const int32_t* sorted_token_ids,
                                  const int32_t* expert_ids, const int32_t* num_tokens_post_pad,
                                  int64_t M, int64_t H, int64_t F, int E, int topk, int block, int dtype,
                                  void* act, void* stream) {
  if (M == 0) return FR_OK;
  FR_REQUIRE(x && w1 && act && sorted_token_ids && expert_ids && num_tokens_post_pad, FR_E_NULL, "fr_moe_gateup_silu: null pointer");
  FR_REQUIRE(valid_block(block), FR_E_SHAPE, "fr_moe_gateup_silu: block=%d not in {16,32,64,128,256}", block);
  FR_REQUIRE(H > 0 && H % k_multiple_for_block(block) == 0, FR_E_SHAPE, "fr_moe_gateup_silu: H=%lld must be a multiple of %d for block %d", (long long)H, k_multiple_for_block(block), block);
  FR_REQUIRE(F > 0 && F % 8 == 0, FR_E_SHAPE, "fr_moe_gateup_silu: F=%lld must be a positive multiple of 8", (long long)F);
  FR_REQUIRE(topk >= 1 && E >= 1 && M * topk < (int64_t(1) << 30), FR_E_SHAPE, "fr_moe_gateup_silu: M*topk too large");
  FR_REQUIRE(aligned16(x) && aligned16(w1) && aligned16(act), FR_E_ALIGN, "fr_moe_gateup_silu: operands must be 16-byte aligned");
  const int64_t n = M * topk, sorted_len = n + int64_t(E) * (block - 1);
  GemmArgs a = {};
  a.X = x; a.ldx = H; a.W = w1; a.w_expert_stride = 2 * F * H; a.ldw = H; a.out = act; a.ldo = F;
  a.sorted = sorted_token_ids; a.expert_ids = expert_ids; a.npost = num_tokens_post_pad;
  a.num_valid = (int)n; a.top_k = topk; a.N = (int)F; a.K = (int)H;
  return dispatch_dtype<EPI_SILU>(a, dtype, block, 1, sorted_len / block * block, static_cast<hipStream_t>(stream));
}

extern "C" int fr_moe_down_combine(const void* act, const void* w2, const float* topk_weights,
                                   const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                   const int32_t* num_tokens_post_pad, int64_t M, int64_t H, int64_t F,
                                   int E, int topk, int block, int split_k, int dtype, float* partial,
                                   void* out, void* stream) {
  if (M == 0) return FR_OK;
  FR_REQUIRE(act && w2 && topk_weights && partial && out && sorted_token_ids && expert_ids && num_tokens_post_pad, FR_E_NULL, "fr_moe_down_combine: null pointer");
  FR_REQUIRE(valid_block(block), FR_E_SHAPE, "fr_moe_down_combine: block=%d not in {16,32,64,128,256}", block);
  FR_REQUIRE(F > 0 && F % k_multiple_for_block(block) == 0, FR_E_SHAPE, "fr_moe_down_combine: F=%lld must be a multiple of %d for block %d", (long long)F, k_multiple_for_block(block), block);
  FR_REQUIRE(H > 0 && H % 4 == 0, FR_E_SHAPE, "fr_moe_down_combine: H=%lld must be a positive multiple of 4", (long long)H);
  FR_REQUIRE(split_k >= 1 && split_k <= 64, FR_E_SHAPE, "fr_moe_down_combine: split_k=%d outside [1, 64]", split_k);
  FR_REQUIRE(topk >= 1 && E >= 1 && M * topk < (int64_t(1) << 30), FR_E_SHAPE, "fr_moe_down_combine: M*topk too large");
  FR_REQUIRE(aligned16(act) && aligned16(w2) && aligned16(partial) && aligned16(out), FR_E_ALIGN, "fr_moe_down_combine: operands must be 16-byte aligned");
  const int64_t n = M * topk, sorted_len = n + int64_t(E) * (block - 1);
  hipStream_t st = static_cast<hipStream_t>(stream);
  // a split whose K range is empty would leave its slice unwritten: shrink split_k so every slice gets work
  const int bk = k_multiple_for_block(block);
  int splits = split_k;
  while (splits > 1 && round_up(ceil_div(F, splits), bk) * (splits - 1) >= F) --splits;
  GemmArgs a = {};
  a.X = act; a.ldx = F; a.W = w2; a.w_expert_stride = H * F; a.ldw = F; a.out = partial; a.ldo = H;
  a.split_stride = n * H;
  a.sorted = sorted_token_ids; a.expert_ids = expert_ids; a.npost = num_tokens_post_pad;
  a.topk_w = topk_weights; a.num_valid = (int)n; a.top_k = 0; a.N = (int)H; a.K = (int)F;
  a.mul_weight = 1;
  int rc = dispatch_dtype<EPI_DOWN>(a, dtype, block, splits, sorted_len / block * block, st);
  if (rc != FR_OK) return rc;
  return launch_combine(partial, n * H, splits, topk, M, (int)H, dtype, out, st);
}
