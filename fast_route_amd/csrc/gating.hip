// Top-k gating for router logits on gfx950.
//
// A group of G lanes (G = next power of two >= E, at most one wavefront) owns
// one token; each lane keeps VPL logits in registers (expert = lane + i*G), so
// a wavefront handles 64/G tokens.  Softmax statistics use the online
// (max, sum) recurrence combined across lanes with one butterfly; top-k is k
// rounds of a cross-lane arg-max under the total order (value descending,
// expert index ascending), which is what a stable descending sort yields.
#include "gating_core.h"

namespace fr {
namespace {

template <typename T, int G, int VPL>
__global__ __launch_bounds__(kGateThreads) void gating_topk_kernel(
    const T* __restrict__ logits, int64_t M, int E, int64_t ld, int topk, int renorm,
    float* __restrict__ w_out, int32_t* __restrict__ ids_out) {
  // grid-stride over tokens: a few tokens per lane group amortise wave launch
  constexpr int64_t kPerBlock = kGateThreads / G;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kPerBlock;
  const int64_t rounds = (M + stride - 1) / stride;  // uniform trip count: every lane joins the cross-lane ops
  int64_t token = static_cast<int64_t>(blockIdx.x) * kPerBlock + threadIdx.x / G;
  for (int64_t it = 0; it < rounds; ++it, token += stride) {
    const bool live = token < M;
    const T* row = logits + (live ? token : 0) * ld;
    gate_token<G, VPL>([&](int e) { return to_float(row[e]); }, live, E, topk, renorm,
                       w_out + token * topk, ids_out + token * topk);
  }
}

// 4 consecutive logits as fp32 from a 4-element-aligned address
template <typename T>
__device__ __forceinline__ f32x4 load4_as_float(const T* p) {
  if constexpr (sizeof(T) == 4) {
    return *reinterpret_cast<const f32x4*>(p);
  } else {
    typedef T vec4 __attribute__((ext_vector_type(4)));
    const vec4 t = *reinterpret_cast<const vec4*>(p);
    return f32x4{to_float(t[0]), to_float(t[1]), to_float(t[2]), to_float(t[3])};
  }
}

template <typename T, int G, int NV>
__global__ __launch_bounds__(kGateThreads) void gating_topk_blocked_kernel(
    const T* __restrict__ logits, int64_t M, int E, int64_t ld, int topk, int renorm,
    float* __restrict__ w_out, int32_t* __restrict__ ids_out) {
  constexpr int64_t kPerBlock = kGateThreads / G;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kPerBlock;
  const int64_t rounds = (M + stride - 1) / stride;  // uniform trip count: every lane joins the cross-lane ops
  int64_t token = static_cast<int64_t>(blockIdx.x) * kPerBlock + threadIdx.x / G;
  for (int64_t it = 0; it < rounds; ++it, token += stride) {
    const bool live = token < M;
    const T* row = logits + (live ? token : 0) * ld;
    gate_token_blocked<G, NV>([&](int e0) { return load4_as_float(row + e0); }, live, E, topk, renorm,
                              w_out + token * topk, ids_out + token * topk);
  }
}

// ---- gate-matrix form: logits tile by MFMA, then the same gating -------------
// The token rows [M, H] are the only real traffic (the gate matrix, [H, E] with experts
// contiguous, stays in L2), so the kernel is shaped to stream them: a workgroup of 4
// wavefronts owns 64 tokens (16 per wavefront), or, while there are too few tokens to fill
// the CUs that way, 16 tokens whose K range the 4 wavefronts split and reduce through LDS.
// The gate is taken in chunks of kRgKC rows, each transposed once through registers into
// expert-major LDS rows (two K rows packed per 32-bit store) that the MFMA "A" operand reads
// as 16-byte vectors; token rows come straight from HBM as the "B" operand, fetched for the
// whole chunk before the barrier that publishes it.
constexpr int kRgMaxE = 128;  // the reference's own bound (ops/stable_route.py:134)

template <typename T> struct Mfma16;
template <> struct Mfma16<bf16_t> {
  typedef bf16x8 vec8;
  static __device__ __forceinline__ f32x4 mma(vec8 a, vec8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};
template <> struct Mfma16<f16_t> {
  typedef f16x8 vec8;
  static __device__ __forceinline__ f32x4 mma(vec8 a, vec8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
};

// KC = K rows of the gate per LDS chunk; TT = 16-token tiles per wavefront in the unsplit form (many
// experts: more tokens per transposed gate chunk).
// G lanes gate a token, VPL logits each: up to G * VPL experts (VPL = 2: 65..128 experts).
template <typename T, int G, bool SPLITK, int KC, int TT, int VPL = 1>
__global__ __launch_bounds__(kGateThreads) void route_gate_kernel(
    const T* __restrict__ hidden, const T* __restrict__ gate, int64_t M, int H, int E, int topk,
    int renorm, float* __restrict__ w_out, int32_t* __restrict__ ids_out) {
  typedef typename Mfma16<T>::vec8 vec8;
  static_assert(kGateThreads == 256, "4 wavefronts");
  static_assert(!SPLITK || TT == 1, "the split form has one token tile");
  constexpr int ET = (G * VPL + 15) / 16;        // expert tiles of 16
  constexpr int TPC = SPLITK ? 16 : 64 * TT;     // tokens per workgroup
  constexpr int KW = SPLITK ? KC / 4 : KC;       // K elements of a chunk one wavefront multiplies
  constexpr int KSTEPS = KW / 32;
  constexpr int PITCH = KC + 8;                  // elements; keeps 16-byte alignment, spreads banks
  constexpr int LP = ET * 16 + 1;                // pitch of a logit row (floats)
  // the transposed gate chunk during the K loop; afterwards the same memory holds the logits (and the K slices' partial sums)
  constexpr int GT_BYTES = ET * 16 * PITCH * static_cast<int>(sizeof(T));
  constexpr int LG_BYTES = (TPC * LP + (SPLITK ? 4 * 16 * LP : 0)) * 4;
  __shared__ __attribute__((aligned(16))) unsigned char smem[GT_BYTES > LG_BYTES ? GT_BYTES : LG_BYTES];
  static_assert(sizeof(smem) <= 65536, "LDS");
  T* gt = reinterpret_cast<T*>(smem);
  float* logit = reinterpret_cast<float*>(smem);
  float* part = logit + TPC * LP;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t tok0 = static_cast<int64_t>(blockIdx.x) * TPC;
  const int kw0 = SPLITK ? wave * KW : 0;        // the wavefront's K range inside a chunk
  int trow[TT];                                  // the lane's tokens inside the workgroup
  const T* xrow[TT];
#pragma unroll
  for (int t = 0; t < TT; ++t) {
    trow[t] = (SPLITK ? 0 : (wave * TT + t) * 16) + (lane & 15);
    const int64_t tok = tok0 + trow[t];
    xrow[t] = hidden + (tok < M ? tok : 0) * H + kw0 + (lane >> 4) * 8;
  }

  for (int i = tid; i < ET * 16 * PITCH; i += kGateThreads) gt[i] = static_cast<T>(0.f);  // experts >= E stay 0
  f32x4 acc[TT][ET];
#pragma unroll
  for (int t = 0; t < TT; ++t)
#pragma unroll
    for (int j = 0; j < ET; ++j) acc[t][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  const bool vec_gate = E % 8 == 0 && (reinterpret_cast<uintptr_t>(gate) & 15u) == 0;

  for (int kc = 0; kc < H; kc += KC) {
    vec8 xf[TT][KSTEPS];
#pragma unroll
    for (int t = 0; t < TT; ++t)
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        const int kk = kc + kw0 + ks * 32 + (lane >> 4) * 8;
        if (kk + 8 <= H) xf[t][ks] = *reinterpret_cast<const vec8*>(xrow[t] + kc + ks * 32);
        else
#pragma unroll
          for (int r = 0; r < 8; ++r) xf[t][ks][r] = static_cast<T>(0.f);
      }
    __syncthreads();  // the previous chunk has been read
    if (vec_gate) {
      // item = (pair of K rows, 8 experts): two 16-byte loads, eight 32-bit stores of (k, k+1) pairs
      const int evs = E / 8;
      for (int item = tid; item < (KC / 2) * evs; item += kGateThreads) {
        const int kp = item % (KC / 2), ev = item / (KC / 2);
        const int k = kc + 2 * kp;
        vec8 r0, r1;
#pragma unroll
        for (int r = 0; r < 8; ++r) { r0[r] = static_cast<T>(0.f); r1[r] = static_cast<T>(0.f); }
        if (k < H) r0 = *reinterpret_cast<const vec8*>(gate + static_cast<int64_t>(k) * E + ev * 8);
        if (k + 1 < H) r1 = *reinterpret_cast<const vec8*>(gate + static_cast<int64_t>(k + 1) * E + ev * 8);
#pragma unroll
        for (int r = 0; r < 8; ++r) {
          typedef T pair_t __attribute__((ext_vector_type(2)));
          const pair_t pr = {r0[r], r1[r]};
          *reinterpret_cast<pair_t*>(&gt[(ev * 8 + r) * PITCH + 2 * kp]) = pr;
        }
      }
    } else {
      for (int i = tid; i < KC * E; i += kGateThreads) {
        const int k = i / E, e = i % E;
        gt[e * PITCH + k] = kc + k < H ? gate[static_cast<int64_t>(kc + k) * E + e] : static_cast<T>(0.f);
      }
    }
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks)
#pragma unroll
      for (int j = 0; j < ET; ++j) {
        const vec8 gf = *reinterpret_cast<const vec8*>(&gt[(j * 16 + (lane & 15)) * PITCH + kw0 + ks * 32 + (lane >> 4) * 8]);
#pragma unroll
        for (int t = 0; t < TT; ++t) acc[t][j] = Mfma16<T>::mma(gf, xf[t][ks], acc[t][j]);
      }
  }
  __syncthreads();  // every wavefront has read its last gate chunk: the memory becomes the logit rows
  // accumulator rows are experts (lane/16*4 + r inside tile j), columns tokens
  float* dst = SPLITK ? part + wave * 16 * LP : logit;
#pragma unroll
  for (int t = 0; t < TT; ++t)
#pragma unroll
    for (int j = 0; j < ET; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) dst[trow[t] * LP + j * 16 + (lane >> 4) * 4 + r] = acc[t][j][r];
  __syncthreads();
  if constexpr (SPLITK) {
    for (int i = tid; i < 16 * ET * 16; i += kGateThreads) {
      const int t = i / (ET * 16), e = i % (ET * 16);
      logit[t * LP + e] = (part[t * LP + e] + part[(16 + t) * LP + e]) + (part[(32 + t) * LP + e] + part[(48 + t) * LP + e]);
    }
    __syncthreads();
  }
  constexpr int PER_PASS = kGateThreads / G;
  for (int t = tid / G; t < TPC; t += PER_PASS) {
    const int64_t token = tok0 + t;
    const bool live = token < M;
    const float* row = logit + t * LP;
    gate_token<G, VPL>([&](int e) { return row[e]; }, live, E, topk, renorm, w_out + token * topk,
                       ids_out + token * topk);
  }
}

template <typename T, int G, int VPL>
void launch(const void* logits, int64_t M, int E, int64_t ld, int topk, int renorm, float* w,
            int32_t* ids, hipStream_t st) {
  const int64_t tokens_per_block = kGateThreads / G;
  int64_t blocks = ceil_div(M, tokens_per_block);
  if (blocks > 4096) blocks = 4096;  // 16 workgroups per CU; the rest is the in-kernel token loop
  const unsigned grid = static_cast<unsigned>(blocks);
  hipLaunchKernelGGL((gating_topk_kernel<T, G, VPL>), dim3(grid), dim3(kGateThreads), 0, st,
                     static_cast<const T*>(logits), M, E, ld, topk, renorm, w, ids);
}

template <typename T, int G, int NV>
void launch_blocked(const void* logits, int64_t M, int E, int64_t ld, int topk, int renorm, float* w,
                    int32_t* ids, hipStream_t st) {
  const int64_t tokens_per_block = kGateThreads / G;
  int64_t blocks = ceil_div(M, tokens_per_block);
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL((gating_topk_blocked_kernel<T, G, NV>), dim3(static_cast<unsigned>(blocks)), dim3(kGateThreads), 0,
                     st, static_cast<const T*>(logits), M, E, ld, topk, renorm, w, ids);
}

template <typename T>
int dispatch(const void* logits, int64_t M, int E, int64_t ld, int topk, int renorm, float* w,
             int32_t* ids, hipStream_t st) {
  // many experts, rows that 4-element vector loads can read: few lanes per token
  const bool vec_ok = E > 16 && E % 4 == 0 && ld % 4 == 0 &&
                      (reinterpret_cast<uintptr_t>(logits) % (4 * sizeof(T))) == 0;
  const int lanes = E <= 64 ? 4 : (E <= 128 ? 8 : 16);
  // (a short batch is latency bound: one logit per lane finishes a token in fewer dependent steps)
  if (vec_ok && M >= 1024 && topk <= kBlockedSlots * lanes) {
    if (E <= 32) launch_blocked<T, 4, 2>(logits, M, E, ld, topk, renorm, w, ids, st);
    else if (E <= 64) launch_blocked<T, 4, 4>(logits, M, E, ld, topk, renorm, w, ids, st);
    else if (E <= 128) launch_blocked<T, 8, 4>(logits, M, E, ld, topk, renorm, w, ids, st);
    else launch_blocked<T, 16, 4>(logits, M, E, ld, topk, renorm, w, ids, st);
    return check_launch("gating_topk_blocked_kernel");
  }
  if (E <= 1) launch<T, 1, 1>(logits, M, E, ld, topk, renorm, w, ids, st);
  else if (E <= 2) launch<T, 2, 1>(logits, M, E, ld, topk, renorm, w, ids, st);
  else if (E <= 4) launch<T, 4, 1>(logits, M, E, ld, topk, renorm, w, ids, st);
  else if (E <= 8) launch<T, 8, 1>(logits, M, E, ld, topk, renorm, w, ids, st);
  else if (E <= 16) launch<T, 16, 1>(logits, M, E, ld, topk, renorm, w, ids, st);
  else if (E <= 32) launch<T, 32, 1>(logits, M, E, ld, topk, renorm, w, ids, st);
  else if (E <= 64) launch<T, 64, 1>(logits, M, E, ld, topk, renorm, w, ids, st);
  else if (E <= 128) launch<T, 64, 2>(logits, M, E, ld, topk, renorm, w, ids, st);
  else launch<T, 64, 4>(logits, M, E, ld, topk, renorm, w, ids, st);
  return check_launch("gating_topk_kernel");
}

}  // namespace
}  // namespace fr

extern "C" int fr_gating_topk(const void* logits, int logits_dtype, int64_t M, int64_t E,
                              int64_t ld, int topk, int renormalize, float* weights_out,
                              int32_t* ids_out, void* stream) {
  using namespace fr;
  FR_REQUIRE(M >= 0, FR_E_SHAPE, "fr_gating_topk: M=%lld < 0", (long long)M);
  if (M == 0) return FR_OK;
  FR_REQUIRE(logits && weights_out && ids_out, FR_E_NULL, "fr_gating_topk: null pointer");
  FR_REQUIRE(E >= 1 && E <= 256, FR_E_SHAPE, "fr_gating_topk: E=%lld outside [1, 256]", (long long)E);
  FR_REQUIRE(topk >= 1 && topk <= E, FR_E_SHAPE, "fr_gating_topk: topk=%d outside [1, E=%lld]", topk, (long long)E);
  FR_REQUIRE(ld >= E, FR_E_SHAPE, "fr_gating_topk: row stride %lld < E", (long long)ld);
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (logits_dtype) {
    case FR_F32: return dispatch<float>(logits, M, (int)E, ld, topk, renormalize, weights_out, ids_out, st);
    case FR_F16: return dispatch<f16_t>(logits, M, (int)E, ld, topk, renormalize, weights_out, ids_out, st);
    case FR_BF16: return dispatch<bf16_t>(logits, M, (int)E, ld, topk, renormalize, weights_out, ids_out, st);
    default: return fail(FR_E_DTYPE, "fr_gating_topk: logits dtype %d not in {f16, bf16, f32}", logits_dtype);
  }
}

namespace fr {
namespace {
template <typename T, int G, int VPL = 1>
void launch_route_gate(const void* hidden, const void* gate, int64_t M, int H, int E, int topk, int renorm,
                       float* w, int32_t* ids, hipStream_t st) {
  constexpr int ET = (G * VPL + 15) / 16;
  // 64 (128 with many experts) tokens per workgroup once that gives every CU a workgroup or two; below,
  // 16 tokens with K split over the wavefronts (more workgroups, a quarter of the row per wavefront)
  if (M >= 16384) {
    constexpr int TT = (ET >= 2 && VPL == 1) ? 2 : 1;
    constexpr int KCU = VPL == 1 ? 256 : 128;  // 128 expert rows of 256 K elements would not fit the LDS
    hipLaunchKernelGGL((route_gate_kernel<T, G, false, KCU, TT, VPL>), dim3(static_cast<unsigned>(ceil_div(M, 64 * TT))), dim3(kGateThreads),
                       0, st, static_cast<const T*>(hidden), static_cast<const T*>(gate), M, H, E, topk, renorm, w, ids);
  } else {
    constexpr int KC = VPL == 1 ? 256 : 128;  // longer chunks for few experts leave fewer workgroups per CU: slower at M = 8192, no gain at M = 1
    hipLaunchKernelGGL((route_gate_kernel<T, G, true, KC, 1, VPL>), dim3(static_cast<unsigned>(ceil_div(M, 16))), dim3(kGateThreads), 0, st,
                       static_cast<const T*>(hidden), static_cast<const T*>(gate), M, H, E, topk, renorm, w, ids);
  }
}
template <typename T>
int dispatch_route_gate(const void* hidden, const void* gate, int64_t M, int H, int E, int topk, int renorm,
                        float* w, int32_t* ids, hipStream_t st) {
  if (E <= 1) launch_route_gate<T, 1>(hidden, gate, M, H, E, topk, renorm, w, ids, st);
  else if (E <= 2) launch_route_gate<T, 2>(hidden, gate, M, H, E, topk, renorm, w, ids, st);
  else if (E <= 4) launch_route_gate<T, 4>(hidden, gate, M, H, E, topk, renorm, w, ids, st);
  else if (E <= 8) launch_route_gate<T, 8>(hidden, gate, M, H, E, topk, renorm, w, ids, st);
  else if (E <= 16) launch_route_gate<T, 16>(hidden, gate, M, H, E, topk, renorm, w, ids, st);
  else if (E <= 32) launch_route_gate<T, 32>(hidden, gate, M, H, E, topk, renorm, w, ids, st);
  else if (E <= 64) launch_route_gate<T, 64>(hidden, gate, M, H, E, topk, renorm, w, ids, st);
  else launch_route_gate<T, 64, 2>(hidden, gate, M, H, E, topk, renorm, w, ids, st);
  return check_launch("route_gate_kernel");
}
}  // namespace
}  // namespace fr

extern "C" int fr_route_gate(const void* hidden, const void* gate, int dtype, int64_t M, int64_t H, int64_t E,
                             int topk, int renormalize, float* weights_out, int32_t* ids_out, void* stream) {
  using namespace fr;
  FR_REQUIRE(M >= 0, FR_E_SHAPE, "fr_route_gate: M=%lld < 0", (long long)M);
  if (M == 0) return FR_OK;
  FR_REQUIRE(hidden && gate && weights_out && ids_out, FR_E_NULL, "fr_route_gate: null pointer");
  FR_REQUIRE(E >= 1 && E <= kRgMaxE, FR_E_SHAPE, "fr_route_gate: E=%lld outside [1, %d]", (long long)E, kRgMaxE);
  FR_REQUIRE(topk >= 1 && topk <= E, FR_E_SHAPE, "fr_route_gate: topk=%d outside [1, E=%lld]", topk, (long long)E);
  FR_REQUIRE(H >= 8 && H % 8 == 0 && H < (int64_t(1) << 30), FR_E_SHAPE, "fr_route_gate: H=%lld must be a multiple of 8", (long long)H);
  FR_REQUIRE(aligned16(hidden), FR_E_ALIGN, "fr_route_gate: hidden must be 16-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == FR_BF16) return dispatch_route_gate<bf16_t>(hidden, gate, M, (int)H, (int)E, topk, renormalize, weights_out, ids_out, st);
  if (dtype == FR_F16) return dispatch_route_gate<f16_t>(hidden, gate, M, (int)H, (int)E, topk, renormalize, weights_out, ids_out, st);
  return fail(FR_E_DTYPE, "fr_route_gate: dtype %d not in {f16, bf16}", dtype);
}
