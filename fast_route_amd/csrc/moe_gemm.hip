// Grouped expert GEMMs on gfx950 MFMA.
//
// One workgroup computes a tile of BT sorted slots (one routing block, hence
// one expert) by BF output features.  Both operands are K-contiguous in HBM
// (tokens [*, K], weights [E, N, K]); tiles of BK are staged through LDS in
// 16-byte chunks under an XOR swizzle and fed to v_mfma with the WEIGHT rows as
// the MFMA "A" operand and the TOKEN rows as "B", so a lane's accumulator
// registers hold 4 consecutive output features of one token and the epilogue
// stores 8/16-byte vectors.  Three epilogues:
//   EPI_PLAIN  C[pair] = acc (* routed weight), scattered by sorted id
//   EPI_SILU   W tile = BF/2 gate rows + the matching BF/2 up rows; writes
//              silu(gate)*up at the slot's own row of act[sorted_len, F]
//   EPI_DOWN   partial[split][pair] = acc * routed weight in fp32 (split-K slices)
// Workgroup ids are first regrouped so that each XCD (ids congruent mod 8) gets
// a contiguous range of tiles, then walked in groups of GROUP_T token blocks x
// all feature tiles so co-resident workgroups share weight tiles in their L2.
#include "fr_common.h"

#include <type_traits>

namespace fr {

enum { EPI_PLAIN = 0, EPI_SILU = 1, EPI_DOWN = 2 };

struct GemmArgs {
  const void* X;        // token rows [*, K]
  int64_t ldx;          // row stride of X in elements
  const void* W;        // [E, w_rows, K]
  int64_t w_expert_stride;
  void* out;
  int64_t ldo;          // row stride of out in elements
  int64_t split_stride; // EPI_DOWN: elements between split-K slices
  const int32_t* sorted;
  const int32_t* expert_ids;
  const int32_t* npost;
  const float* topk_w;  // flat [num_valid] or nullptr
  int num_valid;        // n = M*topk
  int top_k;            // X row = sorted id / top_k; 0 => X row = slot index
  int N;                // output features (EPI_SILU: F, W has 2F rows)
  int K;
  int k_per_split;      // multiple of BK
  int num_t_blocks;     // upper bound on routing blocks
  int num_f_tiles;
  int group_t;
  int mul_weight;
};

template <typename T> struct Mfma;
template <> struct Mfma<bf16_t> {
  typedef bf16x8 vec8;
  typedef bf16x4 vec4;
  static __device__ __forceinline__ f32x16 m32(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 m16(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma<f16_t> {
  typedef f16x8 vec8;
  typedef f16x4 vec4;
  static __device__ __forceinline__ f32x16 m32(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 m16(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

__device__ __forceinline__ float silu(float g) { return g / (1.f + __expf(-g)); }

// Tile configuration.  TILE = 32 uses v_mfma_f32_32x32x16, TILE = 16 v_mfma_f32_16x16x32.
template <int BT_, int BF_, int BK_, int WT_, int WF_, int TILE_>
struct Cfg {
  static constexpr int BT = BT_, BF = BF_, BK = BK_, WT = WT_, WF = WF_, TILE = TILE_;
  static constexpr int NT = WT * WF * kWave;       // threads
  static constexpr int TT = BT / WT, TF = BF / WF; // per-wave tile
  static constexpr int IT = TT / TILE, JF = TF / TILE;
  static constexpr int CPR = BK / 8;               // 16-byte chunks per row
  static constexpr int KSTEP = (TILE == 32) ? 16 : 32;
  static constexpr int KGROUPS = 64 / TILE;        // lane groups along K in one MFMA
  static constexpr int XCH = BT * CPR, WCH = BF * CPR;
  static constexpr int XL = (XCH + NT - 1) / NT, WL = (WCH + NT - 1) / NT;
  static constexpr int LDS_BYTES = 2 * (BT + BF) * BK * 2;
  static_assert(TT % TILE == 0 && TF % TILE == 0, "wave tile must be a multiple of the MFMA tile");
  static_assert(NT % CPR == 0, "threads must cover whole rows");
  static_assert(BK % KSTEP == 0, "BK must be a multiple of the MFMA K");
};

template <int CPR>
__device__ __forceinline__ int swizzle(int row, int chunk) {
  if constexpr (CPR >= 8) return chunk ^ (row & (CPR - 1) & 7) ^ 0;
  else return chunk ^ ((row >> 1) & (CPR - 1));
}

template <typename T, typename C, int EPI>
__global__ __launch_bounds__(C::NT) void moe_gemm_kernel(const GemmArgs a) {
  typedef typename Mfma<T>::vec8 vec8;
  typedef typename std::conditional<C::TILE == 32, f32x16, f32x4>::type acc_t;
  constexpr int BT = C::BT, BF = C::BF, BK = C::BK, CPR = C::CPR, NT = C::NT;
  constexpr int ACC_N = (C::TILE == 32) ? 16 : 4;
  static_assert(EPI != EPI_SILU || C::JF % 2 == 0, "gate and up tiles must pair up inside a wave");

  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  uint4* lds = reinterpret_cast<uint4*>(lds_raw);
  // buffer b: X tile at b*(XCH+WCH), W tile right after it
  constexpr int BUF = C::XCH + C::WCH;

  // ---- tile coordinates ---------------------------------------------------
  const int total = gridDim.x;
  int lin;
  {
    const int pid = blockIdx.x, xcd = pid & 7, idx = pid >> 3;
    const int per = total >> 3, rem = total & 7;
    lin = xcd * per + (xcd < rem ? xcd : rem) + idx;
  }
  const int in_group = a.group_t * a.num_f_tiles;
  const int group_id = lin / in_group;
  const int first_t = group_id * a.group_t;
  const int gsz = min(a.num_t_blocks - first_t, a.group_t);
  const int pid_t = first_t + (lin % in_group) % gsz;
  const int pid_f = (lin % in_group) / gsz;
  const int npost = a.npost[0];
  if (pid_t * BT >= npost) return;
  const int expert = a.expert_ids[pid_t];
  const int split = blockIdx.y;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wt = wave / C::WF, wf = wave % C::WF;

  // ---- global source pointers for this thread's chunks ----------------------
  const T* X = static_cast<const T*>(a.X);
  const T* W = static_cast<const T*>(a.W) + static_cast<int64_t>(expert) * a.w_expert_stride;
  const int k0 = split * a.k_per_split;
  const int k_tiles = min(a.k_per_split, a.K - k0) / BK;
  const int chunk = tid % CPR;
  const int row0 = tid / CPR;
  constexpr int ROWS_PER_PASS = NT / CPR;

  const T* xsrc[C::XL];
  int xdst[C::XL];
#pragma unroll
  for (int i = 0; i < C::XL; ++i) {
    const int r = row0 + i * ROWS_PER_PASS;
    const int rr = r < BT ? r : BT - 1;
    int64_t src_row;
    if (a.top_k > 0) {
      const int sid = a.sorted[pid_t * BT + rr];
      src_row = sid < a.num_valid ? sid / a.top_k : 0;
    } else {
      src_row = static_cast<int64_t>(pid_t) * BT + rr;
    }
    xsrc[i] = X + src_row * a.ldx + k0 + chunk * 8;
    xdst[i] = rr * CPR + swizzle<CPR>(rr, chunk);
  }
  const T* wsrc[C::WL];
  int wdst[C::WL];
#pragma unroll
  for (int i = 0; i < C::WL; ++i) {
    const int r = row0 + i * ROWS_PER_PASS;
    const int rr = r < BF ? r : BF - 1;
    int wrow;
    if constexpr (EPI == EPI_SILU) {
      const int half = rr / (BF / 2), f = pid_f * (BF / 2) + rr % (BF / 2);
      wrow = half * a.N + (f < a.N ? f : a.N - 1);
    } else {
      const int f = pid_f * BF + rr;
      wrow = f < a.N ? f : a.N - 1;
    }
    wsrc[i] = W + static_cast<int64_t>(wrow) * a.K + k0 + chunk * 8;
    wdst[i] = C::XCH + rr * CPR + swizzle<CPR>(rr, chunk);
  }

  uint4 xreg[C::XL], wreg[C::WL];
  auto load_tile = [&](int kt) {
#pragma unroll
    for (int i = 0; i < C::XL; ++i)
      if (C::XCH % NT == 0 || row0 + i * ROWS_PER_PASS < BT)
        xreg[i] = *reinterpret_cast<const uint4*>(xsrc[i] + kt * BK);
#pragma unroll
    for (int i = 0; i < C::WL; ++i)
      if (C::WCH % NT == 0 || row0 + i * ROWS_PER_PASS < BF)
        wreg[i] = *reinterpret_cast<const uint4*>(wsrc[i] + kt * BK);
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int i = 0; i < C::XL; ++i)
      if (C::XCH % NT == 0 || row0 + i * ROWS_PER_PASS < BT) lds[buf * BUF + xdst[i]] = xreg[i];
#pragma unroll
    for (int i = 0; i < C::WL; ++i)
      if (C::WCH % NT == 0 || row0 + i * ROWS_PER_PASS < BF) lds[buf * BUF + wdst[i]] = wreg[i];
  };

  // ---- per-lane fragment rows ---------------------------------------------
  const int frow = lane % C::TILE;  // row inside an MFMA tile
  const int kgrp = lane / C::TILE;  // which 8-element K group of the MFMA this lane feeds
  int xrow[C::IT], wrow_l[C::JF];
#pragma unroll
  for (int i = 0; i < C::IT; ++i) xrow[i] = wt * C::TT + i * C::TILE + frow;
#pragma unroll
  for (int j = 0; j < C::JF; ++j) {
    int base;
    if constexpr (EPI == EPI_SILU) {
      constexpr int HJ = C::JF / 2;  // first half of the wave's tiles: gate, second: up
      base = (j < HJ) ? wf * (C::TF / 2) + j * C::TILE : BF / 2 + wf * (C::TF / 2) + (j - HJ) * C::TILE;
    } else {
      base = wf * C::TF + j * C::TILE;
    }
    wrow_l[j] = base + frow;
  }

  acc_t acc[C::JF][C::IT];
#pragma unroll
  for (int j = 0; j < C::JF; ++j)
#pragma unroll
    for (int i = 0; i < C::IT; ++i)
#pragma unroll
      for (int r = 0; r < ACC_N; ++r) acc[j][i][r] = 0.f;

  // ---- main loop: register-staged double buffering ------------------------
  if (k_tiles > 0) {
    load_tile(0);
    store_tile(0);
  }
  __syncthreads();
  for (int kt = 0; kt < k_tiles; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < k_tiles) load_tile(kt + 1);
    const uint4* xl = lds + buf * BUF;
    const uint4* wl = xl + C::XCH;
#pragma unroll
    for (int ks = 0; ks < BK / C::KSTEP; ++ks) {
      const int kc = ks * C::KGROUPS + kgrp;
      vec8 xf[C::IT], wfr[C::JF];
#pragma unroll
      for (int i = 0; i < C::IT; ++i) {
        const uint4 v = xl[xrow[i] * CPR + swizzle<CPR>(xrow[i], kc)];
        xf[i] = *reinterpret_cast<const vec8*>(&v);
      }
#pragma unroll
      for (int j = 0; j < C::JF; ++j) {
        const uint4 v = wl[wrow_l[j] * CPR + swizzle<CPR>(wrow_l[j], kc)];
        wfr[j] = *reinterpret_cast<const vec8*>(&v);
      }
#pragma unroll
      for (int j = 0; j < C::JF; ++j)
#pragma unroll
        for (int i = 0; i < C::IT; ++i) {
          if constexpr (C::TILE == 32) acc[j][i] = Mfma<T>::m32(wfr[j], xf[i], acc[j][i]);
          else acc[j][i] = Mfma<T>::m16(wfr[j], xf[i], acc[j][i]);
        }
    }
    if (kt + 1 < k_tiles) store_tile(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue -------------------------------------------------------------
  // lane holds token column (lane % TILE) of each token tile and, per accumulator
  // group g (TILE==32: 4 groups of 4 regs; TILE==16: one), 4 consecutive features
  // starting at frow_base(g) = g*8 + kgrp*4 (TILE==32) or kgrp*4 (TILE==16).
  constexpr int GROUPS = ACC_N / 4;
#pragma unroll
  for (int i = 0; i < C::IT; ++i) {
    const int slot = pid_t * BT + wt * C::TT + i * C::TILE + frow;
    int sid = 0;
    float rw = 1.f;
    bool valid = true;
    if constexpr (EPI != EPI_SILU) {
      sid = a.sorted[slot];
      valid = sid < a.num_valid;
      if (valid && a.mul_weight) rw = a.topk_w[sid];
    }
    if constexpr (EPI == EPI_SILU) {
      constexpr int HJ = C::JF / 2;
      T* orow = static_cast<T*>(a.out) + static_cast<int64_t>(slot) * a.ldo;
#pragma unroll
      for (int j = 0; j < HJ; ++j)
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
          const int f = pid_f * (BF / 2) + wf * (C::TF / 2) + j * C::TILE + g * 8 + kgrp * 4;
          typename Mfma<T>::vec4 o;
#pragma unroll
          for (int r = 0; r < 4; ++r)
            o[r] = static_cast<T>(silu(acc[j][i][g * 4 + r]) * acc[j + HJ][i][g * 4 + r]);
          if (f + 3 < a.N) *reinterpret_cast<typename Mfma<T>::vec4*>(orow + f) = o;
          else
            for (int r = 0; r < 4; ++r)
              if (f + r < a.N) orow[f + r] = o[r];
        }
    } else if constexpr (EPI == EPI_DOWN) {
      if (valid) {
        float* orow = static_cast<float*>(a.out) + static_cast<int64_t>(split) * a.split_stride +
                      static_cast<int64_t>(sid) * a.ldo;
#pragma unroll
        for (int j = 0; j < C::JF; ++j)
#pragma unroll
          for (int g = 0; g < GROUPS; ++g) {
            const int f = pid_f * BF + wf * C::TF + j * C::TILE + g * 8 + kgrp * 4;
            f32x4 o;
#pragma unroll
            for (int r = 0; r < 4; ++r) o[r] = acc[j][i][g * 4 + r] * rw;
            if (f + 3 < a.N) *reinterpret_cast<f32x4*>(orow + f) = o;
            else
              for (int r = 0; r < 4; ++r)
                if (f + r < a.N) orow[f + r] = o[r];
          }
      }
    } else {
      if (valid) {
        T* orow = static_cast<T*>(a.out) + static_cast<int64_t>(sid) * a.ldo;
#pragma unroll
        for (int j = 0; j < C::JF; ++j)
#pragma unroll
          for (int g = 0; g < GROUPS; ++g) {
            const int f = pid_f * BF + wf * C::TF + j * C::TILE + g * 8 + kgrp * 4;
            typename Mfma<T>::vec4 o;
#pragma unroll
            for (int r = 0; r < 4; ++r) o[r] = static_cast<T>(acc[j][i][g * 4 + r] * rw);
            if (f + 3 < a.N) *reinterpret_cast<typename Mfma<T>::vec4*>(orow + f) = o;
            else
              for (int r = 0; r < 4; ++r)
                if (f + r < a.N) orow[f + r] = o[r];
          }
      }
    }
  }
}

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
template <typename T, typename C, int EPI>
int launch_gemm(const GemmArgs& a, int splits, hipStream_t st) {
  static bool attr_set = false;
  if (C::LDS_BYTES > 65536 && !attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&moe_gemm_kernel<T, C, EPI>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
    if (e != hipSuccess) return fail(FR_E_LAUNCH, "hipFuncSetAttribute(%d B LDS): %s", C::LDS_BYTES, hipGetErrorString(e));
    attr_set = true;
  }
  const unsigned grid_x = static_cast<unsigned>(a.num_t_blocks) * static_cast<unsigned>(a.num_f_tiles);
  hipLaunchKernelGGL((moe_gemm_kernel<T, C, EPI>), dim3(grid_x, splits), dim3(C::NT), C::LDS_BYTES, st, a);
  return check_launch("moe_gemm_kernel");
}

// Token-block sizes and their tile shapes.  Large blocks: 8 wavefronts, 32x32x16
// MFMA; small blocks (decode): 4 wavefronts side by side along the features,
// 16x16x32 MFMA and a deeper K tile so each workgroup keeps more weight bytes in flight.
typedef Cfg<128, 256, 64, 2, 4, 32> CfgT128;
typedef Cfg<64, 256, 64, 2, 4, 32> CfgT64;
typedef Cfg<32, 128, 128, 1, 4, 16> CfgT32;
typedef Cfg<16, 128, 128, 1, 4, 16> CfgT16;

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
    case 128: fill(128, 256, 64); return launch_gemm<T, CfgT128, EPI>(a, splits, st);
    case 64: fill(64, 256, 64); return launch_gemm<T, CfgT64, EPI>(a, splits, st);
    case 32: fill(32, 128, 128); return launch_gemm<T, CfgT32, EPI>(a, splits, st);
    case 16: fill(16, 128, 128); return launch_gemm<T, CfgT16, EPI>(a, splits, st);
    default: return fail(FR_E_SHAPE, "routing block %d not in {16, 32, 64, 128}", block);
  }
}

int k_multiple_for_block(int block) { return block >= 64 ? 64 : 128; }

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
  FR_REQUIRE(block == 16 || block == 32 || block == 64 || block == 128, FR_E_SHAPE, "fr_moe_grouped_gemm: block=%d not in {16,32,64,128}", block);
  FR_REQUIRE(K > 0 && K % k_multiple_for_block(block) == 0, FR_E_SHAPE, "fr_moe_grouped_gemm: K=%lld must be a positive multiple of %d for block %d", (long long)K, k_multiple_for_block(block), block);
  FR_REQUIRE(N > 0 && N % 4 == 0, FR_E_SHAPE, "fr_moe_grouped_gemm: N=%lld must be a positive multiple of 4", (long long)N);
  FR_REQUIRE(top_k >= 1 && E >= 1, FR_E_SHAPE, "fr_moe_grouped_gemm: top_k=%d E=%d", top_k, E);
  FR_REQUIRE(sorted_len >= block && sorted_len < (int64_t(1) << 31) && num_valid < (int64_t(1) << 31), FR_E_SHAPE, "fr_moe_grouped_gemm: sorted_len=%lld", (long long)sorted_len);
  FR_REQUIRE(lda % 8 == 0 && aligned16(A) && aligned16(B) && aligned16(C), FR_E_ALIGN, "fr_moe_grouped_gemm: operands must be 16-byte aligned, lda %% 8 == 0");
  GemmArgs a = {};
  a.X = A; a.ldx = lda; a.W = B; a.w_expert_stride = N * K; a.out = C; a.ldo = N;
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
  FR_REQUIRE(block == 16 || block == 32 || block == 64 || block == 128, FR_E_SHAPE, "fr_moe_gateup_silu: block=%d not in {16,32,64,128}", block);
  FR_REQUIRE(H > 0 && H % k_multiple_for_block(block) == 0, FR_E_SHAPE, "fr_moe_gateup_silu: H=%lld must be a multiple of %d for block %d", (long long)H, k_multiple_for_block(block), block);
  FR_REQUIRE(F > 0 && F % 8 == 0, FR_E_SHAPE, "fr_moe_gateup_silu: F=%lld must be a positive multiple of 8", (long long)F);
  FR_REQUIRE(topk >= 1 && E >= 1 && M * topk < (int64_t(1) << 30), FR_E_SHAPE, "fr_moe_gateup_silu: M*topk too large");
  FR_REQUIRE(aligned16(x) && aligned16(w1) && aligned16(act), FR_E_ALIGN, "fr_moe_gateup_silu: operands must be 16-byte aligned");
  const int64_t n = M * topk, sorted_len = n + int64_t(E) * (block - 1);
  GemmArgs a = {};
  a.X = x; a.ldx = H; a.W = w1; a.w_expert_stride = 2 * F * H; a.out = act; a.ldo = F;
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
  FR_REQUIRE(block == 16 || block == 32 || block == 64 || block == 128, FR_E_SHAPE, "fr_moe_down_combine: block=%d not in {16,32,64,128}", block);
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
  a.X = act; a.ldx = F; a.W = w2; a.w_expert_stride = H * F; a.out = partial; a.ldo = H;
  a.split_stride = n * H;
  a.sorted = sorted_token_ids; a.expert_ids = expert_ids; a.npost = num_tokens_post_pad;
  a.topk_w = topk_weights; a.num_valid = (int)n; a.top_k = 0; a.N = (int)H; a.K = (int)F;
  a.mul_weight = 1;
  int rc = dispatch_dtype<EPI_DOWN>(a, dtype, block, splits, sorted_len / block * block, st);
  if (rc != FR_OK) return rc;
  return launch_combine(partial, n * H, splits, topk, M, (int)H, dtype, out, st);
}
