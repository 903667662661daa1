// Gate/up projection for a handful of tokens: the decode case.
//
// With at most kRowsMax tokens in the whole batch a routing block holds one or two
// token rows, the MFMA tile is 15/16 padding and the job is to stream each active
// expert's 2F weight rows past those few token rows once, at HBM rate.  The tiled
// kernel does that through LDS rings with one or two wavefronts per SIMD and a
// barrier per K tile; here every wavefront is on its own: it owns a run of output
// features of one routing block, loads the gate row and the up row of a feature
// straight into registers (16 bytes per lane per load, 8 KB of a row per wavefront
// and instruction round), multiplies them with the block's token rows held in LDS
// (v_dot2_f32_{bf16,f16}: two multiply-adds per instruction, fp32 accumulation),
// sums over the 64 lanes and stores silu(gate)*up.  Twelve to sixteen such
// wavefronts per CU keep ~200 KB of loads in flight per CU with no barrier after
// the token rows are in LDS.  Same arguments and output layout as the EPI_SILU
// tile kernel (act[slot, F]), so the down projection that follows is unchanged.
#pragma once
#include "moe_gemm_kernel.h"

namespace fr {

constexpr int kRowsMax = 4;        // tokens in the batch (hence token rows per pass over a routing block) the row form takes
constexpr int kRowsThreads = 256;  // 4 wavefronts
constexpr int kRowsMinK = 4096;    // shorter rows: the tile kernel is as fast (measured at 1024 and 2048)
constexpr int kRowsWaves = 4096;   // wavefronts the feature runs are cut for: 16 on each of 256 CUs
constexpr int kRowsWaveBytes = 7 * 16384;  // weight bytes a wavefront streams
constexpr int kRowsLds = 65536;    // token rows in LDS: the default dynamic limit

template <typename T> struct Dot2;
template <> struct Dot2<bf16_t> {
  static __device__ __forceinline__ float fma2(unsigned w, unsigned x, float c) {
    typedef __bf16 v2 __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2, w), __builtin_bit_cast(v2, x), c, false);
  }
};
template <> struct Dot2<f16_t> {
  static __device__ __forceinline__ float fma2(unsigned w, unsigned x, float c) {
    typedef _Float16 v2 __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(v2, w), __builtin_bit_cast(v2, x), c, false);
  }
};

__device__ __forceinline__ float wave_sum(float v) {
  v += partner_f32<32>(v);
  v += partner_f32<16>(v);
  v += partner_f32<8>(v);
  v += partner_f32<4>(v);
  v += partner_f32<2>(v);
  v += partner_f32<1>(v);
  return v;
}

// CH = 16-byte chunks per lane, row and round: a weight row is `rounds` x CH x 512 elements (CH = 8 for K = 4096
// and 8192, 5 for 5120, 6 for 6144, 7 for 7168); a lane has 2 * CH loads in flight.
// grid.x * 4 wavefronts cover the F features in runs of `fpw`; grid.y = routing blocks (upper bound).
// A block's slots are taken `rows` at a time (rows = tokens in the batch <= kRowsMax): a token
// selects an expert once, so all rows of a block are in its first pass and the later passes find
// nothing; ids with repeated experts per token still come out right, at one more pass over the weights.
template <typename T, int CH>
__global__ void __launch_bounds__(kRowsThreads) gateup_rows_kernel(GemmArgs a, int block, int rows, int fpw) {
  extern __shared__ u32x4 xs[];  // rows x K/8 chunks
  const int b = blockIdx.y;
  if (b * block >= *a.npost) return;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int kch = a.K >> 3;
  const int f0 = (blockIdx.x * (kRowsThreads / kWave) + wave) * fpw;
  const int f1 = f0 + fpw < a.N ? f0 + fpw : a.N;
  const T* wbase = static_cast<const T*>(a.W) + static_cast<int64_t>(a.expert_ids[b]) * a.w_expert_stride;
  const int rounds = kch / (kWave * CH);
  // one load for the block's ids (block <= 64): lane l of every wavefront holds slot l's
  const int sid_l = lane < block ? a.sorted[b * block + lane] : a.num_valid;
  const unsigned long long real = __ballot(sid_l < a.num_valid);
  bool used = false;
  for (int r0 = 0; r0 < block; r0 += rows) {
    const unsigned mask = static_cast<unsigned>(real >> r0) & ((1u << rows) - 1u);  // uniform
    if (mask == 0) continue;
    if (used) __syncthreads();  // the previous pass has read its rows
    used = true;
    for (int r = 0; r < rows; ++r) {
      if (mask >> r & 1) {
        const int sid = __builtin_amdgcn_readlane(sid_l, r0 + r);
        const u32x4* src = reinterpret_cast<const u32x4*>(static_cast<const T*>(a.X) + static_cast<int64_t>(sid / a.top_k) * a.ldx);
        for (int c = threadIdx.x; c < kch; c += kRowsThreads) xs[r * kch + c] = src[c];
      }
    }
    __syncthreads();
    typename Elem<T>::out_t* act = static_cast<typename Elem<T>::out_t*>(a.out) + (static_cast<int64_t>(b) * block + r0) * a.ldo;
    for (int f = f0; f < f1; ++f) {
      float g[kRowsMax], u[kRowsMax];
#pragma unroll
      for (int r = 0; r < kRowsMax; ++r) g[r] = u[r] = 0.f;
      const u32x4* wg = reinterpret_cast<const u32x4*>(wbase + static_cast<int64_t>(f) * a.ldw) + lane;
      const u32x4* wu = reinterpret_cast<const u32x4*>(wbase + (static_cast<int64_t>(a.N) + f) * a.ldw) + lane;
      for (int s = 0; s < rounds; ++s) {
        u32x4 vg[CH], vu[CH];
#pragma unroll
        for (int c = 0; c < CH; ++c) {
          vg[c] = __builtin_nontemporal_load(wg + (s * CH + c) * kWave);
          vu[c] = __builtin_nontemporal_load(wu + (s * CH + c) * kWave);
        }
#pragma unroll
        for (int r = 0; r < kRowsMax; ++r) {
          if (mask >> r & 1) {
            const u32x4* xr = xs + r * kch + s * CH * kWave + lane;
#pragma unroll
            for (int c = 0; c < CH; ++c) {
              const u32x4 x = xr[c * kWave];
#pragma unroll
              for (int d = 0; d < 4; ++d) {
                g[r] = Dot2<T>::fma2(vg[c][d], x[d], g[r]);
                u[r] = Dot2<T>::fma2(vu[c][d], x[d], u[r]);
              }
            }
          }
        }
      }
#pragma unroll
      for (int r = 0; r < kRowsMax; ++r) {
        if (mask >> r & 1) {
          const float gs = wave_sum(g[r]), us = wave_sum(u[r]);
          if (lane == 0) act[static_cast<int64_t>(r) * a.ldo + f] = static_cast<typename Elem<T>::out_t>(silu(gs) * us);
        }
      }
    }
  }
}

// Chunks per round for rows of K elements: the largest of 8..5 that divides K / 512, or 0.
inline int rows_chunks(int64_t K) {
  if (K % 512 != 0) return 0;
  const int64_t nc = K / 512;
  for (int ch = 8; ch >= 5; --ch)
    if (nc % ch == 0) return ch;
  return 0;
}

// Whether the row form takes this gate/up projection: 2-byte operands, at most kRowsMax tokens,
// routing blocks of at most 64 slots, weight rows of whole rounds, token rows that fit the LDS.
inline bool gateup_rows_fits(int64_t M, int64_t K, int block, int64_t sorted_len, int elem_bytes) {
  const int64_t rows = M < block ? M : block;
  return elem_bytes == 2 && M >= 1 && M <= kRowsMax && block <= kWave && K >= kRowsMinK && rows_chunks(K) != 0 &&
         rows * K * 2 <= kRowsLds && sorted_len / block <= 65535;  // routing blocks are the grid's y dimension
}

template <typename T>
int launch_gateup_rows(const GemmArgs& a, int block, int64_t sorted_len, hipStream_t st) {
  const int M = a.num_valid / a.top_k;
  const int rows = M < block ? M : block;
  // blocks that hold rows: at most one per pair and per expert
  const int64_t active = a.num_valid < a.num_experts ? a.num_valid : a.num_experts;
  // features per wavefront: ~112 KB of weight rows each (measured best from 1 to 4 tokens at K = 4096),
  // fewer when that would leave CUs without a workgroup
  const int64_t by_bytes = ceil_div(kRowsWaveBytes, 2 * a.K * static_cast<int64_t>(sizeof(T)));
  const int64_t by_fill = ceil_div(static_cast<int64_t>(a.N) * active, kRowsWaves);
  int fpw = static_cast<int>(by_bytes < by_fill ? by_bytes : by_fill);
  if (fpw < 1) fpw = 1;
  const dim3 grid(static_cast<unsigned>(ceil_div(a.N, static_cast<int64_t>(kRowsThreads / kWave) * fpw)),
                  static_cast<unsigned>(sorted_len / block));
  const size_t lds = static_cast<size_t>(rows) * a.K * sizeof(T);
  switch (rows_chunks(a.K)) {
    case 8: hipLaunchKernelGGL((gateup_rows_kernel<T, 8>), grid, dim3(kRowsThreads), lds, st, a, block, rows, fpw); break;
    case 7: hipLaunchKernelGGL((gateup_rows_kernel<T, 7>), grid, dim3(kRowsThreads), lds, st, a, block, rows, fpw); break;
    case 6: hipLaunchKernelGGL((gateup_rows_kernel<T, 6>), grid, dim3(kRowsThreads), lds, st, a, block, rows, fpw); break;
    case 5: hipLaunchKernelGGL((gateup_rows_kernel<T, 5>), grid, dim3(kRowsThreads), lds, st, a, block, rows, fpw); break;
    default: return fail(FR_E_SHAPE, "gate/up by rows: K=%d", a.K);
  }
  return check_launch("gateup_rows_kernel");
}

}  // namespace fr
