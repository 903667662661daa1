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
#include "gating_core.h"
#include "moe_gemm_kernel.h"

namespace fr {

constexpr int kRowsMax = 4;        // tokens in the batch (hence token rows per pass over a routing block) the row form takes
constexpr int kRowsThreads = 256;  // 4 wavefronts
constexpr int kRowsMinK = 4096;    // shorter rows: the tile kernel is as fast (measured at 1024 and 2048)
constexpr int kRowsMinKRouted = 2048;  // ... unless this launch also does the routing: one launch less ahead of it
constexpr int kRowsWaves = 4096;   // wavefronts the feature runs are cut for: 16 on each of 256 CUs
constexpr int kRowsWaveBytes = 7 * 16384;  // weight bytes a wavefront streams
constexpr int kRowsLds = 62464;    // token rows in LDS: the default limit of 64 KB less the kernel's static arrays

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

// Routing done by the gate/up launch itself (whole layer from router logits, up to kRowsMax tokens): every
// workgroup gates the tokens and sorts the few pairs for itself in LDS - the same gating core and the same
// order as the routing kernels - and workgroup (0, 0) also leaves the arrays in global memory for the down
// projection.  One launch and its gap less in front of a layer that lasts ~110 us.
struct RowsRoute {
  const void* logits;   // [M, E] dense, or nullptr: the routing arrays of GemmArgs are read instead
  int logits_dtype;
  int E, topk, renorm;
  float* w_out;         // [M, topk]
  int32_t* ids_out;     // [M, topk]
  int32_t* sorted_out;  // first npost entries written
  int32_t* expert_out;  // first npost / block entries written
  int32_t* npost_out;
};
constexpr int kRowsPairs = 32;                  // pairs at most (kRowsMax tokens x topk <= 8)
constexpr int kRowsSlots = kRowsPairs * 16;     // slots of the in-LDS routing arrays (blocks of 16)

template <typename LT, int G, int VPL>
__device__ __forceinline__ void rows_gate_as(const LT* logits, int M, int E, int topk, int renorm, float* w, int32_t* ids) {
  constexpr int PER = kWave / G;  // tokens per pass of one wavefront
  const int lane = threadIdx.x & (kWave - 1);
  for (int base = 0; base < M; base += PER) {
    const int token = base + lane / G;
    const bool live = token < M;
    const LT* row = logits + static_cast<int64_t>(live ? token : 0) * E;
    gate_token<G, VPL>([&](int e) { return to_float(row[e]); }, live, E, topk, renorm, w + token * topk, ids + token * topk);
  }
}
template <typename LT>
__device__ __forceinline__ void rows_gate(const LT* logits, int M, int E, int topk, int renorm, float* w, int32_t* ids) {
  if (E <= 1) rows_gate_as<LT, 1, 1>(logits, M, E, topk, renorm, w, ids);
  else if (E <= 2) rows_gate_as<LT, 2, 1>(logits, M, E, topk, renorm, w, ids);
  else if (E <= 4) rows_gate_as<LT, 4, 1>(logits, M, E, topk, renorm, w, ids);
  else if (E <= 8) rows_gate_as<LT, 8, 1>(logits, M, E, topk, renorm, w, ids);
  else if (E <= 16) rows_gate_as<LT, 16, 1>(logits, M, E, topk, renorm, w, ids);
  else if (E <= 32) rows_gate_as<LT, 32, 1>(logits, M, E, topk, renorm, w, ids);
  else if (E <= 64) rows_gate_as<LT, 64, 1>(logits, M, E, topk, renorm, w, ids);
  else if (E <= 128) rows_gate_as<LT, 64, 2>(logits, M, E, topk, renorm, w, ids);
  else rows_gate_as<LT, 64, 4>(logits, M, E, topk, renorm, w, ids);
}

// CH = 16-byte chunks per lane, row and round: a weight row is `rounds` x CH x 512 elements (CH = 8 for K = 4096
// and 8192, 5 for 5120, 6 for 6144, 7 for 7168, 4 for 2048); a lane has 2 * CH loads in flight.
// grid.x * 4 wavefronts cover the F features in runs of `fpw`; grid.y = routing blocks (upper bound).
// A block's slots are taken `rows` at a time (rows = tokens in the batch <= kRowsMax): a token
// selects an expert once, so all rows of a block are in its first pass and the later passes find
// nothing; ids with repeated experts per token still come out right, at one more pass over the weights.
template <typename T, int CH>
__global__ void __launch_bounds__(kRowsThreads) gateup_rows_kernel(GemmArgs a, int block, int rows, int fpw, RowsRoute rt) {
  extern __shared__ u32x4 xs[];  // rows x K/8 chunks
  __shared__ float r_w[kRowsPairs];
  __shared__ int32_t r_ids[kRowsPairs], r_sorted[kRowsSlots], r_expert[kRowsPairs], r_npost;
  const int b = blockIdx.y;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int32_t* sorted = a.sorted;
  const int32_t* expert_ids = a.expert_ids;
  int npost;
  if (rt.logits != nullptr) {
    // ---- routing in LDS: gating by wavefront 0, then the stable sort of the n <= kRowsPairs pairs ----
    const int M = a.num_valid / a.top_k, n = a.num_valid;
    if (wave == 0) {
      if (rt.logits_dtype == FR_F32) rows_gate(static_cast<const float*>(rt.logits), M, rt.E, rt.topk, rt.renorm, r_w, r_ids);
      else if (rt.logits_dtype == FR_BF16) rows_gate(static_cast<const bf16_t*>(rt.logits), M, rt.E, rt.topk, rt.renorm, r_w, r_ids);
      else rows_gate(static_cast<const f16_t*>(rt.logits), M, rt.E, rt.topk, rt.renorm, r_w, r_ids);
    }
    __syncthreads();
    // pair p of expert e goes to slot block * (experts below e that have pairs) + (pairs of e before p);
    // every expert holds at most `block` pairs here (a token names an expert once, tokens <= block)
    for (int i = threadIdx.x; i < n * block; i += kRowsThreads) r_sorted[i] = n;
    __syncthreads();
    // An id outside [0, E) (a token row of NaN logits can leave one behind) is a dropped pair, as in the
    // routing kernels: no slot, no block, never an index into the weights.
    if (threadIdx.x < n) {
      const int p = threadIdx.x, e = r_ids[p];
      int rank = 0, below = 0;
      unsigned long long seen_lo = 0, seen_hi = 0, seen_2 = 0, seen_3 = 0;  // experts < e that occur (E <= 256)
      for (int q = 0; q < n; ++q) {
        const int eq = r_ids[q];
        if (eq < 0 || eq >= rt.E) continue;
        if (eq == e && q < p) ++rank;
        if (eq < e) {
          unsigned long long& word = eq < 64 ? seen_lo : (eq < 128 ? seen_hi : (eq < 192 ? seen_2 : seen_3));
          const unsigned long long bit = 1ull << (eq & 63);
          if (!(word & bit)) { word |= bit; ++below; }
        }
      }
      if (e >= 0 && e < rt.E) {
        r_sorted[below * block + rank] = p;
        if (rank == 0) r_expert[below] = e;
      }
    }
    if (threadIdx.x == 0) {  // blocks = distinct experts
      int blocks = 0;
      unsigned long long s0 = 0, s1 = 0, s2 = 0, s3 = 0;
      for (int q = 0; q < n; ++q) {
        const int eq = r_ids[q];
        if (eq < 0 || eq >= rt.E) continue;
        unsigned long long& word = eq < 64 ? s0 : (eq < 128 ? s1 : (eq < 192 ? s2 : s3));
        const unsigned long long bit = 1ull << (eq & 63);
        if (!(word & bit)) { word |= bit; ++blocks; }
      }
      r_npost = blocks * block;
    }
    __syncthreads();
    npost = r_npost;
    if (blockIdx.x == 0 && blockIdx.y == 0) {  // the arrays the down projection reads
      for (int i = threadIdx.x; i < n; i += kRowsThreads) {
        rt.w_out[i] = r_w[i];
        rt.ids_out[i] = r_ids[i];
      }
      for (int i = threadIdx.x; i < npost; i += kRowsThreads) rt.sorted_out[i] = r_sorted[i];
      for (int i = threadIdx.x; i < npost / block; i += kRowsThreads) rt.expert_out[i] = r_expert[i];
      if (threadIdx.x == 0) rt.npost_out[0] = npost;
    }
    sorted = r_sorted;
    expert_ids = r_expert;
  } else {
    npost = *a.npost;
  }
  if (b * block >= npost) return;
  const int kch = a.K >> 3;
  const int f0 = (blockIdx.x * (kRowsThreads / kWave) + wave) * fpw;
  const int f1 = f0 + fpw < a.N ? f0 + fpw : a.N;
  const int expert = expert_ids[b];
  if (expert < 0 || expert >= a.num_experts) return;  // never form a weight address from an id the routing did not vouch for
  const T* wbase = static_cast<const T*>(a.W) + static_cast<int64_t>(expert) * a.w_expert_stride;
  const int rounds = kch / (kWave * CH);
  // one load for the block's ids (block <= 64): lane l of every wavefront holds slot l's
  const int sid_l = lane < block ? sorted[b * block + lane] : a.num_valid;
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

// Chunks per round for rows of K elements: the largest of 8..4 that divides K / 512, or 0.
inline int rows_chunks(int64_t K) {
  if (K % 512 != 0) return 0;
  const int64_t nc = K / 512;
  for (int ch = 8; ch >= 4; --ch)
    if (nc % ch == 0) return ch;
  return 0;
}

// Whether the row form takes this gate/up projection: 2-byte operands, at most kRowsMax tokens,
// routing blocks of at most 64 slots, weight rows of whole rounds, token rows that fit the LDS.
// Whether the same launch can also do the routing (gating + sort) of the layer.
inline bool gateup_rows_routes(int64_t M, int E, int topk, int block) {
  return M * topk <= kRowsPairs && E <= 256 && topk <= E && M <= block && block <= 16;
}
inline bool gateup_rows_fits(int64_t M, int64_t K, int block, int64_t sorted_len, int elem_bytes, int64_t min_k = kRowsMinK) {
  const int64_t rows = M < block ? M : block;
  return elem_bytes == 2 && M >= 1 && M <= kRowsMax && block <= kWave && K >= min_k && rows_chunks(K) != 0 &&
         rows * K * 2 <= kRowsLds && sorted_len / block <= 65535;  // routing blocks are the grid's y dimension
}

template <typename T>
int launch_gateup_rows(const GemmArgs& a, int block, int64_t sorted_len, hipStream_t st, const RowsRoute& rt = RowsRoute{}) {
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
  // a block holds at least one pair: no more blocks than pairs
  const int64_t max_blocks = sorted_len / block < a.num_valid ? sorted_len / block : a.num_valid;
  const dim3 grid(static_cast<unsigned>(ceil_div(a.N, static_cast<int64_t>(kRowsThreads / kWave) * fpw)),
                  static_cast<unsigned>(max_blocks));
  const size_t lds = static_cast<size_t>(rows) * a.K * sizeof(T);
  switch (rows_chunks(a.K)) {
    case 8: hipLaunchKernelGGL((gateup_rows_kernel<T, 8>), grid, dim3(kRowsThreads), lds, st, a, block, rows, fpw, rt); break;
    case 7: hipLaunchKernelGGL((gateup_rows_kernel<T, 7>), grid, dim3(kRowsThreads), lds, st, a, block, rows, fpw, rt); break;
    case 6: hipLaunchKernelGGL((gateup_rows_kernel<T, 6>), grid, dim3(kRowsThreads), lds, st, a, block, rows, fpw, rt); break;
    case 5: hipLaunchKernelGGL((gateup_rows_kernel<T, 5>), grid, dim3(kRowsThreads), lds, st, a, block, rows, fpw, rt); break;
    case 4: hipLaunchKernelGGL((gateup_rows_kernel<T, 4>), grid, dim3(kRowsThreads), lds, st, a, block, rows, fpw, rt); break;
    default: return fail(FR_E_SHAPE, "gate/up by rows: K=%d", a.K);
  }
  return check_launch("gateup_rows_kernel");
}

// ---- down projection + top-k combine for a handful of pairs -------------------------------
// out[m, h] = sum over the pairs p of token m of topk_w[p] * (act[slot(p), :] . W2[expert(p), h, :]).
// With at most kDownPairs routed pairs in the whole batch the job is again to stream each active
// expert's H weight rows once at HBM rate - but these rows are F elements long (28 KB for F = 14336),
// too long to keep every pair's activated row in LDS next to many resident wavefronts.  So the K range
// is split over the wavefronts of a workgroup: wavefront w keeps ITS slice (CH chunks of 512 elements)
// of every pair's activated row in registers for the whole kernel, and for each of the workgroup's output
// features streams the same slice of the weight row of every active expert (16-byte non-temporal loads,
// HB features x CH chunks in flight per lane), multiplies with v_dot2 in fp32, sums over its lanes and
// leaves the partial sums in LDS; after one barrier per HB features a few threads add the wavefronts'
// partial sums in wavefront order, apply the routed weights, add a token's pairs in slot order and store
// out[m, h] - no partial buffer, no combine launch, no K slices in HBM; the order of every sum is fixed
// by the routing arrays, so results are identical from run to run.
constexpr int kDownPairs = 4;     // routed pairs in the batch, at most (with 8, two weight-row loads per lane and step fit the
                                  // registers next to the activated rows: measured 10-18 % slower than the tile kernel with K slices)
constexpr int kDownWaves = 16;    // wavefronts per workgroup, at most
constexpr int kDownMinK = 4096;   // shorter rows: the tile kernel with K slices is as fast

// CH chunks of 512 elements per wavefront: 1 or 2 (more would spill at 16 wavefronts per CU), the smaller that
// leaves at most kDownWaves wavefronts, or 0: rows of up to 16384 elements
inline int down_rows_chunks(int64_t K) {
  if (K % 512 != 0) return 0;
  const int64_t nc = K / 512;
  for (int ch = 1; ch <= 2; ++ch)
    if (nc % ch == 0 && nc / ch <= kDownWaves) return ch;
  return 0;
}
inline bool down_rows_fits(int64_t n_pairs, int64_t K, int64_t N, int64_t sorted_len, int elem_bytes) {
  return elem_bytes == 2 && n_pairs >= 1 && n_pairs <= kDownPairs && K >= kDownMinK && down_rows_chunks(K) != 0 &&
         N % 8 == 0 && sorted_len <= 4096;
}

// NP = pairs the registers are sized for (>= the batch's), HB = output features per step.
// a.X = act [slots, K], a.W = W2 [E, N, K], a.out = out [tokens, N]; a.group_t = routing block;
// `slots` = whole routing blocks inside sorted_token_ids; hpw = features per workgroup (multiple of HB).
//
// Every wavefront builds the pair table for itself (no LDS, no barrier before the first weight load):
// the real slots in order, kept one pair per LANE of a few registers and read back with v_readlane;
// pairs of one expert are adjacent (the routing arrays are sorted by expert), a run of them is a group.
// The weight stream is a sequence of steps (round of HB features, group); the loads of step i + 1 are in
// flight while step i is multiplied (two register buffers), so the stream never drains inside a workgroup.
template <typename T, int CH, int NP, int HB>
__global__ void __launch_bounds__(kDownWaves * kWave) down_rows_kernel(GemmArgs a, int topk, int slots, int hpw) {
  __shared__ float red[2][kDownWaves][HB * NP];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave, nwaves = blockDim.x / kWave;
  const int block = a.group_t;
  // ---- pair table ------------------------------------------------------------------------------
  int t_slot = 0, t_sid = 0, t_exp = 0, g_first = 0;  // lane p: pair p; lane g: first pair of group g
  int np = 0, ng = 0;
  {
    const int npost = *a.npost;
    int prev_e = -1;
    for (int base = 0; base < slots; base += kWave) {
      const int s = base + lane;
      int sid = a.num_valid, ev = 0;
      if (s < slots) {
        sid = a.sorted[s];
        ev = a.expert_ids[s / block];
      }
      unsigned long long m = __ballot(s < npost && sid < a.num_valid);
      while (m != 0 && np < NP) {
        const int bpos = __builtin_ctzll(m);
        m &= m - 1;
        const int e = __builtin_amdgcn_readlane(ev, bpos);
        t_slot = (lane == np ? (base + bpos) : t_slot);
        t_sid = (lane == np ? (__builtin_amdgcn_readlane(sid, bpos)) : t_sid);
        t_exp = (lane == np ? (e) : t_exp);
        if (e != prev_e) {
          g_first = (lane == ng ? (np) : g_first);
          ++ng;
          prev_e = e;
        }
        ++np;
      }
      if (base + kWave >= npost) break;
    }
    g_first = (lane == ng ? (np) : g_first);  // group g = pairs [g_first[g], g_first[g + 1])
  }
  const float t_w = lane < np ? a.topk_w[t_sid] : 0.f;
  const int t_tok = t_sid / topk;
  const int tokens = a.num_valid / topk;
  // ---- this wavefront's slice of every pair's activated row -----------------------------------
  const int kofs = (wave * CH) * 512 + lane * 8;  // first element of the lane's first chunk
  u32x4 ar[NP][CH];
#pragma unroll
  for (int p = 0; p < NP; ++p)
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      ar[p][c] = u32x4{0u, 0u, 0u, 0u};
      if (p < np)
        ar[p][c] = *reinterpret_cast<const u32x4*>(static_cast<const T*>(a.X) +
                                                   static_cast<int64_t>(__builtin_amdgcn_readlane(t_slot, p)) * a.ldx + kofs + c * 512);
    }
  const int h_begin = blockIdx.x * hpw, h_end = min(h_begin + hpw, a.N);
  if (ng == 0) {  // no valid pair at all (every id out of range): the sum over nothing is zero
    for (int i = threadIdx.x; i < tokens * (h_end - h_begin); i += blockDim.x)
      static_cast<typename Elem<T>::out_t*>(a.out)[static_cast<int64_t>(i / (h_end - h_begin)) * a.ldo + h_begin + i % (h_end - h_begin)] =
          static_cast<typename Elem<T>::out_t>(0.f);
    return;
  }
  const int rounds = (h_end - h_begin + HB - 1) / HB, steps = rounds * ng;
  float acc[HB][NP];
#pragma unroll
  for (int hb = 0; hb < HB; ++hb)
#pragma unroll
    for (int p = 0; p < NP; ++p) acc[hb][p] = 0.f;
  u32x4 w0[HB][CH], w1[HB][CH];
  // loads of step (round r, group g) into wb
#define FR_DR_ISSUE(wb, r_, g_)                                                                                   \
  {                                                                                                               \
    const int e_ = __builtin_amdgcn_readlane(t_exp, __builtin_amdgcn_readlane(g_first, (g_)));                    \
    const T* wp_ = static_cast<const T*>(a.W) + static_cast<int64_t>(e_) * a.w_expert_stride + kofs;              \
    _Pragma("unroll") for (int hb = 0; hb < HB; ++hb) {                                                           \
      const int h_ = h_begin + (r_) * HB + hb < a.N ? h_begin + (r_) * HB + hb : a.N - 1;                         \
      _Pragma("unroll") for (int c = 0; c < CH; ++c)                                                              \
        wb[hb][c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wp_ + static_cast<int64_t>(h_) * a.ldw + c * 512)); \
    }                                                                                                             \
  }
  // step (round r, group g) multiplied from wb
#define FR_DR_FMA(wb, g_)                                                                                         \
  {                                                                                                               \
    const int p0_ = __builtin_amdgcn_readlane(g_first, (g_)), p1_ = __builtin_amdgcn_readlane(g_first, (g_) + 1); \
    _Pragma("unroll") for (int p = 0; p < NP; ++p) {                                                              \
      if (p >= p0_ && p < p1_) {                                                                                  \
        _Pragma("unroll") for (int hb = 0; hb < HB; ++hb)                                                         \
          _Pragma("unroll") for (int c = 0; c < CH; ++c)                                                          \
            _Pragma("unroll") for (int d = 0; d < 4; ++d) acc[hb][p] = Dot2<T>::fma2(wb[hb][c][d], ar[p][c][d], acc[hb][p]); \
      }                                                                                                           \
    }                                                                                                             \
  }
  // after a round's last group the round is summed over lanes, wavefronts and a token's pairs, and stored
#define FR_DR_FINISH(r_, g_)                                                                                      \
  {                                                                                                               \
    if ((g_) == ng - 1) {                                                                                         \
      const int buf_ = (r_) & 1, h0_ = h_begin + (r_) * HB;                                                       \
      _Pragma("unroll") for (int hb = 0; hb < HB; ++hb)                                                           \
        _Pragma("unroll") for (int p = 0; p < NP; ++p) {                                                          \
          if (p < np) {                                                                                           \
            const float v_ = wave_sum(acc[hb][p]);                                                                \
            if (lane == 0) red[buf_][wave][hb * NP + p] = v_;                                                     \
          }                                                                                                       \
          acc[hb][p] = 0.f;                                                                                       \
        }                                                                                                         \
      __syncthreads(); /* one barrier per round: the other buffer is written only after every wavefront passed this one */ \
      if (threadIdx.x < HB * tokens) {                                                                            \
        const int hb = threadIdx.x % HB, m = threadIdx.x / HB, h = h0_ + hb;                                      \
        if (h < h_end) {                                                                                          \
          float s_ = 0.f;                                                                                         \
          for (int p = 0; p < np; ++p) { /* wavefronts in order, then the token's pairs in slot order */          \
            if (__builtin_amdgcn_readlane(t_tok, p) != m) continue;                                               \
            float d_ = 0.f;                                                                                       \
            for (int wv = 0; wv < nwaves; ++wv) d_ += red[buf_][wv][hb * NP + p];                                 \
            s_ += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(t_w), p)) * d_;                         \
          }                                                                                                       \
          static_cast<typename Elem<T>::out_t*>(a.out)[static_cast<int64_t>(m) * a.ldo + h] = static_cast<typename Elem<T>::out_t>(s_); \
        }                                                                                                         \
      }                                                                                                           \
    }                                                                                                             \
  }
#define FR_DR_NEXT(r_, g_) { if (++(g_) == ng) { (g_) = 0; ++(r_); } }
  // a buffer is refilled as soon as its step has been multiplied, before that round's sums: two steps' loads stay in flight
  int r = 0, g = 0, rn = 0, gn = 0;  // step being multiplied, step being loaded
  if (steps > 0) {
    FR_DR_ISSUE(w0, rn, gn)
    FR_DR_NEXT(rn, gn)
  }
  if (steps > 1) {
    FR_DR_ISSUE(w1, rn, gn)
    FR_DR_NEXT(rn, gn)
  }
  for (int i = 0; i < steps; i += 2) {
    FR_DR_FMA(w0, g)
    if (i + 2 < steps) {
      FR_DR_ISSUE(w0, rn, gn)
      FR_DR_NEXT(rn, gn)
    }
    FR_DR_FINISH(r, g)
    FR_DR_NEXT(r, g)
    if (i + 1 >= steps) break;
    FR_DR_FMA(w1, g)
    if (i + 3 < steps) {
      FR_DR_ISSUE(w1, rn, gn)
      FR_DR_NEXT(rn, gn)
    }
    FR_DR_FINISH(r, g)
    FR_DR_NEXT(r, g)
  }
#undef FR_DR_NEXT
#undef FR_DR_FINISH
#undef FR_DR_FMA
#undef FR_DR_ISSUE
}

template <typename T, int CH>
int launch_down_rows_ch(const GemmArgs& a, int topk, int block, int64_t sorted_len, hipStream_t st) {
  const int nwaves = static_cast<int>(a.K / 512 / CH);
  const int np = a.num_valid;
  GemmArgs b = a;
  b.group_t = block;
  const int slots = static_cast<int>(sorted_len / block * block);
  // one workgroup per CU (its wavefronts fill the CU's registers with the activated rows and the two
  // weight buffers: 16 loads of 16 bytes in flight per lane), steps of HB features
  auto go = [&](auto kern, int HB) {
    int hpw = static_cast<int>(ceil_div(a.N, 256));
    hpw = static_cast<int>(round_up(hpw < HB ? HB : hpw, HB));
    const unsigned grid = static_cast<unsigned>(ceil_div(a.N, hpw));
    hipLaunchKernelGGL(kern, dim3(grid), dim3(nwaves * kWave), 0, st, b, topk, slots, hpw);
  };
  constexpr int HB = 8 / CH;
  static_assert(kDownPairs == 4, "register variants below");
  if (np <= 2) go(down_rows_kernel<T, CH, 2, HB>, HB);
  else go(down_rows_kernel<T, CH, 4, HB>, HB);
  return check_launch("down_rows_kernel");
}

template <typename T>
int launch_down_rows(const GemmArgs& a, int topk, int block, int64_t sorted_len, hipStream_t st) {
  switch (down_rows_chunks(a.K)) {
    case 1: return launch_down_rows_ch<T, 1>(a, topk, block, sorted_len, st);
    case 2: return launch_down_rows_ch<T, 2>(a, topk, block, sorted_len, st);
    default: return fail(FR_E_SHAPE, "down projection by rows: K=%d", a.K);
  }
}

}  // namespace fr
