// Block-aligned stable counting sort of (expert, token) pairs on gfx950.
//
// The n flat pairs are cut into segments of seg_len consecutive pairs, one
// wavefront per segment.  (1) every wavefront builds an LDS histogram of its
// segment; (2) an exclusive scan over segments gives each (expert, segment) its
// offset inside the expert's run, and an exclusive scan over the padded expert
// totals gives each run its start; (3) every wavefront walks its segment again
// 64 pairs at a time and ranks the pairs of one expert among themselves with
// wavefront ballots, so flat order survives inside each expert: the result is
// the stable sort.  Small inputs run all three phases in one workgroup with the
// tables in LDS; large ones use a global table and two launches (count + sums per count
// workgroup, scatter + block table) or, with many experts, three (count, per-expert
// segment scan, scatter + block table).
#include "gating_core.h"
#include "quant_core.h"

namespace fr {
namespace {

constexpr int kSmallThreads = 1024;
constexpr int kSmallWaves = kSmallThreads / kWave;
constexpr int kSmallMaxE = 256;
// One workgroup sorts up to this many pairs; above, two launches spread over the CUs are faster.  Measured, gating +
// sort back to back, one workgroup against two launches: 4096 pairs 12.9 / 14.7 us (8 experts), 15.2 / 16.1 (64 experts);
// 8192 pairs 16.2 / 15.4 and 20.0 / 17.7 us.
constexpr int64_t kSmallMaxN = 6144;
// Gating and sort in ONE launch up to this many pairs (above, the gating kernel spread over the CUs plus the
// one-workgroup sort win: 2048 pairs 31.6 against 29.5 us for a small layer, 1536 pairs on 64 experts 51.8 against 26.5)
constexpr int64_t kRouteAlignMaxN = 1024;
constexpr int kMaxE = 1024;
constexpr int kSegThreads = 256;
constexpr int kSegWaves = kSegThreads / kWave;

__device__ __forceinline__ int64_t min64(int64_t a, int64_t b) { return a < b ? a : b; }

__host__ __device__ inline int bits_for(int E) {
  int b = 0;
  while ((1 << b) < E) ++b;
  return b;
}

// lanes (among `valid` ones) holding the same expert as this lane
__device__ __forceinline__ unsigned long long same_expert_lanes(int e, bool valid, int nbits) {
  unsigned long long m = __ballot(valid);
  for (int b = 0; b < nbits; ++b) {
    const bool bit = (e >> b) & 1;
    const unsigned long long vote = __ballot(bit);
    m &= bit ? vote : ~vote;
  }
  return m;
}

__device__ __forceinline__ int wave_inclusive_scan(int v, int lane) {
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int t = __shfl_up(v, d, kWave);
    if (lane >= d) v += t;
  }
  return v;
}

template <typename IdT>
__device__ __forceinline__ void segment_histogram(const IdT* __restrict__ ids, int64_t lo, int64_t hi,
                                                  int E, int lane, int* hist) {
  for (int64_t p = lo + lane; p < hi; p += kWave) {
    const int e = static_cast<int>(ids[p]);
    if (e >= 0 && e < E) atomicAdd(&hist[e], 1);
  }
}

// Walk [lo, hi) in flat order; cnt[e] holds the next free slot of expert e for
// this wavefront and is advanced as pairs are placed.
constexpr int kScatterPF = 4;  // rounds of 64 pairs whose ids are fetched together: the rounds themselves depend on
                               // one another through cnt[], their loads need not wait for that chain
template <typename IdT>
__device__ __forceinline__ void segment_ids(const IdT* __restrict__ ids, int64_t base0, int64_t hi, int lane, int (&ev)[kScatterPF]) {
#pragma unroll
  for (int r = 0; r < kScatterPF; ++r) {
    const int64_t p = base0 + r * kWave + lane;
    ev[r] = (p < hi) ? static_cast<int>(ids[p]) : -1;
  }
}
// `first`: the ids of the first kScatterPF rounds, fetched by the caller ahead of time (segment_ids), or nullptr
template <typename IdT>
__device__ __forceinline__ void segment_scatter(const IdT* __restrict__ ids, int64_t lo, int64_t hi,
                                                int E, int nbits, int lane, volatile int* cnt,
                                                int32_t* __restrict__ sorted, const int* first = nullptr) {
  const unsigned long long below = (1ull << lane) - 1ull;
  for (int64_t base0 = lo; base0 < hi; base0 += kScatterPF * kWave) {
    int ev[kScatterPF];
    if (first != nullptr && base0 == lo) {
#pragma unroll
      for (int r = 0; r < kScatterPF; ++r) ev[r] = first[r];
    } else {
      segment_ids(ids, base0, hi, lane, ev);
    }
#pragma unroll
    for (int r = 0; r < kScatterPF; ++r) {
      const int64_t base = base0 + r * kWave;
      if (base >= hi) break;
      const int64_t p = base + lane;
      int e = ev[r];
      const bool valid = (p < hi) && e >= 0 && e < E;
      if (!valid) e = 0;
      const unsigned long long same = same_expert_lanes(e, valid, nbits);
      if (valid) {
        const int rank = __popcll(same & below);
        const int total = __popcll(same);
        const int old = cnt[e];
        sorted[old + rank] = static_cast<int32_t>(p);
        if (rank == total - 1) cnt[e] = old + total;
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
}

// start[e] = exclusive scan of the padded totals, start[E] = padded length.
// Executed by one wavefront; total/start live in LDS.
__device__ __forceinline__ void scan_padded_totals(const int* total, int* start, int E, int B, int lane) {
  int running = 0;
  for (int base = 0; base < E; base += kWave) {
    const int e = base + lane;
    const int c = (e < E) ? (total[e] + B - 1) / B * B : 0;
    const int incl = wave_inclusive_scan(c, lane);
    if (e < E) start[e] = running + incl - c;
    running += __shfl(incl, kWave - 1, kWave);
  }
  if (lane == 0) start[E] = running;
}

// expert_ids for every block, padding slots of every run, and the tail.
__device__ __forceinline__ void write_block_table(const int* total, const int* start, int E, int B,
                                                  int64_t n, int64_t sorted_len, int tid, int nthreads,
                                                  int32_t* __restrict__ sorted,
                                                  int32_t* __restrict__ expert_ids,
                                                  int32_t* __restrict__ npost_out) {
  const int npost = start[E];
  const int nblocks = npost / B;
  for (int b = tid; b < nblocks; b += nthreads) {
    const int pos = b * B;
    int lo = 0, hi = E;  // largest e with start[e] <= pos and a non-empty run
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (start[mid] <= pos) lo = mid; else hi = mid;
    }
    expert_ids[b] = lo;
  }
  const int lane = tid % kWave, wave = tid / kWave, nwaves = nthreads / kWave;
  for (int e = wave; e < E; e += nwaves) {
    for (int s = start[e] + total[e] + lane; s < start[e + 1]; s += kWave) sorted[s] = static_cast<int32_t>(n);
  }
  for (int64_t s = npost + tid; s < sorted_len; s += nthreads) sorted[s] = static_cast<int32_t>(n);
  if (tid == 0) npost_out[0] = npost;
}

// ---------------------------------------------------------------- small path
template <typename IdT>
__global__ __launch_bounds__(kSmallThreads) void align_small_kernel(
    const IdT* __restrict__ ids, int64_t n, int E, int B, int seg_len, int64_t sorted_len,
    int32_t* __restrict__ sorted, int32_t* __restrict__ expert_ids, int32_t* __restrict__ npost_out) {
  __shared__ int table[kSmallWaves * kSmallMaxE];
  __shared__ int total[kSmallMaxE];
  __shared__ int start[kSmallMaxE + 1];
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  for (int i = tid; i < kSmallWaves * E; i += kSmallThreads) table[i] = 0;
  __syncthreads();
  const int64_t lo = min64(n, static_cast<int64_t>(wave) * seg_len);
  const int64_t hi = min64(n, lo + seg_len);
  segment_histogram(ids, lo, hi, E, lane, &table[wave * E]);
  __syncthreads();
  for (int e = tid; e < E; e += kSmallThreads) {
    int running = 0;
    for (int w = 0; w < kSmallWaves; ++w) {
      const int c = table[w * E + e];
      table[w * E + e] = running;
      running += c;
    }
    total[e] = running;
  }
  __syncthreads();
  if (wave == 0) scan_padded_totals(total, start, E, B, lane);
  __syncthreads();
  for (int i = tid; i < kSmallWaves * E; i += kSmallThreads) table[i] += start[i % E];
  write_block_table(total, start, E, B, n, sorted_len, tid, kSmallThreads, sorted, expert_ids, npost_out);
  __syncthreads();
  segment_scatter(ids, lo, hi, E, bits_for(E), lane, &table[wave * E], sorted);
}

// bf16 token rows [M, K] to quantise to e4m3 alongside (x == nullptr: none)
struct RowQuant {
  const bf16_t* x;
  unsigned char* q;
  float* scale;
  int K;
};

// Small batches, whole routing in one launch: the workgroup first gates every token
// (a group of G lanes per token, 1024/G tokens per pass; weights and ids go to their
// global arrays), then sorts the ids it has just written exactly as above.
template <typename T, int G, int VPL>
__global__ __launch_bounds__(kSmallThreads) void route_align_small_kernel(
    const T* __restrict__ logits, int64_t M, int E, int topk, int renorm, int B, int seg_len, int64_t sorted_len,
    float* __restrict__ w_out, int32_t* __restrict__ ids_out, int32_t* __restrict__ sorted,
    int32_t* __restrict__ expert_ids, int32_t* __restrict__ npost_out, RowQuant rq) {
  __shared__ int table[kSmallWaves * kSmallMaxE];
  __shared__ int total[kSmallMaxE];
  __shared__ int start[kSmallMaxE + 1];
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  if (blockIdx.x > 0) {  // the fp8 layer's token rows are quantised by further workgroups of the same launch
    const int64_t row = static_cast<int64_t>(blockIdx.x - 1) * kSmallWaves + wave;
    if (row < M) quant_row(rq.x + row * rq.K, rq.K, rq.q + row * rq.K, rq.scale + row, lane);
    return;
  }
  for (int i = tid; i < kSmallWaves * E; i += kSmallThreads) table[i] = 0;
  constexpr int kPerPass = kSmallThreads / G;
  for (int64_t base = 0; base < M; base += kPerPass) {  // uniform trip count: every lane joins the cross-lane ops
    const int64_t token = base + tid / G;
    const bool live = token < M;
    const T* row = logits + (live ? token : 0) * E;
    gate_token<G, VPL>([&](int e) { return to_float(row[e]); }, live, E, topk, renorm, w_out + token * topk,
                       ids_out + token * topk);
  }
  __threadfence_block();
  __syncthreads();  // the ids written above are read back below by other lanes of this workgroup
  const int64_t n = M * topk;
  const int64_t lo = min64(n, static_cast<int64_t>(wave) * seg_len);
  const int64_t hi = min64(n, lo + seg_len);
  segment_histogram(ids_out, lo, hi, E, lane, &table[wave * E]);
  __syncthreads();
  for (int e = tid; e < E; e += kSmallThreads) {
    int running = 0;
    for (int w = 0; w < kSmallWaves; ++w) {
      const int c = table[w * E + e];
      table[w * E + e] = running;
      running += c;
    }
    total[e] = running;
  }
  __syncthreads();
  if (wave == 0) scan_padded_totals(total, start, E, B, lane);
  __syncthreads();
  for (int i = tid; i < kSmallWaves * E; i += kSmallThreads) table[i] += start[i % E];
  write_block_table(total, start, E, B, n, sorted_len, tid, kSmallThreads, sorted, expert_ids, npost_out);
  __syncthreads();
  segment_scatter(ids_out, lo, hi, E, bits_for(E), lane, &table[wave * E], sorted);
}

// ---------------------------------------------------------------- large path
// counts is [E][S]: after align_segscan_kernel, counts[e][s] is the offset of
// segment s inside expert e's run and totals[e] the length of the run.
template <typename IdT>
__global__ __launch_bounds__(kSegThreads) void align_count_kernel(
    const IdT* __restrict__ ids, int64_t n, int E, int seg_len, int S, int* __restrict__ counts) {
  extern __shared__ int hist[];  // [kSegWaves][E]
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int seg = blockIdx.x * kSegWaves + wave;
  int* mine = hist + wave * E;
  for (int e = lane; e < E; e += kWave) mine[e] = 0;
  __builtin_amdgcn_wave_barrier();
  if (seg >= S) return;
  const int64_t lo = static_cast<int64_t>(seg) * seg_len;
  const int64_t hi = min64(n, lo + seg_len);
  segment_histogram(ids, lo, hi, E, lane, mine);
  __builtin_amdgcn_wave_barrier();
  for (int e = lane; e < E; e += kWave) counts[static_cast<int64_t>(e) * S + seg] = mine[e];
}

// One workgroup per expert: exclusive scan of that expert's per-segment counts
// (in place) and its total.
__global__ __launch_bounds__(kSegThreads) void align_segscan_kernel(int* __restrict__ counts,
                                                                     int* __restrict__ totals, int S) {
  __shared__ int wave_sum[kSegWaves];
  const int e = blockIdx.x, tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  int* row = counts + static_cast<int64_t>(e) * S;
  int running = 0;
  for (int base = 0; base < S; base += kSegThreads) {
    const int s = base + tid;
    const int c = (s < S) ? row[s] : 0;
    const int incl = wave_inclusive_scan(c, lane);
    if (lane == kWave - 1) wave_sum[wave] = incl;
    __syncthreads();
    int before = 0, all = 0;
#pragma unroll
    for (int w = 0; w < kSegWaves; ++w) {
      const int ws = wave_sum[w];
      before += (w < wave) ? ws : 0;
      all += ws;
    }
    if (s < S) row[s] = running + before + incl - c;
    running += all;
    __syncthreads();
  }
  if (tid == 0) totals[e] = running;
}

// Scatter pass.  Every workgroup rebuilds the run starts from the E totals (cheap),
// workgroup e < E also writes expert e's block table and padding, workgroup 0 the
// tail and the padded length; then each wavefront places its segment.
template <typename IdT>
__global__ __launch_bounds__(kSegThreads) void align_scatter_kernel(
    const IdT* __restrict__ ids, int64_t n, int E, int B, int seg_len, int S, int64_t sorted_len,
    const int* __restrict__ counts, const int* __restrict__ totals, int32_t* __restrict__ sorted,
    int32_t* __restrict__ expert_ids, int32_t* __restrict__ npost_out) {
  extern __shared__ int hist[];  // [kSegWaves][E]
  __shared__ int start[kMaxE + 1];
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  if (wave == 0) scan_padded_totals(totals, start, E, B, lane);
  __syncthreads();
  if (static_cast<int>(blockIdx.x) < E) {
    const int e = blockIdx.x;
    for (int b = start[e] / B + tid; b < start[e + 1] / B; b += kSegThreads) expert_ids[b] = e;
    for (int s = start[e] + totals[e] + tid; s < start[e + 1]; s += kSegThreads) sorted[s] = static_cast<int32_t>(n);
  }
  if (blockIdx.x == 0) {
    for (int64_t s = start[E] + tid; s < sorted_len; s += kSegThreads) sorted[s] = static_cast<int32_t>(n);
    if (tid == 0) npost_out[0] = start[E];
  }
  const int seg = blockIdx.x * kSegWaves + wave;
  if (seg >= S) return;
  int* mine = hist + wave * E;
  for (int e = lane; e < E; e += kWave) mine[e] = start[e] + counts[static_cast<int64_t>(e) * S + seg];
  __builtin_amdgcn_wave_barrier();
  const int64_t lo = static_cast<int64_t>(seg) * seg_len;
  const int64_t hi = min64(n, lo + seg_len);
  segment_scatter(ids, lo, hi, E, bits_for(E), lane, mine, sorted);
}

// ---------------------------------------------------------------- large path, two launches
// The per-expert scan over segments costs a launch of its own only because every scatter workgroup needs
// (a) each expert's total and (b) the pairs of each expert in the segments before its own.  Here a count
// workgroup covers 16 segments, leaves each segment's offset INSIDE the workgroup in counts[e][seg] and the
// workgroup's sums in wgcnt[b][e]; a scatter workgroup then gets (a) and (b) from one pass over the NB x E
// workgroup sums (6144 values for 64 experts and 393 216 pairs: six loads per thread, summed with integer
// LDS atomics, so the order does not matter).  Used while NB x E stays small.
constexpr int kSeg2Threads = 1024;
constexpr int kSeg2Waves = kSeg2Threads / kWave;
constexpr int64_t kTwoLevelMaxEntries = 16384;

template <typename IdT>
__global__ __launch_bounds__(kSeg2Threads) void align_count2_kernel(
    const IdT* __restrict__ ids, int64_t n, int E, int seg_len, int S, int* __restrict__ counts,
    int* __restrict__ wgcnt) {
  extern __shared__ int hist[];  // [kSeg2Waves][E]
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int seg0 = blockIdx.x * kSeg2Waves, seg = seg0 + wave;
  int* mine = hist + wave * E;
  for (int e = lane; e < E; e += kWave) mine[e] = 0;
  __builtin_amdgcn_wave_barrier();
  if (seg < S) {
    const int64_t lo = static_cast<int64_t>(seg) * seg_len;
    const int64_t hi = min64(n, lo + seg_len);
    segment_histogram(ids, lo, hi, E, lane, mine);
  }
  __syncthreads();
  for (int i = tid; i < E * kSeg2Waves; i += kSeg2Threads) {  // (expert, segment of this workgroup)
    const int e = i % E, w = i / E;
    int before = 0;
    for (int v = 0; v < w; ++v) before += hist[v * E + e];
    if (seg0 + w < S) counts[static_cast<int64_t>(e) * S + seg0 + w] = before;
    if (w == kSeg2Waves - 1) wgcnt[static_cast<int64_t>(blockIdx.x) * E + e] = before + hist[w * E + e];
  }
}

template <typename IdT>
__global__ __launch_bounds__(kSeg2Threads) void align_scatter2_kernel(
    const IdT* __restrict__ ids, int64_t n, int E, int B, int seg_len, int S, int NB, int64_t sorted_len,
    const int* __restrict__ counts, const int* __restrict__ wgcnt, int32_t* __restrict__ sorted,
    int32_t* __restrict__ expert_ids, int32_t* __restrict__ npost_out) {
  extern __shared__ int hist[];  // [kSeg2Waves][E]
  __shared__ int start[kMaxE + 1];
  __shared__ int total[kMaxE];
  __shared__ int before[kMaxE];
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int wg = blockIdx.x;
  // this wavefront's segment: its first ids and its offsets inside the workgroup are asked for now, so that
  // their latency passes together with that of the workgroup sums below
  const int seg = wg * kSeg2Waves + wave;
  const int64_t lo = min64(n, static_cast<int64_t>(seg) * seg_len);
  const int64_t hi = seg < S ? min64(n, lo + seg_len) : lo;
  int first[kScatterPF];
  segment_ids(ids, lo, hi, lane, first);
  const int in_wg0 = (seg < S && lane < E) ? counts[static_cast<int64_t>(lane) * S + seg] : 0;
  for (int e = tid; e < E; e += kSeg2Threads) total[e] = before[e] = 0;
  __syncthreads();
  for (int i = tid; i < E * NB; i += kSeg2Threads) {  // expert e: all pairs, and the pairs in the workgroups before this one
    const int b = i / E, e = i % E;
    const int c = wgcnt[i];
    if (c != 0) {
      atomicAdd(&total[e], c);
      if (b < wg) atomicAdd(&before[e], c);
    }
  }
  __syncthreads();
  if (wave == 0) scan_padded_totals(total, start, E, B, lane);
  __syncthreads();
  if (wg < E) {
    const int e = wg;
    for (int b = start[e] / B + tid; b < start[e + 1] / B; b += kSeg2Threads) expert_ids[b] = e;
    for (int s = start[e] + total[e] + tid; s < start[e + 1]; s += kSeg2Threads) sorted[s] = static_cast<int32_t>(n);
  }
  if (wg == 0) {
    for (int64_t s = start[E] + tid; s < sorted_len; s += kSeg2Threads) sorted[s] = static_cast<int32_t>(n);
    if (tid == 0) npost_out[0] = start[E];
  }
  if (seg >= S) return;
  int* mine = hist + wave * E;
  if (lane < E) mine[lane] = start[lane] + before[lane] + in_wg0;
  for (int e = lane + kWave; e < E; e += kWave) mine[e] = start[e] + before[e] + counts[static_cast<int64_t>(e) * S + seg];
  __builtin_amdgcn_wave_barrier();
  segment_scatter(ids, lo, hi, E, bits_for(E), lane, mine, sorted, first);
}

bool use_small_path(int64_t n, int E) { return n <= kSmallMaxN && E <= kSmallMaxE; }

int large_seg_len(int64_t n) {
  const int64_t want = round_up(ceil_div(n, 2048), kWave);
  return static_cast<int>(want < 256 ? 256 : want);
}

template <typename IdT>
int run(const void* ids_v, int64_t n, int E, int B, int32_t* sorted, int32_t* expert_ids,
        int32_t* npost, void* ws, hipStream_t st) {
  const IdT* ids = static_cast<const IdT*>(ids_v);
  const int64_t sorted_len = n + static_cast<int64_t>(E) * (B - 1);
  if (use_small_path(n, E)) {
    int seg_len = static_cast<int>(round_up(ceil_div(n, kSmallWaves), kWave));
    if (seg_len == 0) seg_len = kWave;
    hipLaunchKernelGGL((align_small_kernel<IdT>), dim3(1), dim3(kSmallThreads), 0, st, ids, n, E, B,
                       seg_len, sorted_len, sorted, expert_ids, npost);
    return check_launch("align_small_kernel");
  }
  const int seg_len = large_seg_len(n);
  const int S = static_cast<int>(n > 0 ? ceil_div(n, seg_len) : 1);
  int* counts = static_cast<int*>(ws);
  int* run_start = counts + static_cast<int64_t>(E) * S;
  const unsigned blocks = static_cast<unsigned>(ceil_div(S, kSegWaves));
  const unsigned scatter_blocks = blocks > static_cast<unsigned>(E) ? blocks : static_cast<unsigned>(E);
  const size_t lds = sizeof(int) * kSegWaves * E;
  const int NB = static_cast<int>(ceil_div(S, kSeg2Waves));
  if (static_cast<int64_t>(E) * NB <= kTwoLevelMaxEntries && E <= 512) {  // count (+ workgroup sums), scatter: two launches
    const size_t lds2 = sizeof(int) * kSeg2Waves * E;
    int* wgcnt = counts + static_cast<int64_t>(E) * S;
    hipLaunchKernelGGL((align_count2_kernel<IdT>), dim3(NB), dim3(kSeg2Threads), lds2, st, ids, n, E, seg_len, S, counts, wgcnt);
    hipLaunchKernelGGL((align_scatter2_kernel<IdT>), dim3(NB > E ? NB : E), dim3(kSeg2Threads), lds2, st, ids, n, E, B,
                       seg_len, S, NB, sorted_len, counts, wgcnt, sorted, expert_ids, npost);
    return check_launch("align kernels");
  }
  hipLaunchKernelGGL((align_count_kernel<IdT>), dim3(blocks), dim3(kSegThreads), lds, st, ids, n, E,
                     seg_len, S, counts);
  hipLaunchKernelGGL(align_segscan_kernel, dim3(E), dim3(kSegThreads), 0, st, counts, run_start, S);
  hipLaunchKernelGGL((align_scatter_kernel<IdT>), dim3(scatter_blocks), dim3(kSegThreads), lds, st, ids, n, E, B,
                     seg_len, S, sorted_len, counts, run_start, sorted, expert_ids, npost);
  return check_launch("align kernels");
}

template <typename T, int G, int VPL>
void launch_route_align(const void* logits, int64_t M, int E, int topk, int renorm, int B, int64_t sorted_len,
                        float* w, int32_t* ids, int32_t* sorted, int32_t* expert_ids, int32_t* npost, RowQuant rq,
                        hipStream_t st) {
  int seg_len = static_cast<int>(round_up(ceil_div(M * topk, kSmallWaves), kWave));
  if (seg_len == 0) seg_len = kWave;
  const unsigned grid = 1 + (rq.x ? static_cast<unsigned>(ceil_div(M, kSmallWaves)) : 0u);
  hipLaunchKernelGGL((route_align_small_kernel<T, G, VPL>), dim3(grid), dim3(kSmallThreads), 0, st,
                     static_cast<const T*>(logits), M, E, topk, renorm, B, seg_len, sorted_len, w, ids, sorted,
                     expert_ids, npost, rq);
}

template <typename T>
void dispatch_route_align(const void* logits, int64_t M, int E, int topk, int renorm, int B, int64_t sorted_len,
                          float* w, int32_t* ids, int32_t* sorted, int32_t* expert_ids, int32_t* npost, RowQuant rq,
                          hipStream_t st) {
#define FR_RA(G, VPL) launch_route_align<T, G, VPL>(logits, M, E, topk, renorm, B, sorted_len, w, ids, sorted, expert_ids, npost, rq, st)
  if (E <= 1) FR_RA(1, 1);
  else if (E <= 2) FR_RA(2, 1);
  else if (E <= 4) FR_RA(4, 1);
  else if (E <= 8) FR_RA(8, 1);
  else if (E <= 16) FR_RA(16, 1);
  else if (E <= 32) FR_RA(32, 1);
  else if (E <= 64) FR_RA(64, 1);
  else if (E <= 128) FR_RA(64, 2);
  else FR_RA(64, 4);
#undef FR_RA
}

}  // namespace

// Gating and routing arrays in one launch for small batches; false when the shape is
// outside what one workgroup should do (the caller then runs the two stages separately).
// (one workgroup gates and sorts 1024 pairs in 10.5 us; from there on the gating kernel spread over the CUs
// plus the one-workgroup sort are faster: 8.9 us + a launch gap at 1024 pairs, 12.6 against 26.8 us at 4096)
bool route_align_fits(int64_t M, int E, int topk) {
  return M >= 1 && M * topk <= kRouteAlignMaxN && use_small_path(M * topk, E) && M * E <= 16384 && topk <= E;
}
int route_align_small(const void* logits, int logits_dtype, int64_t M, int E, int topk, int renorm, int block,
                      float* w, int32_t* ids, int32_t* sorted, int32_t* expert_ids, int32_t* npost,
                      const void* qx, int64_t qK, void* qq, float* qscale, hipStream_t st) {
  const int64_t sorted_len = M * topk + int64_t(E) * (block - 1);
  const RowQuant rq = {static_cast<const bf16_t*>(qx), static_cast<unsigned char*>(qq), qscale, static_cast<int>(qK)};
  switch (logits_dtype) {
    case FR_F32: dispatch_route_align<float>(logits, M, E, topk, renorm, block, sorted_len, w, ids, sorted, expert_ids, npost, rq, st); break;
    case FR_F16: dispatch_route_align<f16_t>(logits, M, E, topk, renorm, block, sorted_len, w, ids, sorted, expert_ids, npost, rq, st); break;
    case FR_BF16: dispatch_route_align<bf16_t>(logits, M, E, topk, renorm, block, sorted_len, w, ids, sorted, expert_ids, npost, rq, st); break;
    default: return fail(FR_E_DTYPE, "route_align_small: logits dtype %d not in {f32, f16, bf16}", logits_dtype);
  }
  return check_launch("route_align_small_kernel");
}

}  // namespace fr

extern "C" int64_t fr_moe_align_workspace_bytes(int64_t n, int E) {
  using namespace fr;
  if (n < 0 || E < 1 || E > kMaxE) return -1;
  if (use_small_path(n, E)) return 0;
  const int64_t S = n > 0 ? ceil_div(n, large_seg_len(n)) : 1;
  // [E][S] counts, then E totals (three launches) or [E][ceil(S / 4)] workgroup sums (two launches)
  return static_cast<int64_t>(sizeof(int)) * (static_cast<int64_t>(E) * S + static_cast<int64_t>(E) * (ceil_div(S, kSegWaves) + 1));
}

extern "C" int fr_moe_align(const void* topk_ids, int ids_dtype, int64_t n, int E, int block,
                            int32_t* sorted_token_ids, int32_t* expert_ids,
                            int32_t* num_tokens_post_pad, void* workspace, int64_t workspace_bytes,
                            void* stream) {
  using namespace fr;
  FR_REQUIRE(n >= 0 && n <= (int64_t(1) << 30), FR_E_SHAPE, "fr_moe_align: n=%lld outside [0, 2^30]", (long long)n);
  FR_REQUIRE(E >= 1 && E <= kMaxE, FR_E_SHAPE, "fr_moe_align: E=%d outside [1, %d]", E, kMaxE);
  FR_REQUIRE(block >= 1 && block <= 4096, FR_E_SHAPE, "fr_moe_align: block=%d outside [1, 4096]", block);
  FR_REQUIRE(n + int64_t(E) * block < (int64_t(1) << 31), FR_E_SHAPE, "fr_moe_align: padded length overflows int32");
  FR_REQUIRE(expert_ids && num_tokens_post_pad && (sorted_token_ids || n + int64_t(E) * (block - 1) == 0), FR_E_NULL, "fr_moe_align: null output pointer");
  FR_REQUIRE(n == 0 || topk_ids, FR_E_NULL, "fr_moe_align: null topk_ids");
  FR_REQUIRE(ids_dtype == FR_I32 || ids_dtype == FR_I64, FR_E_DTYPE, "fr_moe_align: ids dtype %d not in {i32, i64}", ids_dtype);
  const int64_t need = fr_moe_align_workspace_bytes(n, E);
  FR_REQUIRE(need == 0 || (workspace && workspace_bytes >= need), FR_E_WORKSPACE,
             "fr_moe_align: workspace %lld < %lld bytes", (long long)workspace_bytes, (long long)need);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (ids_dtype == FR_I32) return run<int32_t>(topk_ids, n, E, block, sorted_token_ids, expert_ids, num_tokens_post_pad, workspace, st);
  return run<int64_t>(topk_ids, n, E, block, sorted_token_ids, expert_ids, num_tokens_post_pad, workspace, st);
}
