// Persistent form of the direct-to-LDS grouped GEMM: one workgroup per resident slot walks
// several tiles, and the LDS ring never drains between them.  While the last K tiles of
// one output tile are being multiplied, the ring is already refilled with the first K
// tiles of the workgroup's next output tile (whose routing data was fetched a whole tile
// earlier), so the start-up of a tile (dependent loads of block table, sorted ids, first
// operand tiles) and the memory side of its epilogue hide behind MFMA work.  It pays for
// tiles that leave room for one workgroup per CU only (256 x 256); smaller tiles already
// overlap one workgroup's start-up with the other's MFMAs.
//
// Same tile shapes, LDS layout, swizzle, fragment double buffering, barrier placement and
// epilogues as moe_gemm_kernel (STAGES >= 2, refill in one group); see there.
//
// Tail split.  The tiles of an XCD rarely fill whole rounds of its workgroups: with 70 tiles
// for 32 workgroups the third round keeps 6 of them busy.  Given scratch (GemmArgs::tail_ws)
// the tiles of that last round are split along K into as many slices as there are idle
// workgroups per tile (at most kTailMaxSplit, each at least kTailMinSlice K tiles long); a
// slice is one more work unit of its workgroup, its fp32 accumulators go to the scratch as
// they are, and tail_fixup_kernel sums the slices of a tile in slice order and applies the
// epilogue.  Nothing waits on another workgroup and the result does not depend on timing.
#pragma once
#include "moe_gemm_kernel.h"

namespace fr {

constexpr int kTailMaxSplit = 8;    // K slices per tile of the last round, at most
constexpr int kTailMinSlice = 8;    // K tiles per slice, at least
constexpr int kTailMinTiles = 32;   // K tiles per output tile below which the split is not worth its fix-up launch
constexpr int kTailUnits = 256;     // workgroups (= slice buffers in the scratch), at most

// Tiles of one XCD: `rounds` whole rounds of the XCD's `nper` workgroups and `rest` tiles after them (from tile
// `tail_base` on), each cut into `slices` K slices.  base: first tile of a contiguous share, or -1 (dealt by rounds).
struct XcdSchedule {
  int base, tail_base, rounds, rest, slices;
};
// by_rounds: round j gives XCD x the nper consecutive tiles from (j * 8 + x) * nper on, so every XCD sees every
// region of the walk; the tiles after the last whole round are dealt to the XCDs in contiguous shares.  Otherwise
// every XCD takes one contiguous eighth of the tiles.  One eighth each left the XCDs up to 20 % apart in the
// compute-bound regime (down projection at 4096 tokens: 1.67 M cycles on the slowest XCD, 1.37 M on the fastest);
// dealt by rounds the layer is 1.8-3.6 % faster from 1024 tokens up.  With about one token block per expert the
// kernel streams every weight tile once from HBM, and there an XCD that stays inside one expert's weights is
// faster (256 tokens: 357 against 412 us for the gate/up GEMM), so the rule follows the blocks per expert.
__device__ __forceinline__ bool schedule_by_rounds(int token_blocks, int num_experts) { return 2 * token_blocks >= 5 * num_experts; }
__device__ __forceinline__ XcdSchedule xcd_schedule(int total, int nper, int xcd, int k_tiles, bool split_tail, bool by_rounds) {
  XcdSchedule s;
  if (by_rounds) {
    const int grid = nper * 8;
    s.rounds = total / grid;
    const int rest_all = total - s.rounds * grid, per = rest_all >> 3, rem = rest_all & 7;
    s.tail_base = s.rounds * grid + xcd * per + (xcd < rem ? xcd : rem);
    s.rest = per + (xcd < rem ? 1 : 0);
    s.base = -1;
  } else {
    const int per = total >> 3, rem = total & 7, count = per + (xcd < rem ? 1 : 0);
    s.base = xcd * per + (xcd < rem ? xcd : rem);
    s.rounds = count / nper;
    s.rest = count - s.rounds * nper;
    s.tail_base = s.base + s.rounds * nper;
  }
  s.slices = 1;
  if (split_tail && s.rest > 0) {
    // Worth it when the time saved, about (0.7 - 1/slices) of a tile's K loop, exceeds the
    // fix-up's: one fp32 tile written and read back per slice plus a launch, in units of
    // about a twelfth of a K tile's time (measured: 10 tiles in 3 slices of 21 K tiles each
    // break even or gain, 6 tiles in 5 slices of 45 gain a fifth of the kernel's time).
    const int sl = min(min(nper / s.rest, k_tiles / kTailMinSlice), kTailMaxSplit);
    if (sl >= 2 && k_tiles * (7 * sl - 10) >= 3 * sl * (s.rest * sl + 10)) s.slices = sl;
  }
  return s;
}
// tile j of workgroup `loc` of XCD `xcd` among the whole rounds
__device__ __forceinline__ int xcd_round_tile(const XcdSchedule& s, int nper, int xcd, int loc, int j) {
  return s.base < 0 ? (j * 8 + xcd) * nper + loc : s.base + j * nper + loc;
}
// Walk order of the tiles.  The token blocks of one expert are consecutive (the routing sort is by
// expert), and only they use that expert's weight tiles.  Tiles are therefore ordered expert by
// expert; an expert's run of blocks is cut into equal chunks of at most group_t blocks and a chunk
// is walked block-fastest over all feature tiles.  Consecutive tiles - the ones an XCD's workgroups
// hold at any moment - then share one expert's weight tiles and a few token blocks, and a weight
// tile is fetched by one chunk only (groups of a fixed number of blocks straddle experts and fetch
// two experts' tiles each: measured 4.6 GB through L2 per launch against 2.1 GB of operands).
constexpr int kWalkTable = 1024;   // ints of LDS for the walk table: with the 160-row tile's ring (159744 bytes) exactly the 160 KB of a CU
constexpr int kMaxExperts = kWalkTable - 2;  // experts the persistent form takes (the routing entry points take 1024: those launches run the plain kernel)
constexpr int kChunkBlocks = 8;    // token blocks per chunk, at most (measured 4 / 8 / 16: 1675 / 1648 / 1640 us at M=4096,
                                   // 8 and 12 best at M=16384)
// off[e] = first token block of expert e among the nt real blocks, off[E] = nt; off[kMaxExperts + 1] = 1
// if expert_ids does not ascend (routing arrays of another producer, legal for the op-level GEMM): then
// every tile takes the plain row-major walk, since the table describes no partition of the blocks.
__device__ __forceinline__ void expert_block_offsets(const GemmArgs& a, int nt, int* off, int tid, int nthreads) {
  if (tid == 0) off[kMaxExperts + 1] = 0;
  for (int e = tid; e <= a.num_experts; e += nthreads) {
    int lo = 0, hi = nt;
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (a.expert_ids[mid] < e) lo = mid + 1;
      else hi = mid;
    }
    off[e] = lo;
  }
  __syncthreads();
  for (int b = tid + 1; b < nt; b += nthreads)
    if (a.expert_ids[b] < a.expert_ids[b - 1]) off[kMaxExperts + 1] = 1;
  __syncthreads();
}
// A tile's place among the tiles that share its weight tile: the `count` token blocks of its chunk, of which it
// is number `index` (1 and 0 without a walk table).
struct TileShare {
  int count, index;
};
__device__ __forceinline__ void tile_coords(const GemmArgs& a, const int* off, int lin, int& pid_t, int& pid_f,
                                            int& expert, TileShare* share = nullptr) {
  const int F = a.num_f_tiles;
  if (off[kMaxExperts + 1]) {
    pid_t = lin / F;
    pid_f = lin % F;
    expert = a.expert_ids[pid_t];
    if (share) *share = TileShare{1, 0};
    return;
  }
  expert = a.expert_ids[lin / F];  // lin / F is one of the expert's blocks: its tiles are [off[e] * F, off[e + 1] * F)
  const int first = off[expert], len = off[expert + 1] - first;
  const int chunks = (len + a.group_t - 1) / a.group_t, base = len / chunks, rem = len - base * chunks;
  int q = lin - first * F;
  const int big = rem * (base + 1) * F;  // the first rem chunks hold one block more
  int gsz, start;
  if (q < big) {
    gsz = base + 1;
    const int c = q / (gsz * F);
    q -= c * gsz * F;
    start = first + c * gsz;
  } else {
    q -= big;
    gsz = base;
    const int c = q / (gsz * F);
    q -= c * gsz * F;
    start = first + rem * (base + 1) + c * gsz;
  }
  pid_t = start + q % gsz;
  pid_f = q / gsz;
  if (share) *share = TileShare{gsz, q % gsz};
}
// Tile column of accumulator tile j of feature wavefront wf (= row of the weight tile in LDS).
template <typename C, int EPI>
__device__ __forceinline__ int acc_tile_col(int wf, int j) {
  if constexpr (EPI == EPI_SILU) {
    constexpr int HJ = C::JF / 2;  // first half of the wave's tiles: gate, second: up
    return (j < HJ) ? wf * (C::TF / 2) + j * C::TILE : C::BF / 2 + wf * (C::TF / 2) + (j - HJ) * C::TILE;
  } else {
    return wf * C::TF + j * C::TILE;
  }
}
// fp32 accumulators of one K slice, as they are, to the slice's [BT][BF] buffer
template <typename C, int EPI, bool AG = false, typename AccT>
__device__ __forceinline__ void tail_store(float* tile, AccT (&acc)[C::JF][C::IT], int wt, int wf, int frow, int kgrp) {
  constexpr int GROUPS = ((C::TILE == 32) ? 16 : 4) / 4;
#pragma unroll
  for (int i = 0; i < C::IT; ++i) {
    float* row = tile + (wt * C::TT + i * C::TILE + frow) * C::BF;
#pragma unroll
    for (int j = 0; j < C::JF; ++j) {
      const AccT ca = AG ? acc_fetch(acc[j][i]) : acc[j][i];
#pragma unroll
      for (int g = 0; g < GROUPS; ++g) {
        const f32x4 o = {ca[g * 4 + 0], ca[g * 4 + 1], ca[g * 4 + 2], ca[g * 4 + 3]};
        *reinterpret_cast<f32x4*>(row + acc_tile_col<C, EPI>(wf, j) + g * 8 + kgrp * 4) = o;
        if constexpr (AG) __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
}

#ifdef FR_PROF  // measurement builds: cycle counts of wavefront 0 of every workgroup (K loops / epilogues / total / K tiles)
#define FR_PROF_PARAM , long long* fr_prof_buf
#define FR_PROF_ARG , fr_prof_host()
inline long long*& fr_prof_host() { static long long* p = nullptr; return p; }
#else
#define FR_PROF_PARAM
#define FR_PROF_ARG
#endif
template <typename T, typename C, int EPI>
__global__ __launch_bounds__(C::NT, C::MINB) void moe_gemm_persistent_kernel(const GemmArgs a FR_PROF_PARAM) {
#if defined(__HIP_DEVICE_COMPILE__)  // buffer resources and LDS-DMA builtins exist in the device pass only
  typedef Elem<T> E;
  typedef typename std::conditional<C::TILE == 32, f32x16, f32x4>::type acc_t;
  typedef __attribute__((address_space(3))) void* lptr_t;
  constexpr int BT = C::BT, BF = C::BF, CPR = C::CPR, FC = E::FC;
  constexpr int EPC = 16 / static_cast<int>(sizeof(T));
  constexpr int BK = C::BKB / static_cast<int>(sizeof(T));
  constexpr int KS = CPR / (C::KGROUPS * FC);
  constexpr int ACC_N = (C::TILE == 32) ? 16 : 4;
  constexpr int S = C::STAGES, NW = C::NW, XIW = C::XIW, WIW = C::WIW, IW = C::IW, NLI = XIW + WIW;
  constexpr int NM = C::JF * C::IT, RD_AT = (NM + 1) / 2 - 1;
  // one fragment buffer for fp8 (8-register fragments) and for the tiles on 16x16 MFMAs (nine to twelve fragments
  // per K-step next to 64 to 128 accumulators: each fragment is read again as soon as its last MFMA of the K-step
  // is issued; measured against two buffers: 256 rows needed it to fit, 160 rows -0.4 .. -1.3 %, 128 rows 0 .. -1 %),
  // two otherwise
  constexpr bool SINGLE = E::SCALED || C::TILE == 16;
  // fp8 epilogue: scales fetched up front where the registers allow it (the 256-row tile keeps 128 accumulators
  // and two address sets alive: measured 603 us with, 589 us without for the down projection at M = 4096; the
  // 128-row tile gains 2-5 %)
  constexpr bool HOIST = BT < 256;
  static_assert(S >= 2 && C::SPREAD <= 1, "persistent form: ring of at least two slots, refill in one group");
  static_assert(SINGLE || KS % 2 == 0, "fragment double buffering needs an even number of K-steps per tile");
  static_assert((S - 1) * NLI <= 63, "vmcnt budget");
  static_assert(EPI != EPI_SILU || C::JF % 2 == 0, "gate and up tiles must pair up inside a wave");
  static_assert(IW >= 1 && NW % IW == 0, "issue width");

  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  u32x4* lds = reinterpret_cast<u32x4*>(lds_raw);
  constexpr int WBASE = S * C::XCH;  // LDS map (16-byte units): X slots first, then W slots

  // ---- schedule ---------------------------------------------------------------
  // The real tile count is dealt to the 8 XCDs (workgroup id mod 8) - round by round, or one contiguous eighth
  // each (xcd_schedule) -; the workgroups of one XCD take consecutive tiles, so at any moment they work on
  // a few token blocks of one expert x consecutive feature tiles (tile_coords), shared in that XCD's L2.
  // Work unit j of a workgroup: tile j of its round-robin walk over all K tiles, or, after the
  // whole rounds, one K slice of a tile of the last round.
  const int npost = a.npost[0];
  const int nt = min(npost / BT, a.num_t_blocks);
  const int total = nt * a.num_f_tiles;
  const int xcd = blockIdx.x & 7, nper = gridDim.x >> 3, loc = blockIdx.x >> 3;
  const int split = blockIdx.y;
  const int k0 = split * a.k_per_split;
  const int k_all = min(a.k_per_split, a.K - k0) / BK;  // K tiles of a whole unit, >= S + 2 (checked by the launcher)
  const XcdSchedule xs = xcd_schedule(total, nper, xcd, k_all, a.tail_ws != nullptr, schedule_by_rounds(nt, a.num_experts));
  const int n_units = xs.rounds + (loc < xs.rest * xs.slices ? 1 : 0);
  if (n_units == 0) return;
  __shared__ int expert_off[kWalkTable];
  expert_block_offsets(a, nt, expert_off, threadIdx.x, C::NT);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wt = wave / C::WF, wf = wave % C::WF;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const bool issuer = wave_u < NW / IW;
  const int wstep = a.w_tiled ? (C::BKB / kTileBytes) * kTilePiece : C::BKB;  // bytes from one K tile of W to the next
  const T* X = static_cast<const T*>(a.X);

  // unit j_ -> tile coordinates, first K tile kb_ and K tile count kn_, slice buffer tu_ (-1: a whole tile)
#define FR_UNIT(j_, pt_, pf_, ex_, kb_, kn_, tu_)                                              \
  {                                                                                            \
    int lin_;                                                                                  \
    if ((j_) < xs.rounds) {                                                                    \
      lin_ = xcd_round_tile(xs, nper, xcd, loc, (j_));                                         \
      kb_ = 0; kn_ = k_all; tu_ = -1;                                                          \
    } else {                                                                                   \
      const int t_ = loc % xs.rest, s_ = loc / xs.rest;                                        \
      lin_ = xs.tail_base + t_;                                                   \
      kb_ = s_ * k_all / xs.slices;                                                            \
      kn_ = (s_ + 1) * k_all / xs.slices - kb_;                                                \
      tu_ = xs.slices > 1 ? s_ * xs.rest + t_ : -1;                                            \
    }                                                                                          \
    tile_coords(a, expert_off, lin_, pt_, pf_, ex_);                                           \
  }
  // rows of the load slots this wavefront issues: load index ih -> tile row
  // (ROWS_: rows of the tile.  With an odd number of loads per issuing wavefront the last index lies beyond the tile
  // for the wavefronts that issue nothing; they only share the address code, and their row is clamped into the tile)
#define FR_SLOT_ROW(ih_, rr_, c_, ROWS_)                                           \
  const int vw_ = (wave_u + ((ih_) % IW) * (NW / IW)) % NW;                        \
  const int slot_ = (((ih_) / IW) * NW + vw_) * kWave + lane;                      \
  const int rr_ = min(slot_ / CPR, (ROWS_) - 1), c_ = swizzle<CPR>(rr_, slot_ % CPR);
  auto w_src_row = [&](int pf, int rr) -> int {
    if constexpr (EPI == EPI_SILU) {
      const int half = rr / (BF / 2), f = pf * (BF / 2) + rr % (BF / 2);
      return half * a.N + (f < a.N ? f : a.N - 1);
    } else {
      const int f = pf * BF + rr;
      return f < a.N ? f : a.N - 1;
    }
  };

  // ---- per-lane fragment rows ---------------------------------------------------
  const int frow = lane % C::TILE, kgrp = lane / C::TILE;
  // All fragment rows of a lane lie a multiple of 16 rows apart, which leaves the swizzle key unchanged: one
  // offset and one key per operand, the fragments at compile-time distances from them (immediate offsets of
  // the LDS reads).
  static_assert(C::TILE % 16 == 0 && (BF / 2) % 16 == 0 && C::TF % 16 == 0 && C::TT % 16 == 0, "fragment rows 16 apart");
  const int xrow0 = wt * C::TT + frow, wrow0 = acc_tile_col<C, EPI>(wf, 0) + frow;
  const int xoff0 = xrow0 * CPR, xkey0 = swizzle<CPR>(xrow0, 0);
  const int woff0 = WBASE + wrow0 * CPR, wkey0 = swizzle<CPR>(wrow0, 0);
#define FR_XD(i_) ((i_) * C::TILE * CPR)
#define FR_WD(j_) ((acc_tile_col<C, EPI>(0, (j_)) - acc_tile_col<C, EPI>(0, 0)) * CPR)
  acc_t acc[C::JF][C::IT];
  u32x4 xf[2][C::IT][FC], wfr[2][C::JF][FC];

  // ---- address sets: A = tile being multiplied, B = the workgroup's next tile --------
  int pid_t, pid_f, expert, kb, kn, tu;  // current unit: tile, first K tile and K tile count, slice buffer
  int n_pid_t = 0, n_pid_f = 0, n_expert = 0, n_kb = 0, n_kn = 0, n_tu = -1;
  int n_sid[XIW];  // sorted ids of the next tile's load rows, fetched a tile ahead
  unsigned xsrcA[XIW], wsrcA[WIW], xsrcB[XIW], wsrcB[WIW];
  __amdgpu_buffer_rsrc_t xrsA, wrsA, xrsB, wrsB;
  // the expert of the tile has ONE token block: each of its weight tiles is read by one tile only, and marked
  // non-temporal the stream does not displace the token rows and its own neighbours in L2
  bool ntA = false, ntB = false;
  constexpr bool NTW = BT < 256;  // the 256-row tiles have no register to spare for the second form of the loads
#define FR_MAKE_SET(pt_, pf_, ex_, kb_, SIDOF, xsrc_, wsrc_, xrs_, wrs_, nt_)                                   \
  {                                                                                                          \
    const int64_t xrow0_ = a.top_k > 0 ? 0 : static_cast<int64_t>(pt_) * BT;                                 \
    const int64_t kfirst_ = k0 + static_cast<int64_t>(kb_) * BK;                                             \
    xrs_ = uniform_rsrc(X + xrow0_ * a.ldx, a.x_span ? a.x_span : 0xFFFFFFFFu);                              \
    wrs_ = uniform_rsrc(static_cast<const T*>(a.W) + static_cast<int64_t>(ex_) * a.w_expert_stride);         \
    nt_ = NTW && !expert_off[kMaxExperts + 1] && expert_off[(ex_) + 1] - expert_off[ex_] == 1;               \
    _Pragma("unroll") for (int ih = 0; ih < XIW; ++ih) {                                                 \
      FR_SLOT_ROW(ih, rr, c, BT)                                                                              \
      int64_t row_ = rr;                                                                                     \
      const int sid_ = SIDOF;                                                                                \
      if (a.top_k > 0) row_ = sid_ < a.num_valid ? sid_ / a.top_k : 0;                                       \
      xsrc_[ih] = static_cast<unsigned>((row_ * a.ldx + kfirst_ + c * EPC) * static_cast<int64_t>(sizeof(T))); \
      if (a.x_span && sid_ >= a.num_valid) xsrc_[ih] = kSkipOffset;                                          \
    }                                                                                                        \
    _Pragma("unroll") for (int ih = 0; ih < WIW; ++ih) {                                                 \
      FR_SLOT_ROW(ih, rr, c, BF)                                                                              \
      wsrc_[ih] = static_cast<unsigned>(w_byte_offset(a.w_tiled, a.ldw, a.K, w_src_row(pf_, rr),             \
                                                      (kfirst_ + c * EPC) * static_cast<int64_t>(sizeof(T)), sizeof(T))); \
    }                                                                                                        \
  }
  FR_UNIT(0, pid_t, pid_f, expert, kb, kn, tu)
  FR_MAKE_SET(pid_t, pid_f, expert, kb, a.sorted[pid_t * BT + rr], xsrcA, wsrcA, xrsA, wrsA, ntA)

  // Measurement switches (compile time; results are WRONG with any of them, only timings mean something):
  //   FR_ABL_NOLOAD  the ring is filled once and never refilled: MFMAs + fragment reads + barriers on real data
  //   FR_ABL_NOLDS   (with NOLOAD) fragments are read once and stay in registers: MFMAs + barriers
  //   FR_ABL_NOBAR   no barrier between K tiles
  //   FR_ABL_NOMFMA  no MFMA is issued (with NOLDS: tile loads + barriers only, the kernel as a pure stream)
  //   FR_ABL_HOTLOAD every refill fetches one of the tile's first four K tiles again (in L2, beyond the reach of
  //                  the 32 KB L1): the loads' own cost (issue, L2 -> LDS transfer) without the misses of L2
  // They split a launch's time into its MFMA floor, the cost of the LDS fragment reads and the cost of the tile loads.
  // load q_ of an issuing wavefront (weight-tile loads first) of K tile tile_ into ring slot slot_
#ifdef FR_ABL_HOTLOAD
#define FR_KOFF(tile_) (((tile_) & 3) * C::BKB)
#define FR_KOFF_W(tile_) (((tile_) & 3) * wstep)
#else
#define FR_KOFF(tile_) ((tile_) * C::BKB)
#define FR_KOFF_W(tile_) ((tile_) * wstep)
#endif
#define FR_ISSUE_REAL(SET, tile_, slot_, q_)                                                                \
  {                                                                                                         \
    const int vwi_ = wave_u + ((q_) % IW) * (NW / IW);                                                      \
    if ((q_) < WIW) {                                                                                   \
      if (NTW && nt##SET)                                                                                   \
        __builtin_amdgcn_raw_ptr_buffer_load_lds(                                                           \
            wrs##SET, (lptr_t)(lds_raw + (WBASE + (slot_) * C::WCH) * 16 + (((q_) / IW) * NW + vwi_) * (kWave * 16)), \
            16, wsrc##SET[(q_) < WIW ? (q_) : 0], FR_KOFF_W(tile_), 0, 2);                                  \
      else                                                                                                  \
        __builtin_amdgcn_raw_ptr_buffer_load_lds(                                                           \
            wrs##SET, (lptr_t)(lds_raw + (WBASE + (slot_) * C::WCH) * 16 + (((q_) / IW) * NW + vwi_) * (kWave * 16)), \
            16, wsrc##SET[(q_) < WIW ? (q_) : 0], FR_KOFF_W(tile_), 0, 0);                                  \
    } else {                                                                                                \
      __builtin_amdgcn_raw_ptr_buffer_load_lds(                                                             \
          xrs##SET, (lptr_t)(lds_raw + (slot_) * (C::XCH * 16) + ((((q_) - WIW) / IW) * NW + vwi_) * (kWave * 16)), \
          16, xsrc##SET[(q_) < WIW ? 0 : (q_) - WIW], FR_KOFF(tile_), 0, 0);                            \
    }                                                                                                       \
  }
#ifdef FR_ABL_NOLOAD
#define FR_ISSUE_ONE(SET, tile_, slot_, q_) {}
#else
#define FR_ISSUE_ONE(SET, tile_, slot_, q_) FR_ISSUE_REAL(SET, tile_, slot_, q_)
#endif
#define FR_READ_FRAGS_REAL(sl_, ks_, fb_)                                               \
  {                                                                                     \
    const u32x4* xt = lds + (sl_) * C::XCH;                                             \
    const u32x4* wtl = lds + (sl_) * C::WCH;                                            \
    _Pragma("unroll") for (int c = 0; c < FC; ++c) {                                    \
      const int kc = ((ks_) * C::KGROUPS + kgrp) * FC + c;                              \
      const u32x4* xp_ = xt + xoff0 + (kc ^ xkey0);                                     \
      const u32x4* wp_ = wtl + woff0 + (kc ^ wkey0);                                    \
      _Pragma("unroll") for (int i = 0; i < C::IT; ++i) xf[fb_][i][c] = xp_[FR_XD(i)];  \
      _Pragma("unroll") for (int j = 0; j < C::JF; ++j) wfr[fb_][j][c] = wp_[FR_WD(j)]; \
    }                                                                                   \
  }
#ifdef FR_ABL_NOLDS
#define FR_READ_FRAGS(sl_, ks_, fb_) {}
#define FR_ABL_INIT1 FR_READ_FRAGS_REAL(0, 1, 1);
#else
#define FR_READ_FRAGS(sl_, ks_, fb_) FR_READ_FRAGS_REAL(sl_, ks_, fb_)
#define FR_ABL_INIT1
#endif
#ifdef FR_ABL_NOMFMA
#define FR_MFMA(j_, i_, fbw_, fbx_) {}
#else
#define FR_MFMA(j_, i_, fbw_, fbx_)                                                                 \
  {                                                                                                 \
    if constexpr (C::TILE == 32) acc[j_][i_] = E::m32(wfr[fbw_][j_], xf[fbx_][i_], acc[j_][i_]);    \
    else acc[j_][i_] = E::m16(wfr[fbw_][j_], xf[fbx_][i_], acc[j_][i_]);                            \
  }
#endif
#ifdef FR_ABL_NOBAR
#define FR_KT_BARRIER
#else
#define FR_KT_BARRIER __builtin_amdgcn_s_barrier();
#endif
  // fragment i_ of the token operand / j_ of the weight operand alone, into buffer 0
#define FR_READ_X1(sl_, ks_, i_)                                                        \
  {                                                                                     \
    const u32x4* xt = lds + (sl_) * C::XCH;                                             \
    _Pragma("unroll") for (int c = 0; c < FC; ++c) {                                    \
      const int kc = ((ks_) * C::KGROUPS + kgrp) * FC + c;                              \
      xf[0][i_][c] = xt[xoff0 + (kc ^ xkey0) + FR_XD(i_)];                              \
    }                                                                                   \
  }
#define FR_READ_W1(sl_, ks_, j_)                                                        \
  {                                                                                     \
    const u32x4* wtl = lds + (sl_) * C::WCH;                                            \
    _Pragma("unroll") for (int c = 0; c < FC; ++c) {                                    \
      const int kc = ((ks_) * C::KGROUPS + kgrp) * FC + c;                              \
      wfr[0][j_][c] = wtl[woff0 + (kc ^ wkey0) + FR_WD(j_)];                            \
    }                                                                                   \
  }
  // One K-step: NM MFMAs, weight tile j outer, token tile i inner.  HAVE_NEXT: the fragments of K-step
  // NKS of ring slot NSL follow.  With two fragment buffers they are all read after the first half of
  // the MFMAs into the other buffer.  With one buffer (SINGLE: fp8, whose fragments are twice as
  // large) each fragment is read again as soon as its last MFMA of this step has been issued - the
  // weight fragment j after token tile IT-1, the token fragment i during the last weight tile - which
  // leaves at least IT-1 MFMAs (64 cycles each for fp8) between a read and its first use.
  // The refill loads (ISS_: this wavefront issues, set SET) go out one at a time between the MFMAs.
#define FR_KSTEP(fb_, HAVE_NEXT, NSL, NKS, ISS_, SET, tile_, slot_)                           \
  if (on_) {                                                                                  \
    const int fbc = SINGLE ? 0 : (fb_);                                                       \
    _Pragma("unroll") for (int m = 0; m < NM; ++m) {                                          \
      const int j = m / C::IT, i = m % C::IT;                                                 \
      FR_MFMA(j, i, fbc, fbc)                                                                 \
      __builtin_amdgcn_sched_barrier(0);                                                      \
      if (HAVE_NEXT) {                                                                        \
        if constexpr (SINGLE) {                                                               \
          if (i == C::IT - 1) FR_READ_W1(NSL, NKS, j)                                         \
          if (j == C::JF - 1) FR_READ_X1(NSL, NKS, i)                                         \
          if (i == C::IT - 1 || j == C::JF - 1) __builtin_amdgcn_sched_barrier(0);            \
        } else if (m == RD_AT) {                                                              \
          FR_READ_FRAGS(NSL, NKS, fbc ^ 1);                                                   \
          __builtin_amdgcn_sched_barrier(0);                                                  \
        }                                                                                     \
      }                                                                                       \
      if (ISS_) {                                                                             \
        _Pragma("unroll") for (int r = 0; r < NLI; ++r)                                       \
          if (m == ((2 * r + 1) * NM) / (2 * NLI)) {                                          \
            FR_ISSUE_ONE(SET, tile_, slot_, r);                                               \
            __builtin_amdgcn_sched_barrier(0);                                                \
          }                                                                                   \
      }                                                                                       \
    }                                                                                         \
  }
  // One K tile of the current output tile.  REFILL: 0 none (the data is the last this
  // workgroup loads), else the slot of this K tile is refilled from set SET with K tile
  // rtile_ after the barrier that publishes the next K tile; LAST: nothing follows this K
  // tile at all (no barrier, no fragment read-ahead).
#define FR_KTILE(ISS_, REFILL, SET, rtile_, LAST, VMC)                                         \
  {                                                                                            \
    const int sn = (sl + 1 == S) ? 0 : sl + 1;                                                 \
    _Pragma("unroll") for (int ks = 0; ks < KS; ++ks) {                                        \
      if (ks + 1 < KS) {                                                                       \
        FR_KSTEP(ks & 1, true, sl, ks + 1, false, A, 0, 0);                                    \
      } else if (LAST) {                                                                       \
        FR_KSTEP(ks & 1, false, 0, 0, false, A, 0, 0);                                         \
      } else {                                                                                 \
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(VMC) : "memory");                  \
        FR_KT_BARRIER                                                                          \
        FR_KSTEP(ks & 1, true, sn, 0, (ISS_) && (REFILL), SET, rtile_, sl);                    \
      }                                                                                        \
    }                                                                                          \
    sl = sn;                                                                                   \
  }
  // One output tile.  NEXT (compile time): the workgroup has another tile after this one, whose
  // routing data is asked for at the start, turned into the address set B after two K tiles
  // (straight-line code in between, so the wait for it is exact) and whose first S K tiles
  // refill the ring during the last S K tiles of this one.
#define FR_TILE(ISS_, NEXT)                                                                                \
  {                                                                                                        \
    FR_STAMP(0)                                                                                            \
    /* A wavefront that issues no loads and whose token rows of this block are all padding (the upper */   \
    /* half of a block that holds at most half a block of pairs) has nothing to multiply: it keeps the */  \
    /* barriers and leaves the MFMA pipe and the LDS to the wavefront it shares the SIMD with.  When */     \
    /* it has rows again, the fragments its skipped read-ahead would have brought are read here. */         \
    bool on_ = true;                                                                                       \
    if (!(ISS_)) {                                                                                         \
      bool any_ = false;                                                                                   \
      _Pragma("unroll") for (int r0_ = 0; r0_ < C::TT; r0_ += kWave)                                       \
        any_ |= r0_ + lane < C::TT && a.sorted[pid_t * BT + wt * C::TT + r0_ + lane] < a.num_valid;        \
      on_ = __ballot(any_) != 0;                                                                           \
      if (on_) FR_READ_FRAGS(sl, 0, 0)                                                                     \
    }                                                                                                      \
    if (NEXT) {                                                                                            \
      FR_UNIT(unit + 1, n_pid_t, n_pid_f, n_expert, n_kb, n_kn, n_tu)                                      \
      _Pragma("unroll") for (int ih = 0; ih < XIW; ++ih) {                                             \
        FR_SLOT_ROW(ih, rr, c, BT)                                                                          \
        (void)c;                                                                                           \
        n_sid[ih] = a.sorted[n_pid_t * BT + rr];                                                           \
      }                                                                                                    \
    }                                                                                                      \
    _Pragma("unroll") for (int j = 0; j < C::JF; ++j)                                                      \
      _Pragma("unroll") for (int i = 0; i < C::IT; ++i)                                                    \
        _Pragma("unroll") for (int r = 0; r < ACC_N; ++r) acc[j][i][r] = 0.f;                              \
    /* vmcnt(0) once per tile: the previous tile's epilogue stores share the counter with the loads */     \
    FR_KTILE(ISS_, true, A, S, false, 0)                                                                   \
    FR_KTILE(ISS_, true, A, S + 1, false, (S - 2) * NLI)                                                   \
    if (NEXT) FR_MAKE_SET(n_pid_t, n_pid_f, n_expert, n_kb, n_sid[ih], xsrcB, wsrcB, xrsB, wrsB, ntB)      \
    __builtin_amdgcn_s_waitcnt(0xC07F); /* lgkmcnt(0): no scalar load pending inside the loops */          \
    for (int kt = 2; kt < kn - S; ++kt) FR_KTILE(ISS_, true, A, kt + S, false, (S - 2) * NLI)              \
    if (NEXT) {                                                                                            \
      for (int kt = 0; kt < S; ++kt) FR_KTILE(ISS_, true, B, kt, false, (S - 2) * NLI)                     \
    } else {                                                                                               \
      for (int kt = 0; kt < S - 1; ++kt) FR_KTILE(ISS_, false, A, 0, false, 0)                             \
      FR_KTILE(ISS_, false, A, 0, true, 0)                                                                 \
    }                                                                                                      \
    FR_STAMP(1)                                                                                            \
    if (tu < 0) gemm_epilogue<T, C, EPI, HOIST>(a, acc, pid_t, pid_f, expert, split, wt, wf, frow, kgrp);         \
    else tail_store<C, EPI>(a.tail_ws + static_cast<int64_t>(xcd * nper + tu) * (BT * BF), acc, wt, wf, frow, kgrp); \
  }
  // Fill of the ring with the first S K tiles of set A and the first fragments.
#define FR_FILL(ISS_)                                                                                      \
  {                                                                                                        \
    _Pragma("unroll") for (int t = 0; t < S; ++t)                                                          \
      if (ISS_) { _Pragma("unroll") for (int q = 0; q < NLI; ++q) FR_ISSUE_REAL(A, t, t, q); }              \
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((S - 1) * NLI) : "memory");                                   \
    __builtin_amdgcn_s_barrier();                                                                          \
    FR_READ_FRAGS_REAL(0, 0, 0);                                                                           \
    FR_ABL_INIT1                                                                                           \
  }
  // Whole pipeline for an issuing (ISS_ = true) or a non-issuing wavefront.
#define FR_PERSIST(ISS_)                                                                                   \
  {                                                                                                        \
    FR_FILL(ISS_)                                                                                          \
    int sl = 0;                                                                                            \
    int unit = 0;                                                                                          \
    for (; unit + 1 < n_units; ++unit) { /* a next unit exists: hand the ring over to it */                \
      FR_TILE(ISS_, true)                                                                                  \
      pid_t = n_pid_t; pid_f = n_pid_f; expert = n_expert; xrsA = xrsB; wrsA = wrsB; ntA = ntB;            \
      kb = n_kb; kn = n_kn; tu = n_tu;                                                                     \
      _Pragma("unroll") for (int ih = 0; ih < XIW; ++ih) xsrcA[ih] = xsrcB[ih];                        \
      _Pragma("unroll") for (int ih = 0; ih < WIW; ++ih) wsrcA[ih] = wsrcB[ih];                        \
    }                                                                                                      \
    FR_TILE(ISS_, false)                                                                                   \
    FR_STAMP(2)                                                                                            \
  }
#ifdef FR_PROF
  long long pf_t[2] = {0, 0}, pf_last = __builtin_readcyclecounter(), pf_periods = 0;
  const long long pf_begin = pf_last;
#define FR_STAMP(k_)                                                                   \
  {                                                                                    \
    const long long n_ = __builtin_readcyclecounter();                                 \
    pf_t[(k_) == 1 ? 0 : 1] += n_ - pf_last;                                           \
    pf_last = n_;                                                                      \
    if ((k_) == 1) pf_periods += kn;                                                   \
    if ((k_) == 2 && threadIdx.x == 0 && fr_prof_buf) {                                \
      long long* o_ = fr_prof_buf + blockIdx.x * 4;                                    \
      o_[0] = pf_t[0]; o_[1] = pf_t[1]; o_[2] = n_ - pf_begin; o_[3] = pf_periods;     \
    }                                                                                  \
  }
#else
#define FR_STAMP(k_)
#endif
  if (IW == 1 || issuer) FR_PERSIST(true) else FR_PERSIST(false)
#undef FR_STAMP
#undef FR_PERSIST
#undef FR_FILL
#undef FR_TILE
#undef FR_KTILE
#undef FR_KSTEP
#undef FR_READ_W1
#undef FR_XD
#undef FR_WD
#undef FR_READ_X1
#undef FR_READ_FRAGS
#undef FR_ISSUE_ONE
#undef FR_ISSUE_REAL
#undef FR_READ_FRAGS_REAL
#undef FR_ABL_INIT1
#undef FR_KOFF
#undef FR_KOFF_W
#undef FR_MFMA
#undef FR_KT_BARRIER
#undef FR_MAKE_SET
#undef FR_SLOT_ROW
#undef FR_UNIT
#endif
}

// Sums the K slices of the tiles of each XCD's last round in slice order and applies the
// epilogue the GEMM would have applied: routed weight and scatter to the pair's row (EPI_DOWN
// in fp32, EPI_PLAIN in the operand type), or silu(gate)*up to the slot's row of act (EPI_SILU).
// Grid: 8 XCDs x nper/2 tiles (a split tail has at most that many) x BT/32 row groups; blocks
// without a split tile leave at once.  nper = workgroups per XCD of the GEMM launch.
constexpr int kFixupRows = 32;
template <typename T, typename C, int EPI>
__global__ __launch_bounds__(256) void tail_fixup_kernel(const GemmArgs a, int nper) {
  typedef Elem<T> E;
  typedef typename E::out_t out_t;
  typedef typename E::out4 out4;
  constexpr int BT = C::BT, BF = C::BF, BK = C::BKB / static_cast<int>(sizeof(T));
  constexpr int COLS = (EPI == EPI_SILU) ? BF / 2 : BF;  // output columns of a tile
  constexpr int CG = COLS / 4, RPP = 256 / CG;           // 4-column groups per row, rows per pass
  static_assert(256 % CG == 0 && kFixupRows % RPP == 0 && BT % kFixupRows == 0, "fix-up thread map");
  constexpr int BPT = BT / kFixupRows;
  const int half = nper / 2;
  const int xcd = blockIdx.x / (half * BPT), t = (blockIdx.x / BPT) % half, rb = blockIdx.x % BPT;
  const int nt = min(a.npost[0] / BT, a.num_t_blocks);
  const XcdSchedule xs = xcd_schedule(nt * a.num_f_tiles, nper, xcd, a.K / BK, true, schedule_by_rounds(nt, a.num_experts));
  if (xs.slices < 2 || t >= xs.rest) return;
  __shared__ int expert_off[kWalkTable];
  expert_block_offsets(a, nt, expert_off, threadIdx.x, 256);
  int pid_t, pid_f, expert;
  tile_coords(a, expert_off, xs.tail_base + t, pid_t, pid_f, expert);
  const float* wsc = nullptr;
  if constexpr (E::SCALED) wsc = a.w_scale + static_cast<int64_t>(expert) * a.w_rows;
  const float* first = a.tail_ws + static_cast<int64_t>(xcd * nper + t) * (BT * BF);
  const int64_t slice_stride = static_cast<int64_t>(xs.rest) * (BT * BF);
  const int cg = threadIdx.x % CG;
#pragma unroll
  for (int p = 0; p < kFixupRows / RPP; ++p) {
    const int row = rb * kFixupRows + p * RPP + threadIdx.x / CG;
    const int slot = pid_t * BT + row;
    const float* src = first + row * BF + cg * 4;
    if constexpr (EPI != EPI_SILU) {
      const int sid = a.sorted[slot];
      if (sid >= a.num_valid) continue;
      f32x4 sum = *reinterpret_cast<const f32x4*>(src);
      for (int s = 1; s < xs.slices; ++s) sum += *reinterpret_cast<const f32x4*>(src + s * slice_stride);
      float rw = a.mul_weight ? a.topk_w[sid] : 1.f;
      if constexpr (E::SCALED) {  // per-row scales of both fp8 operands
        rw *= a.top_k > 0 ? a.x_scale[sid / a.top_k] : a.x_scale[slot];
        const f32x4 ws = *reinterpret_cast<const f32x4*>(wsc + pid_f * BF + cg * 4);
        sum *= ws;
      }
      const int64_t at = static_cast<int64_t>(sid) * a.ldo + pid_f * BF + cg * 4;
      if constexpr (EPI == EPI_DOWN) {
        const f32x4 o = {sum[0] * rw, sum[1] * rw, sum[2] * rw, sum[3] * rw};
        *reinterpret_cast<f32x4*>(static_cast<float*>(a.out) + at) = o;
      } else {
        out4 o;
#pragma unroll
        for (int r = 0; r < 4; ++r) o[r] = static_cast<out_t>(sum[r] * rw);
        if (a.add_div) atomic_add4(static_cast<out_t*>(a.out) + static_cast<int64_t>(sid / a.add_div) * a.ldo + pid_f * BF + cg * 4, o);
        else *reinterpret_cast<out4*>(static_cast<out_t*>(a.out) + at) = o;
      }
    } else {
      f32x4 g = *reinterpret_cast<const f32x4*>(src), u = *reinterpret_cast<const f32x4*>(src + BF / 2);
      for (int s = 1; s < xs.slices; ++s) {
        g += *reinterpret_cast<const f32x4*>(src + s * slice_stride);
        u += *reinterpret_cast<const f32x4*>(src + s * slice_stride + BF / 2);
      }
      if constexpr (E::SCALED) {
        const int sid = a.sorted[slot];
        const float xsc = a.top_k > 0 ? (sid < a.num_valid ? a.x_scale[sid / a.top_k] : 1.f) : a.x_scale[slot];
        const f32x4 gs = *reinterpret_cast<const f32x4*>(wsc + pid_f * (BF / 2) + cg * 4);
        const f32x4 us = *reinterpret_cast<const f32x4*>(wsc + a.N + pid_f * (BF / 2) + cg * 4);
        g *= gs * xsc;
        u *= us * xsc;
      }
      out4 o;
#pragma unroll
      for (int r = 0; r < 4; ++r) o[r] = static_cast<out_t>(silu(g[r]) * u[r]);
      out_t* orow = static_cast<out_t*>(a.out) + static_cast<int64_t>(slot) * a.ldo + pid_f * (BF / 2) + cg * 4;
      *reinterpret_cast<out4*>(orow) = o;
    }
  }
}

// Workgroups resident at once on the current device (a multiple of 8, one share per XCD).
template <typename T, typename C, int EPI>
int persistent_grid(int* grid_out) {
  constexpr int kMaxDevices = 64;
  static int cached[kMaxDevices] = {};  // per device; a race between threads writes the same value twice
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail(FR_E_LAUNCH, "persistent GEMM: device %d (%s)", dev, hipGetErrorString(e));
  if (!cached[dev]) {
    if (C::LDS_BYTES > 65536)
      e = hipFuncSetAttribute(reinterpret_cast<const void*>(&moe_gemm_persistent_kernel<T, C, EPI>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
    int cus = 0, per_cu = 0;
    if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e == hipSuccess)
      e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, moe_gemm_persistent_kernel<T, C, EPI>, C::NT, C::LDS_BYTES);
    if (e != hipSuccess) {
      (void)hipGetLastError();  // reported here: not to be found again by the next launch check
      return fail(FR_E_LAUNCH, "persistent GEMM set-up (%d B LDS): %s", C::LDS_BYTES, hipGetErrorString(e));
    }
    if (per_cu < 1 || cus < 8) return fail(FR_E_LAUNCH, "persistent GEMM: occupancy %d on %d CUs", per_cu, cus);
    cached[dev] = cus * per_cu / 8 * 8;
  }
  *grid_out = cached[dev];
  return FR_OK;
}

// Launches the persistent form when every split has at least STAGES + 2 K tiles, else the plain one.
// a.tail_ws (kTailUnits buffers of BT x BF floats, or nullptr) enables the split of the last round.
template <typename T, typename C, int EPI>
int launch_gemm_persistent(const GemmArgs& a_in, int splits, hipStream_t st) {
  GemmArgs a = a_in;
  constexpr int BK = C::BKB / static_cast<int>(sizeof(T));
  const int last_k = a.K - (splits - 1) * a.k_per_split;  // K range of the last split
  // The plain kernel double-buffers its fragments over an even number of K-steps per K tile; a tile without that
  // (fp8 on the 16x16x128 MFMA: one K-step per 128-byte K tile) exists in the persistent form only.
  constexpr bool kPlainForm = (C::CPR / (C::KGROUPS * Elem<T>::FC)) % 2 == 0;
  auto plain = [&](const GemmArgs& g) -> int {
    if constexpr (kPlainForm) {
      return launch_gemm<T, C, EPI>(g, splits, st);
    } else {
      if (g.setup_only) return FR_OK;
      return fail(FR_E_SHAPE, "the %d-row tile of this element type needs at least %d K tiles per K slice and at most %d experts",
                  C::BT, C::STAGES + 2, kMaxExperts);
    }
  };
  if (a.setup_only) {  // both forms a launch may take
    int resident = 0;
    const int rc = persistent_grid<T, C, EPI>(&resident);
    return rc != FR_OK ? rc : plain(a);
  }
  if (a.k_per_split / BK < C::STAGES + 2 || last_k / BK < C::STAGES + 2 || a.num_experts < 1 || a.num_experts > kMaxExperts) {
    a.tail_ws = nullptr;
    return plain(a);
  }
  const int64_t x_rows = a.top_k > 0 ? a.num_valid / a.top_k : C::BT;
  const int64_t w_rows = EPI == EPI_SILU ? 2 * static_cast<int64_t>(a.N) : a.N;
  const int64_t lim = int64_t(1) << 32, es = sizeof(T);
  if (x_rows * a.ldx * es >= lim || w_rows * a.ldw * es >= lim)
    return fail(FR_E_SHAPE, "token rows (%lld x %lld) or one expert's weights (%lld x %lld) span 4 GiB or more",
                (long long)x_rows, (long long)a.ldx, (long long)w_rows, (long long)a.ldw);
  a.group_t = tunables().group_m ? tunables().group_m : kChunkBlocks;
  if (tunables().no_tail_split) a.tail_ws = nullptr;
  a.x_span = x_rows * a.ldx * es < (int64_t(1) << 31) ? static_cast<unsigned>(x_rows * a.ldx * es) : 0u;
  int resident = 0;
  const int rc = persistent_grid<T, C, EPI>(&resident);
  if (rc != FR_OK) return rc;
  // the fix-up writes whole tiles of 4-column groups: the feature count must be a multiple of the tile's
  constexpr int COLS = (EPI == EPI_SILU) ? C::BF / 2 : C::BF;
  // tiles the fix-up's thread map covers: 4-column groups of a row over 256 threads, 32-row groups
  constexpr bool kFixable = C::BT % kFixupRows == 0 && 256 % (COLS / 4) == 0 && kFixupRows % (256 / (COLS / 4)) == 0;
  const bool tail = kFixable && a.tail_ws && splits == 1 && a.K / BK >= kTailMinTiles && a.N % COLS == 0;
  if (!tail) a.tail_ws = nullptr;
  const int64_t worst = static_cast<int64_t>(a.num_t_blocks) * a.num_f_tiles;
  int64_t grid = resident / (splits > 1 ? splits : 1) / 8 * 8;  // the splits share the device
  if (grid < 8) grid = 8;
  if (tail) {
    if (grid > kTailUnits) grid = kTailUnits;  // one slice buffer per workgroup
  } else if (grid > (worst + 7) / 8 * 8) {
    grid = (worst + 7) / 8 * 8;
  }
  hipLaunchKernelGGL((moe_gemm_persistent_kernel<T, C, EPI>), dim3(static_cast<unsigned>(grid), splits), dim3(C::NT),
                     C::LDS_BYTES, st, a FR_PROF_ARG);
  int lrc = check_launch("moe_gemm_persistent_kernel");
  if (lrc != FR_OK || !tail) return lrc;
  if constexpr (kFixable) {
    const int nper = static_cast<int>(grid / 8);
    if (nper >= 2) {
      hipLaunchKernelGGL((tail_fixup_kernel<T, C, EPI>), dim3(8 * (nper / 2) * (C::BT / kFixupRows)), dim3(256), 0, st, a, nper);
      lrc = check_launch("tail_fixup_kernel");
    }
  }
  return lrc;
}

}  // namespace fr
