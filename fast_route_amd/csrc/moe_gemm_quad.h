// Persistent grouped GEMM with ONE wavefront per SIMD: 256 sorted slots x 256 features per workgroup, four
// wavefronts of 128 x 128 each, 16x16x32 MFMAs (2-byte operands) or 32x32x64 MFMAs (fp8).
//
// Why.  In the eight-wavefront tiles a wavefront owns 128 x 64 outputs and reads twelve operand fragments from
// LDS for thirty-two MFMAs; with 128 x 128 per wavefront it reads sixteen for sixty-four, a third less LDS traffic
// for the same arithmetic and half as many wavefronts issuing instructions, and the part's clock under MFMA load
// follows the energy a flop costs.  The 256 accumulator registers of a lane live in the accumulation half of the
// register file (one wavefront per SIMD has 512 registers per lane); the ordinary half holds two fragment buffers
// of one K-step each (128 registers) and the two address sets of the persistent hand-off.
//
// Stream.  With a single wavefront per SIMD nobody fills the issue slots a burst of loads or a wait leaves, so the
// wavefront's own instruction stream is even: a K tile of 64 elements is two K-steps of 64 MFMAs; during a K-step
// the sixteen fragments of the following K-step are read, one after every third or fourth MFMA, into the other
// fragment buffer; the one barrier per K tile sits between its two K-steps, where every fragment of the tile has
// been read: the tile's ring slot is free from there on and takes the sixteen loads per wavefront of the K tile
// after next, one after every fourth MFMA of the second K-step, which leaves them the first K-step of the next
// K tile to land.
//
// What such a stream cannot hide is a load that misses L2: the ring has two slots, so at most one K tile per
// workgroup is in flight, and a wavefront that finds the memory pipeline backed up stalls at the issue of its
// next load with its MFMAs behind it.  Hence the L2 touch: the workgroups an XCD runs at one time share their
// operand tiles (the token blocks of one chunk share a weight tile, the feature tiles of one token block its
// rows), and each of them asks for its share of the rows of a K tile several K tiles ahead - one dword per
// 128-byte row piece, into a sink in LDS - so that the tile loads proper find their lines in L2.
//
// Half tiles.  A block whose upper 128 slots are all padding (the last block of every other expert) is multiplied
// as 128 rows x 256 features with the FEATURES split four ways over the wavefronts (128 x 64 each): half the MFMAs
// per K-step, 12 loads per K tile.  Both forms of the K loop exist for every place in the persistent walk; the kind
// of the next unit is known a tile ahead, and the hand-over always loads a whole tile's first two K tiles, so any
// kind may follow any other.
//
// Same tile walk, tail split, LDS swizzle, epilogues and fix-up kernel as moe_gemm_persistent_kernel; the result
// is bit-identical to the eight-wavefront kernels on the same MFMA shape (same K order per accumulator).
//
// Measurement switches (compile time, -D): FQ_TOUCH=0 no L2 touch, FQ_HALF=0 no half tiles, FQ_AHEAD=n touch
// distance in K tiles, FQ_XSHARE=n ways the token rows' touch is shared; results stay correct with all of them.
#pragma once
#include "moe_gemm_persistent.h"

namespace fr {

// 2-byte operands: 16x16x32 MFMAs (8 x 8 accumulator tiles of 4 registers per wavefront); fp8: 32x32x64 (4 x 4 tiles of
// 16 registers).  Either way a K tile of 128 bytes per row is two K-steps, a K-step's fragments are 16 reads of 16
// bytes per lane and 64 registers, and a wavefront issues 16 tile loads per K tile.
template <typename T> struct QuadTile { static constexpr int kTile = sizeof(T) == 1 ? 32 : 16; };
template <typename T> using QuadCfg = Cfg<256, 256, 128, 2, 2, QuadTile<T>::kTile, 1, 2, 0, 1>;
// output geometry of a half tile: 128 rows, a quarter of the features per wavefront
template <typename T> using QuadHalfCfg = Cfg<128, 256, 128, 1, 4, QuadTile<T>::kTile, 1, 2, 0, 1>;
constexpr int kQuadMinTiles = 8;    // K tiles per work unit, at least (two peeled at each end, the touch distance)
#ifndef FQ_AHEAD
#define FQ_AHEAD 3
#endif
constexpr int kQuadTouchAhead = FQ_AHEAD;  // K tiles between a touch and the tile loads of the same rows
constexpr int kQuadSink = 1024;     // bytes of LDS the touches land in (256 per wavefront)

#ifndef FQ_TAIL_LONG_K  // measurement switches of the host side: K tiles from which a K loop counts as long, and
#define FQ_TAIL_LONG_K 112
#endif
#ifndef FQ_TAIL_ROUNDS_SHORT  // whole rounds after which a shorter one stops splitting its last round
#define FQ_TAIL_ROUNDS_SHORT 8
#endif
#ifndef FQ_XSHARE
#define FQ_XSHARE 4
#endif
#ifndef FQ_HALF
#define FQ_HALF 1
#endif
#ifndef FQ_TOUCH
#define FQ_TOUCH 1
#endif

template <typename T, int EPI>
__global__ __launch_bounds__(256, 1) void moe_gemm_quad_kernel(const GemmArgs a FR_PROF_PARAM) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef QuadCfg<T> C;
  typedef QuadHalfCfg<T> CH;
  typedef Elem<T> E;
  typedef __attribute__((address_space(3))) void* lptr_t;
  typedef typename std::conditional<C::TILE == 32, f32x16, f32x4>::type acc_t;
  constexpr int ES = static_cast<int>(sizeof(T));
  constexpr int BT = C::BT, BF = C::BF, CPR = C::CPR, BK = C::BKB / ES, EPC = 16 / ES, FC = E::FC;
  constexpr int TILE = C::TILE, KG = C::KGROUPS;
  constexpr int NF = 128 / TILE;              // fragments per operand and K-step (8, fp8: 4)
  constexpr int NM = NF * NF;                 // MFMAs per K-step (64 of 16 cycles, fp8: 16 of 64 cycles)
  constexpr int NW = 4, XI = 8, WI = 8, NL = XI + WI;  // tile loads per wavefront and K tile
  constexpr int XBYTES = C::XCH * 16, WBYTES = C::WCH * 16, SLOT = XBYTES + WBYTES;  // a ring slot: X rows, then W rows
  // Whole tile, 2-byte operands: one fragment read after every 3rd / 4th MFMA of the first / second K-step, tile
  // load q after MFMA 2 + 4 q of the second.  fp8 has a quarter of the MFMAs, four times as long: two fragment reads
  // after each of the first eight, one tile load after every one of the second K-step.
  constexpr int RD0 = FC == 1 ? 3 : 1, RD1 = FC == 1 ? 4 : 1, RPS = FC;
  constexpr int LD_POS = FC == 1 ? 2 : 0, LD_EVERY = FC == 1 ? 4 : 1;
  static_assert(C::IT == NF && C::JF == NF && C::XIW == XI && C::WIW == WI && CPR == 8 && CPR / (KG * FC) == 2, "128 x 128 per wavefront, two K-steps per K tile");

  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];

  // ---- schedule (as in moe_gemm_persistent_kernel) -----------------------------------------
  const int npost = a.npost[0];
  const int nt = min(npost / BT, a.num_t_blocks);
  const int total = nt * a.num_f_tiles;
  const int xcd = blockIdx.x & 7, nper = gridDim.x >> 3, loc = blockIdx.x >> 3;
  const int k_all = a.K / BK;
  const XcdSchedule xs = xcd_schedule(total, nper, xcd, k_all, a.tail_ws != nullptr, schedule_by_rounds(nt, a.num_experts));
  const int n_units = xs.rounds + (loc < xs.rest * xs.slices ? 1 : 0);
  if (n_units == 0) return;
  __shared__ int expert_off[kWalkTable];
  expert_block_offsets(a, nt, expert_off, threadIdx.x, C::NT);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave_u = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wt = wave_u >> 1, wf = wave_u & 1;
  const int wstep = a.w_tiled ? (C::BKB / kTileBytes) * kTilePiece : C::BKB;  // bytes from one K tile of W to the next
  const T* X = static_cast<const T*>(a.X);

#define FQ_UNIT(j_, pt_, pf_, ex_, kb_, kn_, tu_, sh_)                                         \
  {                                                                                            \
    int lin_;                                                                                  \
    if ((j_) < xs.rounds) {                                                                    \
      lin_ = xcd_round_tile(xs, nper, xcd, loc, (j_));                                         \
      kb_ = 0; kn_ = k_all; tu_ = -1;                                                          \
    } else {                                                                                   \
      const int t_ = loc % xs.rest, s_ = loc / xs.rest;                                        \
      lin_ = xs.tail_base + t_;                                                                \
      kb_ = s_ * k_all / xs.slices;                                                            \
      kn_ = (s_ + 1) * k_all / xs.slices - kb_;                                                \
      tu_ = xs.slices > 1 ? s_ * xs.rest + t_ : -1;                                            \
    }                                                                                          \
    tile_coords(a, expert_off, lin_, pt_, pf_, ex_, &sh_);                                     \
  }
  // load q of this wavefront fills LDS rows [8 * (q * NW + wave), + 8) of the X or W tile: lane -> (row, chunk)
#define FQ_SLOT_ROW(q_, rr_, c_)                                   \
  const int slot_ = ((q_) * NW + wave_u) * kWave + lane;           \
  const int rr_ = slot_ / CPR, c_ = swizzle<CPR>(rr_, slot_ % CPR);
  auto w_src_row = [&](int pf, int rr) -> int {
    if constexpr (EPI == EPI_SILU) {
      const int half = rr / (BF / 2), f = pf * (BF / 2) + rr % (BF / 2);
      return half * a.N + (f < a.N ? f : a.N - 1);
    } else {
      const int f = pf * BF + rr;
      return f < a.N ? f : a.N - 1;
    }
  };

  // ---- fragment addresses: one per operand and K-step, the fragments at immediate offsets ------
  // Whole tile: wavefront (wt, wf) owns token rows [wt * 128, + 128) x the weight rows acc_tile_col<C>(wf, .).
  // Half tile (the block's upper 128 slots are all padding): wavefront w owns token rows [0, 128) x the weight
  // rows acc_tile_col<CH>(w, .) - a quarter of the features each, so that the four MFMA pipes share what is left.
  // All of a lane's fragment rows lie multiples of 16 apart (one swizzle key), and the two forms differ by
  // wavefront-uniform distances.
  const int frow = lane % TILE, kgrp = lane / TILE;
  const int key0 = swizzle<CPR>(frow, 0);
  int xadr[2][FC];  // byte addresses in slot 0 of the chunks of row frow of the X tile (the W tile: XBYTES further)
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int c = 0; c < FC; ++c) xadr[s][c] = (frow * CPR + (((s * KG + kgrp) * FC + c) ^ key0)) * 16;
  const int xbaseF = wt * C::TT * CPR * 16, wbaseF = acc_tile_col<C, EPI>(wf, 0) * CPR * 16;
  const int wbaseH = acc_tile_col<CH, EPI>(wave_u, 0) * CPR * 16;
#define FQ_XD(i_) ((i_) * TILE * CPR * 16)
#define FQ_WD(HALF, j_) ((HALF) ? (acc_tile_col<CH, EPI>(0, (j_)) - acc_tile_col<CH, EPI>(0, 0)) * CPR * 16 \
                               : (acc_tile_col<C, EPI>(0, (j_)) - acc_tile_col<C, EPI>(0, 0)) * CPR * 16)

  acc_t acc[NF][NF];
  u32x4 fw[2][NF][FC], fx[2][NF][FC];

  // ---- address sets: A = unit being multiplied, B = the workgroup's next unit ---------------------
  int pid_t, pid_f, expert, kb, kn, tu;
  int n_pid_t = 0, n_pid_f = 0, n_expert = 0, n_kb = 0, n_kn = 0, n_tu = -1;
  bool half = false, n_half = false;  // the unit is a half tile
  TileShare shA, shB;
  int n_sid[XI], n_tsid = 0, n_up0 = 0, n_up1 = 0;
  unsigned xsrcA[XI], wsrcA[WI], xsrcB[XI], wsrcB[WI];
  unsigned twA = 0, txA = 0, twB = 0, txB = 0;  // touch offsets (weight rows, token rows) of this lane
  __amdgpu_buffer_rsrc_t xrsA, wrsA, xrsB, wrsB;
  // Touch shares.  Weight K tile (256 rows): shared by the sh.count token blocks of the tile's chunk, block
  // sh.index asks for rows [index * per, + per), per = ceil(256 / count), a quarter of them per wavefront.
  // Token K tile (256 gathered rows): shared by the feature tiles of the block an XCD holds at one time, about
  // 32 / count of them, at most FQ_XSHARE: feature tile f asks for share f % that many.
#define FQ_TOUCH_ROWS(sh_, pf_, wrow_, xrow_, xon_)                                            \
  {                                                                                            \
    const int cnt_ = max(1, min((sh_).count, 32));                                             \
    const int per_ = (BF + cnt_ - 1) / cnt_, pw_ = (per_ + NW - 1) / NW;                       \
    wrow_ = min((sh_).index * per_ + wave_u * pw_ + (lane < pw_ ? lane : 0), BF - 1);          \
    const int xs_ = max(1, min(FQ_XSHARE, 32 / cnt_)), xper_ = BT / xs_, xw_ = xper_ / NW;     \
    xrow_ = ((pf_) % xs_) * xper_ + wave_u * xw_ + (lane < xw_ ? lane : 0);                    \
    xon_ = lane < xw_;                                                                         \
  }
  // the sorted ids of the upper 128 slots of block pt_, two per lane: a block is a half tile when none holds a pair
#define FQ_UPPER_IDS(pt_, u0_, u1_)                                \
  {                                                                \
    u0_ = a.sorted[(pt_) * BT + BT / 2 + lane];                    \
    u1_ = a.sorted[(pt_) * BT + BT / 2 + kWave + lane];            \
  }
#define FQ_IS_HALF(u0_, u1_) (FQ_HALF && __ballot((u0_) < a.num_valid || (u1_) < a.num_valid) == 0)
#define FQ_MAKE_SET(pt_, pf_, ex_, kb_, sh_, SIDOF, TSIDOF, xsrc_, wsrc_, xrs_, wrs_, tw_, tx_)                 \
  {                                                                                                          \
    const int64_t xrow0_ = a.top_k > 0 ? 0 : static_cast<int64_t>(pt_) * BT;                                 \
    const int64_t kfirst_ = static_cast<int64_t>(kb_) * BK;                                                  \
    xrs_ = uniform_rsrc(X + xrow0_ * a.ldx, a.x_span ? a.x_span : 0xFFFFFFFFu);                              \
    wrs_ = uniform_rsrc(static_cast<const T*>(a.W) + static_cast<int64_t>(ex_) * a.w_expert_stride);         \
    _Pragma("unroll") for (int q = 0; q < XI; ++q) {                                                         \
      FQ_SLOT_ROW(q, rr, c)                                                                                  \
      int64_t row_ = rr;                                                                                     \
      const int sid_ = SIDOF;                                                                                \
      if (a.top_k > 0) row_ = sid_ < a.num_valid ? sid_ / a.top_k : 0;                                       \
      xsrc_[q] = static_cast<unsigned>((row_ * a.ldx + kfirst_ + c * EPC) * ES);                              \
      if (a.x_span && sid_ >= a.num_valid) xsrc_[q] = kSkipOffset;                                           \
    }                                                                                                        \
    _Pragma("unroll") for (int q = 0; q < WI; ++q) {                                                         \
      FQ_SLOT_ROW(q, rr, c)                                                                                  \
      wsrc_[q] = static_cast<unsigned>(w_byte_offset(a.w_tiled, a.ldw, a.K, w_src_row(pf_, rr), (kfirst_ + c * EPC) * ES, ES)); \
    }                                                                                                        \
    if (FQ_TOUCH) {                                                                                          \
      int wrow_, xrow_; bool xon_;                                                                           \
      FQ_TOUCH_ROWS(sh_, pf_, wrow_, xrow_, xon_)                                                            \
      (void)xrow_;                                                                                           \
      tw_ = static_cast<unsigned>(w_byte_offset(a.w_tiled, a.ldw, a.K, w_src_row(pf_, wrow_), kfirst_ * ES, ES)); \
      int64_t trow_ = xrow_;                                                                                 \
      const int tsid_ = TSIDOF;                                                                              \
      if (a.top_k > 0) trow_ = tsid_ < a.num_valid ? tsid_ / a.top_k : 0;                                    \
      tx_ = static_cast<unsigned>((trow_ * a.ldx + kfirst_) * ES);                                            \
      if (a.x_span && (tsid_ >= a.num_valid || !xon_)) tx_ = kSkipOffset;                                    \
    }                                                                                                        \
  }
  // tile load q (weight rows first) of K tile tile_ of set SET into ring slot slot_
#define FQ_ISSUE(SET, tile_, slot_, q_)                                                                     \
  {                                                                                                         \
    if ((q_) < WI) {                                                                                        \
      __builtin_amdgcn_raw_ptr_buffer_load_lds(                                                             \
          wrs##SET, (lptr_t)(lds_raw + (slot_) * SLOT + XBYTES + ((q_) * NW + wave_u) * (kWave * 16)),      \
          16, wsrc##SET[(q_) < WI ? (q_) : 0], (tile_) * wstep, 0, 0);                                      \
    } else {                                                                                                \
      __builtin_amdgcn_raw_ptr_buffer_load_lds(                                                             \
          xrs##SET, (lptr_t)(lds_raw + (slot_) * SLOT + (((q_) - WI) * NW + wave_u) * (kWave * 16)),        \
          16, xsrc##SET[(q_) < WI ? 0 : (q_) - WI], (tile_) * C::BKB, 0, 0);                                \
    }                                                                                                       \
  }
  // touch of K tile tile_ of the unit whose set is (tw_, tx_, wrs_, xrs_)
#define FQ_TOUCH_ISSUE(wrs_, xrs_, tw_, tx_, tile_)                                                         \
  {                                                                                                         \
    __builtin_amdgcn_raw_ptr_buffer_load_lds(wrs_, (lptr_t)(lds_raw + 2 * SLOT + wave_u * 256), 4, tw_, (tile_) * wstep, 0, 0);  \
    __builtin_amdgcn_raw_ptr_buffer_load_lds(xrs_, (lptr_t)(lds_raw + 2 * SLOT + wave_u * 256), 4, tx_, (tile_) * C::BKB, 0, 0); \
  }
#define FQ_READ_W(HALF, buf_, j_, c_, s_, sl_)                                                             \
  fw[buf_][j_][c_] = *reinterpret_cast<const u32x4*>(lds_raw + XBYTES + xadr[s_][c_] + ((HALF) ? wbaseH : wbaseF) + \
                                                     (sl_) * SLOT + FQ_WD(HALF, j_));
#define FQ_READ_X(HALF, buf_, i_, c_, s_, sl_) \
  fx[buf_][i_][c_] = *reinterpret_cast<const u32x4*>(lds_raw + xadr[s_][c_] + ((HALF) ? 0 : xbaseF) + (sl_) * SLOT + FQ_XD(i_));
  // read r of a K-step's fragment reads (FC chunks per fragment): whole tile X0 W0 X1 W1 ..., half tile X0 X1 W0
  // X2 X3 W1 ... (twice as many token as weight fragments)
#define FQ_READ_NTH(HALF, r_, buf_, s_, sl_)                                                               \
  {                                                                                                        \
    const int f_ = (r_) / FC, c_ = (r_) % FC;                                                          \
    if (HALF) {                                                                                            \
      if (f_ % 3 == 2) { FQ_READ_W(true, buf_, f_ / 3, c_, s_, sl_) }                                      \
      else { FQ_READ_X(true, buf_, (f_ / 3) * 2 + f_ % 3, c_, s_, sl_) }                                   \
    } else {                                                                                               \
      if (f_ & 1) { FQ_READ_W(false, buf_, f_ >> 1, c_, s_, sl_) } else { FQ_READ_X(false, buf_, f_ >> 1, c_, s_, sl_) } \
    }                                                                                                      \
  }
  // One K-step: the MFMAs of fragment buffer S (a half tile: half as many, its weight fragments are half).
  // FIRST: the accumulators start from zero.  RD: the fragments of K-step S ^ 1 of ring slot rsl_ are read into
  // the other buffer.  NLD_ (0: none): the first NLD_ loads of K tile ltile_ of set LSET go into slot lsl_.
  // TCH: the touch (resources and offsets given) of K tile ttile_, behind the last load.
#define FQ_KSTEP(HALF, S, FIRST, RD, rsl_, NLD_, LSET, ltile_, lsl_, TCH, twrs_, txrs_, tw_, tx_, ttile_)   \
  {                                                                                                        \
    constexpr int NMk = (HALF) ? NM / 2 : NM, NR = ((HALF) ? NF + NF / 2 : 2 * NF) * FC;                   \
    constexpr int RE = (HALF) ? (FC == 1 ? 2 : 1) : ((S) == 0 ? RD0 : RD1);                                \
    constexpr int LP = (HALF) ? (FC == 1 ? 1 : 0) : LD_POS, LE = (HALF) ? (FC == 1 ? 2 : 1) : LD_EVERY;    \
    constexpr int LPS = ((HALF) && FC == 2) ? 2 : 1;  /* loads per MFMA slot */                            \
    static_assert(LP + ((NL + LPS - 1) / LPS - 1) * LE < NMk && ((NR + RPS - 1) / RPS - 1) * RE < NMk,     \
                  "loads and reads fit the K-step");                                                       \
    _Pragma("unroll") for (int m = 0; m < NMk; ++m) {                                                      \
      const int j = m / NF, i = m % NF;                                                                    \
      if (FIRST) {                                                                                         \
        const acc_t z_ = {};                                                                               \
        if constexpr (TILE == 32) acc[j][i] = E::m32(fw[S][j], fx[S][i], z_);                              \
        else acc[j][i] = E::m16(fw[S][j], fx[S][i], z_);                                                   \
      } else {                                                                                             \
        if constexpr (TILE == 32) acc[j][i] = E::m32(fw[S][j], fx[S][i], acc[j][i]);                       \
        else acc[j][i] = E::m16(fw[S][j], fx[S][i], acc[j][i]);                                            \
      }                                                                                                    \
      __builtin_amdgcn_sched_barrier(0);                                                                   \
      if ((RD) && m % RE == 0) {                                                                           \
        _Pragma("unroll") for (int rr = 0; rr < RPS; ++rr)                                                 \
          if ((m / RE) * RPS + rr < NR) {                                                                  \
            FQ_READ_NTH(HALF, (m / RE) * RPS + rr, (S) ^ 1, (S) ^ 1, rsl_)                                 \
            __builtin_amdgcn_sched_barrier(0);                                                             \
          }                                                                                                \
      }                                                                                                    \
      if ((NLD_) > 0 && m >= LP && (m - LP) % LE == 0) {                                                   \
        _Pragma("unroll") for (int ll = 0; ll < LPS; ++ll)                                                 \
          if (((m - LP) / LE) * LPS + ll < (NLD_)) {                                                       \
            FQ_ISSUE(LSET, ltile_, lsl_, ((m - LP) / LE) * LPS + ll)                                       \
            __builtin_amdgcn_sched_barrier(0);                                                             \
          }                                                                                                \
      }                                                                                                    \
      if ((TCH) && FQ_TOUCH && m == NMk - 1) {                                                             \
        FQ_TOUCH_ISSUE(twrs_, txrs_, tw_, tx_, ttile_)                                                     \
        __builtin_amdgcn_sched_barrier(0);                                                                 \
      }                                                                                                    \
    }                                                                                                      \
  }
  // the two newest memory operations of a wavefront at the barrier are the touches of the K tile before:
  // everything older - the tile loads the barrier publishes - has landed
#define FQ_SYNC                                                                          \
  {                                                                                      \
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(FQ_TOUCH ? 2 : 0) : "memory");   \
    __builtin_amdgcn_s_barrier();                                                        \
    __builtin_amdgcn_sched_barrier(0);                                                   \
  }
#define FQ_SYNC0                                                                         \
  {                                                                                      \
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");                          \
    __builtin_amdgcn_s_barrier();                                                        \
    __builtin_amdgcn_sched_barrier(0);                                                   \
  }
  // A period: K tile t of the unit from ring slot par; its slot takes K tile ltile_ of the unit (a half tile loads
  // the weight rows and the lower 128 token rows: 12 loads).  Touch of K tile ttile_ of the unit.
#define FQ_PERIOD_A(HALF, FIRST, ltile_, ttile_)                                                                   \
  {                                                                                                                \
    FQ_KSTEP(HALF, 0, FIRST, true, par, 0, A, 0, 0, false, wrsA, xrsA, twA, txA, 0)                                \
    if (FIRST) FQ_SYNC0 else FQ_SYNC                                                                               \
    FQ_KSTEP(HALF, 1, false, true, par ^ 1, ((HALF) ? WI + XI / 2 : NL), A, ltile_, par, true, wrsA, xrsA, twA, txA, ttile_) \
    par ^= 1;                                                                                                      \
  }
  // One work unit (an output tile, or a K slice of one): kn >= kQuadMinTiles K tiles.  The ring holds the unit's
  // first two K tiles when it starts.  NEXT: the workgroup has another unit after this one, whose routing data is
  // asked for at the start, turned into the address set B after two K tiles, and whose first two K tiles (all 16
  // loads: its kind need not be this unit's) refill the ring during the last two K tiles of this one.
#define FQ_TILE(NEXT, HALF)                                                                                        \
  {                                                                                                                \
    FQ_STAMP(0)                                                                                                    \
    _Pragma("unroll") for (int r = 0; r < ((HALF) ? NF + NF / 2 : 2 * NF) * FC; ++r) FQ_READ_NTH(HALF, r, 0, 0, par) \
    if (NEXT) {                                                                                                    \
      FQ_UNIT(unit + 1, n_pid_t, n_pid_f, n_expert, n_kb, n_kn, n_tu, shB)                                         \
      _Pragma("unroll") for (int q = 0; q < XI; ++q) {                                                             \
        FQ_SLOT_ROW(q, rr, c)                                                                                      \
        (void)c;                                                                                                   \
        n_sid[q] = a.sorted[n_pid_t * BT + rr];                                                                    \
      }                                                                                                            \
      FQ_UPPER_IDS(n_pid_t, n_up0, n_up1)                                                                          \
      if (FQ_TOUCH) {                                                                                              \
        int wrow_, xrow_; bool xon_;                                                                               \
        FQ_TOUCH_ROWS(shB, n_pid_f, wrow_, xrow_, xon_)                                                            \
        (void)wrow_; (void)xon_;                                                                                   \
        n_tsid = a.sorted[n_pid_t * BT + xrow_];                                                                   \
      }                                                                                                            \
    }                                                                                                              \
    FQ_PERIOD_A(HALF, true, 2, kQuadTouchAhead)                                                                    \
    FQ_PERIOD_A(HALF, false, 3, 1 + kQuadTouchAhead)                                                               \
    if (NEXT) {                                                                                                    \
      FQ_MAKE_SET(n_pid_t, n_pid_f, n_expert, n_kb, shB, n_sid[q], n_tsid, xsrcB, wsrcB, xrsB, wrsB, twB, txB)     \
      n_half = FQ_IS_HALF(n_up0, n_up1);                                                                           \
    }                                                                                                              \
    __builtin_amdgcn_s_waitcnt(0xC07F); /* lgkmcnt(0): no scalar load pending inside the loop */                   \
    for (int t = 2; t < kn - kQuadTouchAhead; ++t) FQ_PERIOD_A(HALF, false, t + 2, t + kQuadTouchAhead)            \
    if (NEXT) {                                                                                                    \
      /* the unit's last kQuadTouchAhead K tiles: touches go to the next unit's first K tiles */                   \
      int tb_ = 0;                                                                                                 \
      for (int t = kn - kQuadTouchAhead; t < kn - 2; ++t, ++tb_) {                                                 \
        FQ_KSTEP(HALF, 0, false, true, par, 0, A, 0, 0, false, wrsA, xrsA, twA, txA, 0)                            \
        FQ_SYNC                                                                                                    \
        FQ_KSTEP(HALF, 1, false, true, par ^ 1, ((HALF) ? WI + XI / 2 : NL), A, t + 2, par, true, wrsB, xrsB, twB, txB, tb_) \
        par ^= 1;                                                                                                  \
      }                                                                                                            \
      FQ_KSTEP(HALF, 0, false, true, par, 0, A, 0, 0, false, wrsA, xrsA, twA, txA, 0)                              \
      FQ_SYNC                                                                                                      \
      FQ_KSTEP(HALF, 1, false, true, par ^ 1, NL, B, 0, par, true, wrsB, xrsB, twB, txB, tb_)                      \
      par ^= 1;                                                                                                    \
      FQ_KSTEP(HALF, 0, false, true, par, 0, A, 0, 0, false, wrsA, xrsA, twA, txA, 0)                              \
      FQ_SYNC                                                                                                      \
      FQ_KSTEP(HALF, 1, false, false, 0, NL, B, 1, par, true, wrsB, xrsB, twB, txB, tb_ + 1)                       \
      par ^= 1;                                                                                                    \
    } else {                                                                                                       \
      for (int t = kn - kQuadTouchAhead; t < kn - 2; ++t) FQ_PERIOD_A(HALF, false, t + 2, kn - 1)                  \
      FQ_KSTEP(HALF, 0, false, true, par, 0, A, 0, 0, false, wrsA, xrsA, twA, txA, 0)                              \
      FQ_SYNC                                                                                                      \
      FQ_KSTEP(HALF, 1, false, true, par ^ 1, 0, A, 0, 0, false, wrsA, xrsA, twA, txA, 0)                          \
      par ^= 1;                                                                                                    \
      FQ_KSTEP(HALF, 0, false, true, par, 0, A, 0, 0, false, wrsA, xrsA, twA, txA, 0)                              \
      FQ_SYNC0                                                                                                     \
      FQ_KSTEP(HALF, 1, false, false, 0, 0, A, 0, 0, false, wrsA, xrsA, twA, txA, 0)                               \
    }                                                                                                              \
    FQ_STAMP(1)                                                                                                    \
    /* the last MFMA's result is 16 cycles away: the fetches below are beyond the compiler's hazard checks */      \
    asm volatile("s_nop 7\n\ts_nop 7" ::: "memory");                                                               \
    float* tws_ = a.tail_ws + static_cast<int64_t>(xcd * nper + (tu < 0 ? 0 : tu)) * (BT * BF);                    \
    if (HALF) {                                                                                                    \
      acc_t(&acch_)[NF / 2][NF] = reinterpret_cast<acc_t(&)[NF / 2][NF]>(acc);                                     \
      if (tu < 0) gemm_epilogue<T, CH, EPI, true, true>(a, acch_, 2 * pid_t, pid_f, expert, 0, 0, wave_u, frow, kgrp); \
      else tail_store<CH, EPI, true>(tws_, acch_, 0, wave_u, frow, kgrp);                                          \
    } else {                                                                                                       \
      if (tu < 0) gemm_epilogue<T, C, EPI, true, true>(a, acc, pid_t, pid_f, expert, 0, wt, wf, frow, kgrp);       \
      else tail_store<C, EPI, true>(tws_, acc, wt, wf, frow, kgrp);                                                \
    }                                                                                                              \
  }

  FQ_UNIT(0, pid_t, pid_f, expert, kb, kn, tu, shA)
  {
    int tsid0 = 0, up0, up1;
    FQ_UPPER_IDS(pid_t, up0, up1)
    half = FQ_IS_HALF(up0, up1);
    if (FQ_TOUCH) {
      int wrow_, xrow_; bool xon_;
      FQ_TOUCH_ROWS(shA, pid_f, wrow_, xrow_, xon_)
      (void)wrow_; (void)xon_;
      tsid0 = a.sorted[pid_t * BT + xrow_];
    }
    FQ_MAKE_SET(pid_t, pid_f, expert, kb, shA, a.sorted[pid_t * BT + rr], tsid0, xsrcA, wsrcA, xrsA, wrsA, twA, txA)
  }
  // fill: K tiles 0 and 1 into slots 0 and 1
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int q = 0; q < NL; ++q) FQ_ISSUE(A, t, t, q)
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NL) : "memory");
  __builtin_amdgcn_s_barrier();
  int par = 0;
  int unit = 0;
#ifdef FR_PROF  // cycle counts of wavefront 0 of every workgroup: K loops / epilogues and hand-over / total / K tiles
  long long pf_t[2] = {0, 0}, pf_last = __builtin_readcyclecounter(), pf_periods = 0;
  const long long pf_begin = pf_last;
#define FQ_STAMP(k_)                                                                   \
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
#define FQ_STAMP(k_)
#endif
  for (; unit + 1 < n_units; ++unit) {
    if (half) FQ_TILE(true, true) else FQ_TILE(true, false)
    pid_t = n_pid_t; pid_f = n_pid_f; expert = n_expert; xrsA = xrsB; wrsA = wrsB;
    kb = n_kb; kn = n_kn; tu = n_tu; twA = twB; txA = txB; half = n_half;
#pragma unroll
    for (int q = 0; q < XI; ++q) xsrcA[q] = xsrcB[q];
#pragma unroll
    for (int q = 0; q < WI; ++q) wsrcA[q] = wsrcB[q];
  }
  if (half) FQ_TILE(false, true) else FQ_TILE(false, false)
  FQ_STAMP(2)
#undef FQ_STAMP
#undef FQ_TILE
#undef FQ_PERIOD_A
#undef FQ_SYNC0
#undef FQ_SYNC
#undef FQ_KSTEP
#undef FQ_READ_NTH
#undef FQ_READ_X
#undef FQ_READ_W
#undef FQ_TOUCH_ISSUE
#undef FQ_ISSUE
#undef FQ_MAKE_SET
#undef FQ_IS_HALF
#undef FQ_UPPER_IDS
#undef FQ_TOUCH_ROWS
#undef FQ_XD
#undef FQ_WD
#undef FQ_SLOT_ROW
#undef FQ_UNIT
#endif
}

// Workgroups resident at once on the current device: one per CU (a multiple of 8, one share per XCD).
template <typename T, int EPI>
int quad_grid(int* grid_out) {
  typedef QuadCfg<T> C;
  constexpr int kMaxDevices = 64;
  constexpr int kLds = C::LDS_BYTES + kQuadSink;
  static int cached[kMaxDevices] = {};  // per device; a race between threads writes the same value twice
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail(FR_E_LAUNCH, "quad GEMM: device %d (%s)", dev, hipGetErrorString(e));
  if (!cached[dev]) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(&moe_gemm_quad_kernel<T, EPI>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    int cus = 0, per_cu = 0;
    if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e == hipSuccess) e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, moe_gemm_quad_kernel<T, EPI>, C::NT, kLds);
    if (e != hipSuccess) {
      (void)hipGetLastError();  // reported here: not to be found again by the next launch check
      return fail(FR_E_LAUNCH, "quad GEMM set-up (%d B LDS): %s", kLds, hipGetErrorString(e));
    }
    if (per_cu < 1 || cus < 8) return fail(FR_E_LAUNCH, "quad GEMM: occupancy %d on %d CUs", per_cu, cus);
    cached[dev] = cus / 8 * 8;  // one workgroup per CU: a second would share the SIMDs' MFMA pipes
  }
  *grid_out = cached[dev];
  return FR_OK;
}

// Launches the one-wavefront-per-SIMD form of the 256-row tile for a single K split with at least kQuadMinTiles
// K tiles per work unit.  Returns 1 when the shape is not one it takes (nothing launched: the caller takes
// launch_gemm_persistent).
template <typename T, int EPI>
int launch_gemm_quad(const GemmArgs& a_in, int splits, hipStream_t st) {
  typedef QuadCfg<T> C;
  GemmArgs a = a_in;
  constexpr int ES = static_cast<int>(sizeof(T)), BK = C::BKB / ES;
  if (a.setup_only) {
    int resident = 0;
    return quad_grid<T, EPI>(&resident);
  }
  // a K slice of the split tail has at least k tiles / kTailMaxSplit K tiles (and never under kTailMinSlice)
  if (splits != 1 || a.K % BK != 0 || a.K / BK < 2 * kQuadMinTiles || a.num_experts < 1 || a.num_experts > kMaxExperts) return 1;
  const int64_t x_rows = a.top_k > 0 ? a.num_valid / a.top_k : C::BT;
  const int64_t w_rows = EPI == EPI_SILU ? 2 * static_cast<int64_t>(a.N) : a.N;
  const int64_t lim = int64_t(1) << 32;
  if (x_rows * a.ldx * ES >= lim || w_rows * a.ldw * ES >= lim)
    return fail(FR_E_SHAPE, "token rows (%lld x %lld) or one expert's weights (%lld x %lld) span 4 GiB or more",
                (long long)x_rows, (long long)a.ldx, (long long)w_rows, (long long)a.ldw);
  a.group_t = tunables().group_m ? tunables().group_m : kChunkBlocks;
  if (tunables().no_tail_split) a.tail_ws = nullptr;
  a.x_span = x_rows * a.ldx * ES < (int64_t(1) << 31) ? static_cast<unsigned>(x_rows * a.ldx * ES) : 0u;
  int resident = 0;
  const int rc = quad_grid<T, EPI>(&resident);
  if (rc != FR_OK) return rc;
  constexpr int COLS = (EPI == EPI_SILU) ? C::BF / 2 : C::BF;
  const int64_t worst = static_cast<int64_t>(a.num_t_blocks) * a.num_f_tiles;
  // After many whole rounds the workgroups are no longer in step (half tiles, hand-overs), and cutting the last
  // round buys less than its slices' fp32 round trip costs - the sooner the shorter a tile's K loop is: gate/up
  // (64 K tiles) with / without the split 681 / 684 us at 8.8 rounds (1536 tokens), 832 / 816 at 10.5, 1030 / 988
  // at 12.5, 1521 / 1505 at 17.5, 5743 / 5723 at 70; the down projection (224 K tiles) 785 / 915 at 2.7 rounds,
  // 2803 / 2979 at 11; fp8 down projection (112 K tiles) 1743 / 1794 at 8.5 rounds; 96 K tiles (H = 6144) 1138 / 1135
  // at 10 rounds, 1442 / 1437 at 12.
  const int64_t max_rounds = a.K / BK >= FQ_TAIL_LONG_K ? 16 : FQ_TAIL_ROUNDS_SHORT;
  const bool tail = a.tail_ws && a.K / BK >= kTailMinTiles && a.N % COLS == 0 && worst < max_rounds * static_cast<int64_t>(resident);
  if (!tail) a.tail_ws = nullptr;
  int64_t grid = resident;
  if (tail) {
    if (grid > kTailUnits) grid = kTailUnits;
  } else if (grid > (worst + 7) / 8 * 8) {
    grid = (worst + 7) / 8 * 8;
  }
  hipLaunchKernelGGL((moe_gemm_quad_kernel<T, EPI>), dim3(static_cast<unsigned>(grid)), dim3(C::NT), C::LDS_BYTES + kQuadSink, st, a FR_PROF_ARG);
  int lrc = check_launch("moe_gemm_quad_kernel");
  if (lrc != FR_OK || !tail) return lrc;
  const int nper = static_cast<int>(grid / 8);
  if (nper >= 2) {
    hipLaunchKernelGGL((tail_fixup_kernel<T, C, EPI>), dim3(8 * (nper / 2) * (C::BT / kFixupRows)), dim3(256), 0, st, a, nper);
    lrc = check_launch("tail_fixup_kernel");
  }
  return lrc;
}

}  // namespace fr
