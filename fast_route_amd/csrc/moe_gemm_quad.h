// Persistent grouped GEMM with ONE wavefront per SIMD: 256 sorted slots x 256 features per workgroup,
// four wavefronts of 128 x 128 each (2-byte operands).
//
// Why.  In the eight-wavefront tile a wavefront owns 128 x 64 outputs and reads six operand
// fragments from LDS for every eight MFMAs; with 128 x 128 per wavefront it reads eight for sixteen,
// a third less LDS traffic for the same arithmetic, and the part's clock under MFMA load follows the
// bytes it moves.  The 256 accumulator registers of a lane live in the accumulation half of the
// register file (one wavefront per SIMD has 512 registers per lane), which leaves the 256 ordinary
// registers for the pipeline below.
//
// Pipeline.  With a single wavefront per SIMD nobody fills the issue slots a burst of tile loads or a
// wait leaves, so the wavefront's own instruction stream has to be even: per K tile of 64 elements it
// holds 64 MFMAs, 32 fragment reads and 16 tile loads, and no two memory instructions are adjacent.
// A lane keeps the fragments of a WHOLE K tile in registers (4 K-steps x 8 fragments x 4 registers).
// While K tile t is multiplied from registers, every fragment is re-read - K tile t+1, from the other
// LDS slot - right after the last MFMA of the K-step that used it, i.e. a whole K tile (2048 MFMA
// cycles) ahead of its use: no MFMA ever waits for LDS.  The slot that held K tile t was read out
// during K tile t-1, so it is free for the loads of K tile t+2 from the one barrier of the period
// (after the first four MFMAs, when the last fragment reads of the previous period have long
// returned) onwards, and those loads go out one at a time between MFMAs over the first half of the
// period.  The ring is handed from one output tile to the workgroup's next one the same way: the
// last two periods load the next tile's first two K tiles and the last one reads its first
// fragments, so only the epilogue itself separates the MFMAs of two tiles.
//
// Same tile walk, tail split, LDS swizzle, epilogues and fix-up kernel as moe_gemm_persistent_kernel;
// results are bit-identical to it (same MFMA shape, same K order per accumulator).
#pragma once
#include "moe_gemm_persistent.h"

namespace fr {

template <int TILE> struct QuadCfgOf { typedef Cfg<256, 256, 128, 2, 2, TILE, 1, 2, 0, 1> type; };
#ifndef FR_QUAD_TILE
#define FR_QUAD_TILE 16  // MFMA shape: 16 = 16x16x32, 32 = 32x32x16
#endif
typedef QuadCfgOf<FR_QUAD_TILE>::type QuadCfg;

#ifndef FR_QUAD_LOAD_EVERY
#define FR_QUAD_LOAD_EVERY (FR_QUAD_TILE == 16 ? 4 : 2)  // one tile load after every n-th MFMA, from the barrier on
#endif

// measurement switches (results are wrong with any of them)
#ifdef FQ_NOLOAD
#define FQ_DO_LOAD false
#else
#define FQ_DO_LOAD true
#endif
#ifdef FQ_NOREAD
#define FQ_DO_READ false
#else
#define FQ_DO_READ true
#endif
#ifdef FQ_NOBAR
#define FQ_BARRIER
#else
#define FQ_BARRIER __builtin_amdgcn_s_barrier(); __builtin_amdgcn_sched_barrier(0);
#endif
#ifdef FQ_NOWAIT
#define FQ_WAIT
#else
#define FQ_WAIT asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
#endif
#ifndef FQ_BAR_AT
#define FQ_BAR_AT (FR_QUAD_TILE == 16 ? 7 : 3)
#endif

template <typename T, int EPI>
__global__ __launch_bounds__(256, 1) void moe_gemm_quad_kernel(const GemmArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef QuadCfg C;
  typedef Elem<T> E;
  typedef __attribute__((address_space(3))) void* lptr_t;
  static_assert(sizeof(T) == 2, "2-byte operands");
  constexpr int BT = C::BT, BF = C::BF, CPR = C::CPR, BK = C::BKB / 2, EPC = 8;
  constexpr int TILE = C::TILE, NF = 128 / TILE;  // MFMA tile edge; fragments per operand and K-step
  constexpr int KG = C::KGROUPS, KS = CPR / KG;   // lane groups along K in one MFMA; K-steps per K tile
  constexpr int NM = NF * NF;                     // MFMAs per K-step
  typedef typename std::conditional<TILE == 32, f32x16, f32x4>::type acc_t;
  constexpr int NW = 4, XI = C::XI, WI = C::WI, NL = XI + WI;  // tile loads per wavefront and K tile: 8 + 8
  constexpr int LE = FR_QUAD_LOAD_EVERY;
  static_assert(C::IT == NF && C::JF == NF && XI == 8 && WI == 8 && KS * KG == CPR, "128 x 128 per wavefront");
  static_assert(FQ_BAR_AT + 1 + (NL - 1) * LE < KS * NM, "the loads of a period must fit the period");

  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  constexpr int XBYTES = C::XCH * 16, WBYTES = C::WCH * 16, WBASE_B = 2 * XBYTES;  // X slots, then W slots

  // ---- schedule (as in moe_gemm_persistent_kernel) -----------------------------------------
  const int npost = a.npost[0];
  const int nt = min(npost / BT, a.num_t_blocks);
  const int total = nt * a.num_f_tiles;
  const int xcd = blockIdx.x & 7, nper = gridDim.x >> 3, loc = blockIdx.x >> 3;
  const int k_all = a.K / BK;
  const XcdSchedule xs = xcd_schedule(total, nper, xcd, k_all, a.tail_ws != nullptr);
  const int n_units = xs.rounds + (loc < xs.rest * xs.slices ? 1 : 0);
  if (n_units == 0) return;
  __shared__ int expert_off[kWalkTable];
  expert_block_offsets(a, nt, expert_off, threadIdx.x, C::NT);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave_u = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wt = wave_u >> 1, wf = wave_u & 1;
  const T* X = static_cast<const T*>(a.X);

#define FQ_UNIT(j_, pt_, pf_, ex_, kb_, kn_, tu_)                                              \
  {                                                                                            \
    int lin_;                                                                                  \
    if ((j_) < xs.rounds) {                                                                    \
      lin_ = xs.base + (j_) * nper + loc;                                                      \
      kb_ = 0; kn_ = k_all; tu_ = -1;                                                          \
    } else {                                                                                   \
      const int t_ = loc % xs.rest, s_ = loc / xs.rest;                                        \
      lin_ = xs.base + xs.rounds * nper + t_;                                                  \
      kb_ = s_ * k_all / xs.slices;                                                            \
      kn_ = (s_ + 1) * k_all / xs.slices - kb_;                                                \
      tu_ = xs.slices > 1 ? s_ * xs.rest + t_ : -1;                                            \
    }                                                                                          \
    tile_coords(a, expert_off, lin_, pt_, pf_, ex_);                                           \
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
  const int frow = lane % TILE, kgrp = lane / TILE;
  const int xrow0 = wt * C::TT + frow, wrow0 = acc_tile_col<C, EPI>(wf, 0) + frow;
  const int xkey0 = swizzle<CPR>(xrow0, 0), wkey0 = swizzle<CPR>(wrow0, 0);
  int xadr[KS], wadr[KS];  // byte addresses in slot 0
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    xadr[s] = (xrow0 * CPR + ((s * KG + kgrp) ^ xkey0)) * 16;
    wadr[s] = WBASE_B + (wrow0 * CPR + ((s * KG + kgrp) ^ wkey0)) * 16;
  }
#define FQ_XD(i_) ((i_) * TILE * CPR * 16)
#define FQ_WD(j_) ((acc_tile_col<C, EPI>(0, (j_)) - acc_tile_col<C, EPI>(0, 0)) * CPR * 16)

  auto mma = [](const u32x4* wa, const u32x4* xb, acc_t c) -> acc_t {
    if constexpr (TILE == 32) return E::m32(wa, xb, c);
    else return E::m16(wa, xb, c);
  };
  acc_t acc[NF][NF];
  u32x4 rw[KS][NF], rx[KS][NF];

  int pid_t, pid_f, expert, kb, kn, tu;
  int n_pid_t = 0, n_pid_f = 0, n_expert = 0, n_kb = 0, n_kn = 0, n_tu = -1;
  int n_sid[XI];
  unsigned xsrcA[XI], wsrcA[WI], xsrcB[XI], wsrcB[WI];
  __amdgpu_buffer_rsrc_t xrsA, wrsA, xrsB, wrsB;
#define FQ_MAKE_SET(pt_, pf_, ex_, kb_, SIDOF, xsrc_, wsrc_, xrs_, wrs_)                                     \
  {                                                                                                          \
    const int64_t xrow0_ = a.top_k > 0 ? 0 : static_cast<int64_t>(pt_) * BT;                                 \
    const int64_t kfirst_ = static_cast<int64_t>(kb_) * BK;                                                  \
    xrs_ = uniform_rsrc(X + xrow0_ * a.ldx);                                                                 \
    wrs_ = uniform_rsrc(static_cast<const T*>(a.W) + static_cast<int64_t>(ex_) * a.w_expert_stride);         \
    _Pragma("unroll") for (int q = 0; q < XI; ++q) {                                                         \
      FQ_SLOT_ROW(q, rr, c)                                                                                  \
      int64_t row_ = rr;                                                                                     \
      if (a.top_k > 0) {                                                                                     \
        const int sid_ = SIDOF;                                                                              \
        row_ = sid_ < a.num_valid ? sid_ / a.top_k : 0;                                                      \
      }                                                                                                      \
      xsrc_[q] = static_cast<unsigned>((row_ * a.ldx + kfirst_ + c * EPC) * 2);                              \
    }                                                                                                        \
    _Pragma("unroll") for (int q = 0; q < WI; ++q) {                                                         \
      FQ_SLOT_ROW(q, rr, c)                                                                                  \
      wsrc_[q] = static_cast<unsigned>((static_cast<int64_t>(w_src_row(pf_, rr)) * a.ldw + kfirst_ + c * EPC) * 2); \
    }                                                                                                        \
  }
  // tile load q (weight rows first) of K tile tile_ of set SET into ring slot slot_
#define FQ_ISSUE(SET, tile_, slot_, q_)                                                                     \
  {                                                                                                         \
    if ((q_) < WI) {                                                                                        \
      __builtin_amdgcn_raw_ptr_buffer_load_lds(                                                             \
          wrs##SET, (lptr_t)(lds_raw + WBASE_B + (slot_) * WBYTES + ((q_) * NW + wave_u) * (kWave * 16)),   \
          16, wsrc##SET[(q_) < WI ? (q_) : 0], (tile_) * C::BKB, 0, 0);                                     \
    } else {                                                                                                \
      __builtin_amdgcn_raw_ptr_buffer_load_lds(                                                             \
          xrs##SET, (lptr_t)(lds_raw + (slot_) * XBYTES + (((q_) - WI) * NW + wave_u) * (kWave * 16)),      \
          16, xsrc##SET[(q_) < WI ? 0 : (q_) - WI], (tile_) * C::BKB, 0, 0);                                \
    }                                                                                                       \
  }
#define FQ_READ_W(s_, j_, sb_) rw[s_][j_] = *reinterpret_cast<const u32x4*>(lds_raw + (wadr[s_] + (sb_) * WBYTES + FQ_WD(j_)));
#define FQ_READ_X(s_, i_, sb_) rx[s_][i_] = *reinterpret_cast<const u32x4*>(lds_raw + (xadr[s_] + (sb_) * XBYTES + FQ_XD(i_)));
  // One period: K tile t is multiplied from registers.  FIRST: the accumulators start from zero.  READ: the
  // fragments of the following K tile are read from slot par ^ 1 as their registers fall free.  LSET (0: none): the
  // 16 loads of K tile ltile_ of set LSET go into slot par, one after every LE-th MFMA from the barrier on.
#define FQ_PERIOD(FIRST, READ, HAVE_LOAD, LSET, ltile_)                                        \
  {                                                                                            \
    const int rs_ = par ^ 1, ls_ = par;                                                        \
    _Pragma("unroll") for (int s = 0; s < KS; ++s) {                                           \
      _Pragma("unroll") for (int m = 0; m < NM; ++m) {                                         \
        const int j = m / NF, i = m % NF, g = s * NM + m;                                      \
        if ((FIRST) && s == 0) {                                                               \
          acc_t z_;                                                                            \
          _Pragma("unroll") for (int r = 0; r < (TILE == 32 ? 16 : 4); ++r) z_[r] = 0.f;        \
          acc[j][i] = mma(&rw[s][j], &rx[s][i], z_);                                           \
        } else {                                                                               \
          acc[j][i] = mma(&rw[s][j], &rx[s][i], acc[j][i]);                                    \
        }                                                                                      \
        __builtin_amdgcn_sched_barrier(0);                                                     \
        if (g == FQ_BAR_AT) {                                                                  \
          FQ_WAIT                                                                              \
          FQ_BARRIER                                                                           \
          __builtin_amdgcn_sched_barrier(0);                                                   \
        }                                                                                      \
        if ((READ) && FQ_DO_READ) {                                                            \
          if (i == NF - 1) FQ_READ_W(s, j, rs_)                                                \
          if (j == NF - 1) FQ_READ_X(s, i, rs_)                                                \
          if (i == NF - 1 || j == NF - 1) __builtin_amdgcn_sched_barrier(0);                             \
        }                                                                                      \
        if ((HAVE_LOAD) && FQ_DO_LOAD) {                                                       \
          if (g >= FQ_BAR_AT + 1 && (g - FQ_BAR_AT - 1) % LE == 0 && (g - FQ_BAR_AT - 1) / LE < NL) { \
            FQ_ISSUE(LSET, ltile_, ls_, (g - FQ_BAR_AT - 1) / LE)                                      \
            __builtin_amdgcn_sched_barrier(0);                                                 \
          }                                                                                    \
        }                                                                                      \
      }                                                                                        \
    }                                                                                          \
    par ^= 1;                                                                                  \
  }
  // One output tile (or K slice of one): kn >= 3 K tiles.
#define FQ_TILE(NEXT)                                                                                      \
  {                                                                                                        \
    if (NEXT) {                                                                                            \
      FQ_UNIT(unit + 1, n_pid_t, n_pid_f, n_expert, n_kb, n_kn, n_tu)                                      \
      if (a.top_k > 0) {                                                                                   \
        _Pragma("unroll") for (int q = 0; q < XI; ++q) {                                                   \
          FQ_SLOT_ROW(q, rr, c)                                                                            \
          (void)c;                                                                                         \
          n_sid[q] = a.sorted[n_pid_t * BT + rr];                                                          \
        }                                                                                                  \
      }                                                                                                    \
    }                                                                                                      \
    FQ_PERIOD(true, true, true, A, 2)                                                                      \
    if (NEXT) FQ_MAKE_SET(n_pid_t, n_pid_f, n_expert, n_kb, n_sid[q], xsrcB, wsrcB, xrsB, wrsB)            \
    __builtin_amdgcn_s_waitcnt(0xC07F); /* lgkmcnt(0): no scalar load pending inside the loop */           \
    for (int t = 1; t < kn - 2; ++t) FQ_PERIOD(false, true, true, A, t + 2)                                \
    if (NEXT) {                                                                                            \
      FQ_PERIOD(false, true, true, B, 0)                                                                   \
      FQ_PERIOD(false, true, true, B, 1)                                                                   \
    } else {                                                                                               \
      FQ_PERIOD(false, true, false, A, 0)                                                                  \
      FQ_PERIOD(false, false, false, A, 0)                                                                 \
    }                                                                                                      \
    if (tu < 0) gemm_epilogue<T, C, EPI, true>(a, acc, pid_t, pid_f, expert, 0, wt, wf, frow, kgrp);       \
    else tail_store<C, EPI>(a.tail_ws + static_cast<int64_t>(xcd * nper + tu) * (BT * BF), acc, wt, wf, frow, kgrp); \
  }

  FQ_UNIT(0, pid_t, pid_f, expert, kb, kn, tu)
  FQ_MAKE_SET(pid_t, pid_f, expert, kb, a.sorted[pid_t * BT + rr], xsrcA, wsrcA, xrsA, wrsA)
  // fill: K tiles 0 and 1 into slots 0 and 1, then all fragments of K tile 0
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int q = 0; q < NL; ++q) FQ_ISSUE(A, t, t, q)
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NL) : "memory");
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int s = 0; s < KS; ++s)
#pragma unroll
    for (int f = 0; f < NF; ++f) {
      FQ_READ_W(s, f, 0)
      FQ_READ_X(s, f, 0)
    }
  int par = 0;
  int unit = 0;
  for (; unit + 1 < n_units; ++unit) {
    FQ_TILE(true)
    pid_t = n_pid_t; pid_f = n_pid_f; expert = n_expert; xrsA = xrsB; wrsA = wrsB;
    kb = n_kb; kn = n_kn; tu = n_tu;
#pragma unroll
    for (int q = 0; q < XI; ++q) xsrcA[q] = xsrcB[q];
#pragma unroll
    for (int q = 0; q < WI; ++q) wsrcA[q] = wsrcB[q];
  }
  FQ_TILE(false)
#undef FQ_TILE
#undef FQ_PERIOD
#undef FQ_READ_X
#undef FQ_READ_W
#undef FQ_ISSUE
#undef FQ_MAKE_SET
#undef FQ_XD
#undef FQ_WD
#undef FQ_SLOT_ROW
#undef FQ_UNIT
#endif
}

// Workgroups resident at once on the current device: one per CU (a multiple of 8, one share per XCD).
template <typename T, int EPI>
int quad_grid(int* grid_out) {
  typedef QuadCfg C;
  constexpr int kMaxDevices = 64;
  static int cached[kMaxDevices] = {};
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail(FR_E_LAUNCH, "quad GEMM: device %d (%s)", dev, hipGetErrorString(e));
  if (!cached[dev]) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(&moe_gemm_quad_kernel<T, EPI>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
    int cus = 0, per_cu = 0;
    if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e == hipSuccess)
      e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, moe_gemm_quad_kernel<T, EPI>, C::NT, C::LDS_BYTES);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      return fail(FR_E_LAUNCH, "quad GEMM set-up (%d B LDS): %s", C::LDS_BYTES, hipGetErrorString(e));
    }
    if (per_cu < 1 || cus < 8) return fail(FR_E_LAUNCH, "quad GEMM: occupancy %d on %d CUs", per_cu, cus);
    cached[dev] = cus / 8 * 8;  // one workgroup per CU: a second would share the SIMDs' MFMA pipes
  }
  *grid_out = cached[dev];
  return FR_OK;
}

// Launches the one-wavefront-per-SIMD form for a single K split of at least 4 K tiles per unit; the caller falls
// back to launch_gemm_persistent otherwise (returns 1: nothing launched).
template <typename T, int EPI>
int launch_gemm_quad(const GemmArgs& a_in, int splits, hipStream_t st) {
  typedef QuadCfg C;
  GemmArgs a = a_in;
  constexpr int BK = C::BKB / 2;
  if (a.setup_only) {
    int resident = 0;
    return quad_grid<T, EPI>(&resident);
  }
  if (splits != 1 || a.K % BK != 0 || a.K / BK < 4 || a.num_experts < 1 || a.num_experts > kMaxExperts) return 1;
  const int64_t x_rows = a.top_k > 0 ? a.num_valid / a.top_k : C::BT;
  const int64_t w_rows = EPI == EPI_SILU ? 2 * static_cast<int64_t>(a.N) : a.N;
  const int64_t lim = int64_t(1) << 32;
  if (x_rows * a.ldx * 2 >= lim || w_rows * a.ldw * 2 >= lim)
    return fail(FR_E_SHAPE, "token rows (%lld x %lld) or one expert's weights (%lld x %lld) span 4 GiB or more",
                (long long)x_rows, (long long)a.ldx, (long long)w_rows, (long long)a.ldw);
  a.group_t = tunables().group_m ? tunables().group_m : kChunkBlocks;
  if (tunables().no_tail_split) a.tail_ws = nullptr;
  int resident = 0;
  const int rc = quad_grid<T, EPI>(&resident);
  if (rc != FR_OK) return rc;
  constexpr int COLS = (EPI == EPI_SILU) ? C::BF / 2 : C::BF;
  const bool tail = a.tail_ws && a.K / BK >= kTailMinTiles && a.N % COLS == 0;
  if (!tail) a.tail_ws = nullptr;
  const int64_t worst = static_cast<int64_t>(a.num_t_blocks) * a.num_f_tiles;
  int64_t grid = resident;
  if (tail) {
    if (grid > kTailUnits) grid = kTailUnits;
  } else if (grid > (worst + 7) / 8 * 8) {
    grid = (worst + 7) / 8 * 8;
  }
  hipLaunchKernelGGL((moe_gemm_quad_kernel<T, EPI>), dim3(static_cast<unsigned>(grid)), dim3(C::NT), C::LDS_BYTES, st, a);
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
