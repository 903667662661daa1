// Tile table of the grouped expert GEMMs and the launch of one (element type, epilogue)
// combination.  Each combination is instantiated in its own translation unit
// (moe_gemm_inst_*.hip) so that the library builds in parallel; moe_gemm.hip sees only
// the declaration of dispatch_block.
#pragma once
#include "moe_gemm_quad.h"

namespace fr {

// ---- host side ----------------------------------------------------------------
// Token-block sizes and their tile shapes.  K tiles are 128 bytes per row (256 for
// the 16-row block); every block except 64 streams tiles HBM -> LDS directly.
//   256 / 128 rows: 8 wavefronts, 32x32 MFMA, 2- or 3-slot ring (compute-bound regime);
//                   in the 256-row tile one wavefront per SIMD issues the loads of both;
//   64 rows:        3-slot ring, 8 wavefronts (4 with 256-byte row segments for the gate/up GEMM, persistent);
//                   (the register-staged double buffer of STAGES == 0 is no longer used by any tile);
//   32 / 16 rows:   decode regime, 16x16 MFMA, 3-slot ring, two workgroups per CU:
//                   weight streaming at HBM rate.  The gate/up GEMM (short weight rows
//                   of H elements, many of them) streams faster with 512-byte row
//                   segments: T32L / T16L, used when H allows.
template <typename T> struct Tiles {  // bf16 / fp16
  typedef Cfg<256, 256, 128, 2, 4, 32, 1, 2, 0, 2> T256;
  // The same tile on v_mfma_f32_16x16x32: half the accumulator-register traffic per flop of the 32x32x16 shape.
  // The part's clock under MFMA load follows the power drawn: a pure stream of 16x16x32 MFMAs holds 2.0 GHz where
  // 32x32x16 holds 1.4-1.8 GHz.  One fragment buffer (the second would not fit next to 128 accumulators and two
  // address sets).  Gate/up at 4096 / 16384 tokens: -2.5 % / -5 %, down projection -3 % / -4 %; with a short K loop
  // (2048: half as many K tiles to spread a tile's hand-over on) it loses 4 %, hence kSmallMfmaMinK.
  typedef Cfg<256, 256, 128, 2, 4, 16, 1, 2, 0, 2> T256S;
  typedef T256 T256G;
  typedef Cfg<128, 256, 128, 2, 4, 32, 1, 3, 3> T128;
  typedef Cfg<128, 256, 128, 2, 4, 16, 1, 3, 0, 2> T128P;  // persistent form; one wavefront per SIMD issues the loads (2-4 % over each its own); 16x16x32 MFMAs: 2-3 % over 32x32x16
  // 160 token rows on the same three-slot ring: 159744 bytes, with the walk table all 160 KB of a CU.  A quarter more
  // rows per pass of an expert's weight tiles through LDS, and room for the spread of the experts' loads around a
  // multiple of 128 (n pairs on E experts: n/E +- sqrt(n/E) rows each, so with n/E = 128, 256, 512 every other expert
  // needs one 128-row block more than n/E / 128).  Five token tiles x four weight tiles per wavefront, five of the
  // thirteen loads per issuing wavefront and K tile for the token rows.
  typedef Cfg<160, 256, 128, 2, 4, 16, 1, 3, 0, 2> T160P;
  typedef Cfg<64, 256, 128, 2, 4, 32, 1, 3, 3> T64;    // 3-slot ring like the 128-row tile (5 % over the register-staged form)
  typedef Cfg<64, 128, 256, 2, 2, 32, 1, 3> T64U;      // gate/up: 256-byte row segments, 4 wavefronts (another 5 %)
  typedef Cfg<32, 128, 128, 1, 4, 16, 2, 3> T32;
  typedef Cfg<16, 64, 256, 1, 2, 16, 2, 3> T16;
  typedef Cfg<32, 128, 512, 1, 4, 16, 1, 2> T32L;
  typedef Cfg<16, 64, 512, 1, 2, 16, 2, 2> T16L;
};
template <> struct Tiles<fp8_t> {  // the 16x16x128 MFMA eats 256 bytes of K per two K-steps
  // every wavefront issues its own tile loads: half the address registers per wavefront (the persistent down
  // projection spills 16 instead of 57 registers: 586 vs 595 us at M=4096 although no wavefront can then skip an
  // all-padding half tile; the plain gate/up kernel is unchanged)
  typedef Cfg<256, 256, 128, 2, 4, 32, 1, 2, 0, 1> T256G;  // gate/up GEMM (plain kernel, two fragment buffers)
  typedef Cfg<256, 256, 128, 2, 4, 32, 1, 2, 0, 1> T256;
  typedef T256 T256S;
  typedef Cfg<128, 256, 128, 2, 4, 32, 1, 3, 3> T128;
  typedef Cfg<128, 256, 128, 2, 4, 32, 1, 3, 0, 2> T128P;
  typedef Cfg<160, 256, 128, 2, 4, 16, 1, 3, 0, 2> T160P;  // on the 16x16x128 MFMA (80 rows per wavefront are no multiple of 32)
  typedef Cfg<64, 256, 128, 2, 4, 32, 1, 3, 3> T64;
  typedef Cfg<64, 128, 256, 2, 2, 32, 1, 3> T64U;
  typedef Cfg<32, 128, 256, 1, 4, 16, 2, 2> T32;
  typedef Cfg<16, 64, 256, 1, 2, 16, 2, 3> T16;
  typedef Cfg<32, 128, 512, 1, 4, 16, 1, 2> T32L;
  typedef Cfg<16, 64, 512, 1, 2, 16, 2, 2> T16L;
};

constexpr int kSmallMfmaMinK = 4096;  // K from which the 256-row tile of 2-byte operands takes the 16x16x32 MFMA form

inline bool valid_block(int block) { return block == 16 || block == 32 || block == 64 || block == 128 || block == 160 || block == 256; }
inline int elem_bytes(int dtype) { return dtype == FR_FP8_E4M3 ? 1 : 2; }
inline int tile_k_bytes(int block, int dtype) { return (block == 16 || (block == 32 && dtype == FR_FP8_E4M3)) ? 256 : 128; }
inline int k_multiple(int dtype, int block) { return tile_k_bytes(block, dtype) / elem_bytes(dtype); }

template <typename T, int EPI>
int dispatch_block(GemmArgs a, int block, int splits, int64_t sorted_len, hipStream_t st) {
  typedef Tiles<T> TL;
  auto fill = [&](int BT, int BF, int bkb) {
    const int bk = bkb / static_cast<int>(sizeof(T));
    a.num_t_blocks = static_cast<int>(ceil_div(sorted_len, BT));
    const int fper = (EPI == EPI_SILU) ? BF / 2 : BF;
    a.num_f_tiles = static_cast<int>(ceil_div(a.N, fper));
    a.group_t = tunables().group_m ? tunables().group_m : (BT >= 64 ? 4 : 8);
    a.k_per_split = static_cast<int>(round_up(ceil_div(a.K, splits), bk));
  };
  switch (block) {
    case 256:
      fill(256, TL::T256::BF, TL::T256::BKB);
      // One workgroup per CU: the persistent form hides each tile's ring fill and drain behind its
      // neighbour's.  fp8 runs it with one fragment buffer (registers for the second address set): 4-5 %
      // faster for the down projection, but 6 % slower for the gate/up GEMM (short K, register-starved
      // epilogue: the hand-off K tiles spill; without the hand-off it is within 1 % of the plain kernel),
      // which keeps the plain kernel.
      // one wavefront per SIMD, 128 x 128 outputs each (see moe_gemm_quad.h), where its K loop is long enough
      if (!tunables().no_quad) {
        const int rc = launch_gemm_quad<T, EPI>(a, splits, st);
        if (rc != 1) return rc;
      }
      if constexpr (sizeof(T) == 1 && EPI == EPI_SILU) return launch_gemm<T, typename TL::T256G, EPI>(a, splits, st);
      else {
        // 2-byte operands, long K: the 16x16x32 MFMA form (see Tiles::T256S)
        if constexpr (sizeof(T) == 2) {
          if (a.K >= kSmallMfmaMinK) return launch_gemm_persistent<T, typename TL::T256S, EPI>(a, splits, st);
        }
        return launch_gemm_persistent<T, typename TL::T256, EPI>(a, splits, st);
      }
    case 128:
      fill(128, TL::T128::BF, TL::T128::BKB);
      // The gate/up GEMM always takes the persistent form (its walk by expert fetches each expert's
      // weights once per chunk of token blocks); the down projection of the layer (few feature tiles,
      // long K) takes it for the split of the last round, a plain grouped GEMM keeps the plain kernel.
      if constexpr (EPI != EPI_SILU) {
        if (a.long_k) return launch_gemm_persistent<T, typename TL::T128P, EPI>(a, splits, st);
      } else {
        return launch_gemm_persistent<T, typename TL::T128P, EPI>(a, splits, st);
      }
      return launch_gemm<T, typename TL::T128, EPI>(a, splits, st);
    case 160:
      fill(160, TL::T160P::BF, TL::T160P::BKB);
      return launch_gemm_persistent<T, typename TL::T160P, EPI>(a, splits, st);
    case 64:
      // The persistent form hides each tile's ring fill behind its predecessor's last K tiles: the 64-row gate/up
      // GEMM streams the weights at 6.3 instead of 5.9 TB/s (128 tokens: 318 -> 298 us, fp8 192 -> 170 us).  The
      // down projection's 64-row tile gains nothing from it (147 us either way) and stays plain.
      if (EPI == EPI_SILU && a.K % (TL::T64U::BKB / static_cast<int>(sizeof(T))) == 0) {
        fill(64, TL::T64U::BF, TL::T64U::BKB);
        return launch_gemm_persistent<T, typename TL::T64U, EPI>(a, splits, st);
      }
      fill(64, TL::T64::BF, TL::T64::BKB);
      return launch_gemm<T, typename TL::T64, EPI>(a, splits, st);
    case 32:
      if (EPI == EPI_SILU && a.K % (TL::T32L::BKB / static_cast<int>(sizeof(T))) == 0) {
        fill(32, TL::T32L::BF, TL::T32L::BKB);
        return launch_gemm<T, typename TL::T32L, EPI>(a, splits, st);
      }
      fill(32, TL::T32::BF, TL::T32::BKB);
      return launch_gemm<T, typename TL::T32, EPI>(a, splits, st);
    case 16:
      if (EPI == EPI_SILU && a.K % (TL::T16L::BKB / static_cast<int>(sizeof(T))) == 0) {
        fill(16, TL::T16L::BF, TL::T16L::BKB);
        return launch_gemm<T, typename TL::T16L, EPI>(a, splits, st);
      }
      fill(16, TL::T16::BF, TL::T16::BKB);
      return launch_gemm<T, typename TL::T16, EPI>(a, splits, st);
    default: return fail(FR_E_SHAPE, "routing block %d not in {16, 32, 64, 128, 160, 256}", block);
  }
}

// Per-device set-up (dynamic LDS limits, occupancy queries) of every kernel dispatch_block<T, EPI> can launch,
// so that no later call has anything left to set up - e.g. a first call under graph capture.
template <typename T, int EPI>
int prepare_tiles() {
  typedef Tiles<T> TL;
  GemmArgs a = {};
  a.setup_only = 1;
  int rc = launch_gemm_persistent<T, typename TL::T256, EPI>(a, 1, nullptr);
  if constexpr (sizeof(T) == 2) {
    if (rc == FR_OK) rc = launch_gemm_persistent<T, typename TL::T256S, EPI>(a, 1, nullptr);
  }
  if (rc == FR_OK) rc = launch_gemm_quad<T, EPI>(a, 1, nullptr);
  if (rc == FR_OK) rc = launch_gemm_persistent<T, typename TL::T128P, EPI>(a, 1, nullptr);
  if (rc == FR_OK) rc = launch_gemm_persistent<T, typename TL::T160P, EPI>(a, 1, nullptr);
  if (rc == FR_OK) rc = launch_gemm<T, typename TL::T128, EPI>(a, 1, nullptr);
  if (rc == FR_OK) rc = launch_gemm<T, typename TL::T64, EPI>(a, 1, nullptr);
  if (rc == FR_OK) rc = launch_gemm<T, typename TL::T32, EPI>(a, 1, nullptr);
  if (rc == FR_OK) rc = launch_gemm<T, typename TL::T16, EPI>(a, 1, nullptr);
  if constexpr (EPI == EPI_SILU) {
    if (rc == FR_OK) rc = launch_gemm_persistent<T, typename TL::T64U, EPI>(a, 1, nullptr);
    if (rc == FR_OK) rc = launch_gemm<T, typename TL::T32L, EPI>(a, 1, nullptr);
    if (rc == FR_OK) rc = launch_gemm<T, typename TL::T16L, EPI>(a, 1, nullptr);
  }
  return rc;
}

}  // namespace fr
