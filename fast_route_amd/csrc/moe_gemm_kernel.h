// Grouped expert GEMM kernel template for gfx950 MFMA.
//
// One workgroup computes a tile of BT sorted slots (one routing block, hence
// one expert) by BF output features.  Both operands are K-contiguous in HBM
// (tokens [*, K], weights [E, N, K]); K tiles of BKB bytes per row are staged
// through LDS in 16-byte chunks under an XOR swizzle and fed to v_mfma with the
// WEIGHT rows as the MFMA "A" operand and the TOKEN rows as "B", so a lane's
// accumulator registers hold 4 consecutive output features of one token and the
// epilogue stores 8/16-byte vectors.  Element types: bf16, fp16
// (v_mfma_f32_{32x32x16,16x16x32}) and OCP fp8 e4m3 (v_mfma_f32_{32x32x64,16x16x128}_f8f6f4,
// per-row fp32 scales of both operands applied in the epilogue).  Epilogues:
//   EPI_PLAIN  C[pair] = acc (* routed weight), scattered by sorted id
//   EPI_SILU   W tile = BF/2 gate rows + the matching BF/2 up rows; writes
//              silu(gate)*up at the slot's own row of act[sorted_len, F]
//   EPI_DOWN   partial[split][pair] = acc * routed weight in fp32 (split-K slices)
#pragma once
#include "fr_common.h"

#include <type_traits>

namespace fr {

enum { EPI_PLAIN = 0, EPI_SILU = 1, EPI_DOWN = 2 };

// Cache policy bits of the weight-tile loads (0 = default, 2 = non-temporal).  Tiles of up to 64 token
// rows stream every weight byte once (one or two blocks per expert): marked non-temporal the stream does
// not displace the token rows and its own neighbours in L2, and the 16-row gate/up GEMM goes from 6.5 to
// 6.9 TB/s, the down projection from 5.96 to 6.65 TB/s.  The larger tiles re-read weight tiles from L2
// for the other token blocks of an expert and keep the default (non-temporal in the persistent 128-row
// kernel: -2 % at M = 224..384 with one block per expert, +14 % at M = 512 on 8 experts).
#ifndef FR_W_AUX
#define FR_W_AUX (C::BT <= 64 ? 2 : 0)
#endif

struct GemmArgs {
  const void* X;        // token rows [*, K]
  int64_t ldx;          // row stride of X in elements
  const void* W;        // [E, w_rows, K]
  int64_t w_expert_stride;  // elements between experts
  int64_t ldw;          // row stride of W in elements
  void* out;
  int64_t ldo;          // row stride of out in elements
  int64_t split_stride; // EPI_DOWN: elements between split-K slices
  const int32_t* sorted;
  const int32_t* expert_ids;
  const int32_t* npost;
  const float* topk_w;  // flat [num_valid] or nullptr
  const float* x_scale; // fp8 only: one scale per X row (indexed like the X rows)
  const float* w_scale; // fp8 only: [E, w_rows]
  int w_rows;           // rows of W per expert (scale indexing)
  int num_valid;        // n = M*topk
  int top_k;            // X row = sorted id / top_k; 0 => X row = slot index
  int N;                // output features (EPI_SILU: F, W has 2F rows)
  int K;
  int k_per_split;      // multiple of BK
  int num_t_blocks;     // upper bound on routing blocks
  int num_f_tiles;
  int group_t;
  int mul_weight;
  int num_experts;      // E (persistent form: walk order by expert)
  int long_k;           // down projection (few feature tiles, long K): hint for the 128-row tile's form
  float* tail_ws;       // persistent form only: slice buffers for splitting the last round of tiles along K, or nullptr
  unsigned x_span;      // bytes of X the tile loads may address (from X in gather mode, from a block's first row otherwise), or 0:
                        // with it, the loads of padding slots fall outside the buffer resource and fetch nothing
  int add_div;          // EPI_PLAIN: 0 = store row `sorted id` of out; k > 0 = add into row (sorted id / k) of a zero-filled out (packed atomics)
  int w_tiled;          // W is in the prepared layout (see w_byte_offset), not [E, w_rows, K] row-major
  int setup_only;       // do the per-device set-up of the kernel a launch would take (LDS limit, occupancy) and launch nothing
};

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Prepared weight layout (fr_moe_prepare_weights): inside an expert, groups of kTileRows consecutive rows; inside a
// group, K tiles of kTileBytes per row; inside a K tile the group's rows one after the other.  A (row group, K tile)
// piece is 8 KB of consecutive memory, a group's whole K range one run of memory, where the row-major layout has a
// weight tile in as many 128-byte pieces as it has rows, one row length apart.
constexpr int kTileRows = 64, kTileBytes = 128, kTilePiece = kTileRows * kTileBytes;
// byte offset of byte kb of row `row` inside one expert's weights; es = bytes per element
__device__ __host__ __forceinline__ int64_t w_byte_offset(int w_tiled, int64_t ldw, int64_t K, int row, int64_t kb, int es) {
  if (w_tiled) {
    const int64_t ktiles = (K * es) / kTileBytes;
    return ((static_cast<int64_t>(row / kTileRows) * ktiles + kb / kTileBytes) * kTilePiece) + (row % kTileRows) * kTileBytes + kb % kTileBytes;
  }
  return static_cast<int64_t>(row) * ldw * es + kb;
}
struct fp8_t { unsigned char bits; };  // OCP e4m3fn storage

// Element traits: FC = 16-byte chunks one lane feeds to one MFMA, out_t = type the
// half-precision epilogues store.
template <typename T> struct Elem;
template <> struct Elem<bf16_t> {
  typedef bf16_t out_t;
  typedef bf16x4 out4;
  static constexpr int FC = 1;
  static constexpr bool SCALED = false;
  static __device__ __forceinline__ f32x16 m32(const u32x4* a, const u32x4* b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[0]), __builtin_bit_cast(bf16x8, b[0]), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 m16(const u32x4* a, const u32x4* b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a[0]), __builtin_bit_cast(bf16x8, b[0]), c, 0, 0, 0);
  }
};
template <> struct Elem<f16_t> {
  typedef f16_t out_t;
  typedef f16x4 out4;
  static constexpr int FC = 1;
  static constexpr bool SCALED = false;
  static __device__ __forceinline__ f32x16 m32(const u32x4* a, const u32x4* b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a[0]), __builtin_bit_cast(f16x8, b[0]), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 m16(const u32x4* a, const u32x4* b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a[0]), __builtin_bit_cast(f16x8, b[0]), c, 0, 0, 0);
  }
};
template <> struct Elem<fp8_t> {
  typedef bf16_t out_t;
  typedef bf16x4 out4;
  static constexpr int FC = 2;
  static constexpr bool SCALED = true;
  static __device__ __forceinline__ i32x8 join(const u32x4* p) {
    return __builtin_bit_cast(i32x8, __builtin_shufflevector(p[0], p[1], 0, 1, 2, 3, 4, 5, 6, 7));
  }
  // format selectors 0 = e4m3 for both operands; scale operands 0 = no block scaling
  static __device__ __forceinline__ f32x16 m32(const u32x4* a, const u32x4* b, f32x16 c) {
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(join(a), join(b), c, 0, 0, 0, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 m16(const u32x4* a, const u32x4* b, f32x4 c) {
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(join(a), join(b), c, 0, 0, 0, 0, 0, 0);
  }
};

// g * sigmoid(g).  The quotient is a multiplication by v_rcp_f32 (1 ulp) instead of the IEEE division's ten
// instructions: the result is rounded to 8 or 11 bits right after, and the epilogue's VALU time is MFMA idle time.
// out[0..3] += v (2-byte elements), two packed atomic adds.  With exactly two contributions to a zero-filled
// element the result does not depend on their order: 0 + a is exact, a + b is rounded once.
#if defined(__HIP_DEVICE_COMPILE__)
__device__ __forceinline__ void atomic_add4(bf16_t* p, bf16x4 v) {
  typedef short s2 __attribute__((ext_vector_type(2)));
  typedef __bf16 b2 __attribute__((ext_vector_type(2)));
  typedef __attribute__((address_space(1))) s2* gptr;
  const b2 lo = {v[0], v[1]}, hi = {v[2], v[3]};
  __builtin_amdgcn_global_atomic_fadd_v2bf16((gptr)(p), __builtin_bit_cast(s2, lo));
  __builtin_amdgcn_global_atomic_fadd_v2bf16((gptr)(p + 2), __builtin_bit_cast(s2, hi));
}
__device__ __forceinline__ void atomic_add4(f16_t* p, f16x4 v) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  typedef __attribute__((address_space(1))) h2* gptr;
  const h2 lo = {v[0], v[1]}, hi = {v[2], v[3]};
  __builtin_amdgcn_global_atomic_fadd_v2f16((gptr)(p), lo);
  __builtin_amdgcn_global_atomic_fadd_v2f16((gptr)(p + 2), hi);
}
#else
__device__ __forceinline__ void atomic_add4(bf16_t*, bf16x4) {}
__device__ __forceinline__ void atomic_add4(f16_t*, f16x4) {}
#endif

__device__ __forceinline__ float silu(float g) { return g * __builtin_amdgcn_rcpf(1.f + __expf(-g)); }

// Tile configuration.  BKB = bytes of K per row per tile (64 bf16 or 128 fp8 = 128 B,
// the L2 line: shorter row segments halve the L2->LDS rate).  TILE = 32 uses the
// 32x32 MFMA shapes, TILE = 16 the 16x16 ones.  WT x WF wavefronts split the BT x BF
// tile; MINB = workgroups per CU the register allocation should allow.
// STAGES == 0: tiles go HBM -> registers -> LDS with two LDS buffers (one tile in
// flight).  STAGES >= 2: tiles go HBM -> LDS directly (global_load_lds_dwordx4)
// through rings of STAGES token-tile and weight-tile slots; a slot is refilled once
// its tile's last fragments are in registers, the loads spread over SPREAD K-steps.
template <int BT_, int BF_, int BKB_, int WT_, int WF_, int TILE_, int MINB_ = 1, int STAGES_ = 0, int SPREAD_ = 0, int IW_ = 1>
struct Cfg {
  static constexpr int BT = BT_, BF = BF_, BKB = BKB_, WT = WT_, WF = WF_, TILE = TILE_, MINB = MINB_;
  static constexpr int STAGES = STAGES_;  // ring slots of the token and of the weight tiles
  static constexpr int IW = IW_;          // 2: only the first half of the wavefronts issue tile loads, each for two
  static constexpr int SPREAD = SPREAD_;  // K-steps over which the refill of a slot is spread (<= 1: one burst)
  static constexpr int NBUF = STAGES_ == 0 ? 2 : STAGES_;
  static constexpr int NT = WT * WF * kWave;       // threads
  static constexpr int NW = NT / kWave;
  static constexpr int TT = BT / WT, TF = BF / WF; // per-wave tile
  static constexpr int IT = TT / TILE, JF = TF / TILE;
  static constexpr int CPR = BKB / 16;             // 16-byte chunks per row
  static constexpr int KGROUPS = 64 / TILE;        // lane groups along K in one MFMA
  static constexpr int XCH = BT * CPR, WCH = BF * CPR;
  static constexpr int XL = (XCH + NT - 1) / NT, WL = (WCH + NT - 1) / NT;
  // direct-to-LDS loads per ISSUING wavefront and tile (an issuing wavefront issues for IW wavefronts: load ih covers
  // the 64 chunks of virtual wavefront (wave + (ih % IW) * NW / IW) in group ih / IW of NW * 64 chunks; with an odd
  // count - the 160-row token tile with IW = 2 - the last group is half a group, all of it virtual wavefronts 0..NW/IW-1)
  static constexpr int XIW = XCH * IW / (kWave * NW), WIW = WCH * IW / (kWave * NW);
  static constexpr int LDS_BYTES = (STAGES_ == 0 ? 2 : STAGES_) * (BT + BF) * BKB;
  static_assert(TT % TILE == 0 && TF % TILE == 0, "wave tile must be a multiple of the MFMA tile");
  static_assert(NT % CPR == 0, "threads must cover whole rows");
  static_assert(STAGES_ == 0 || (STAGES_ >= 2 && (XCH * IW) % (kWave * NW) == 0 && (WCH * IW) % (kWave * NW) == 0),
                "direct-to-LDS tiles must split evenly over the issuing wavefronts");
};

// LDS is 64 banks x 4 B: a 16-lane phase of ds_read_b128 is conflict-free when its
// 16 rows land on 16 different 16-byte columns of a 256-byte line.  Rows shorter
// than a line share it (16/CPR rows per line), so the XOR key is the line index.
template <int CPR>
__device__ __forceinline__ int swizzle(int row, int chunk) {
  constexpr int ROWS_PER_LINE = CPR >= 16 ? 1 : 16 / CPR;
  constexpr int MASK = CPR >= 16 ? 15 : CPR - 1;
  return chunk ^ ((row / ROWS_PER_LINE) & MASK);
}

// Epilogue of one tile: the lane holds token column (lane % TILE) of each token tile of its
// wavefront and, per accumulator group, 4 consecutive features.
#if defined(__HIP_DEVICE_COMPILE__)
// Buffer resource over the whole address space from `p` on.  The pointer is the same in every
// lane; reading it through the first lane tells the compiler so, which otherwise may keep the
// resource in vector registers and wrap each load in a loop over the distinct lane values.
// Byte offset given to the lanes of padding slots when GemmArgs::x_span is set: beyond any span (spans stay below
// 2 GiB), so the buffer's range check drops the load - no request, no bytes moved; what the LDS then holds for
// those rows only ever reaches accumulator columns of padding slots, which no epilogue stores as a pair's result.
constexpr unsigned kSkipOffset = 0x80000000u;
template <typename T>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t uniform_rsrc(const T* p, unsigned num_records = 0xFFFFFFFFu) {
  const uint64_t v = reinterpret_cast<uint64_t>(p);
  const uint64_t lo = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(static_cast<uint32_t>(v))));
  const uint64_t hi = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(static_cast<uint32_t>(v >> 32))));
  return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(hi << 32 | lo), 0, static_cast<int>(num_records), 0x00020000);
}
#endif

#if defined(__HIP_DEVICE_COMPILE__)
// The four registers of an accumulator tile that lives in the accumulation half of the register file, copied to
// ordinary registers here and now.  (Left to itself the register allocator moves every accumulator to an ordinary
// register right behind its last MFMA - a wait for the MFMA's result each, and 256 values that do not fit.)
__device__ __forceinline__ f32x4 acc_fetch(const f32x4& v) {
  f32x4 o;
  asm volatile("v_accvgpr_read_b32 %0, %4\n\tv_accvgpr_read_b32 %1, %5\n\tv_accvgpr_read_b32 %2, %6\n\tv_accvgpr_read_b32 %3, %7"
               : "=v"(o[0]), "=v"(o[1]), "=v"(o[2]), "=v"(o[3])
               : "a"(v[0]), "a"(v[1]), "a"(v[2]), "a"(v[3]));
  return o;
}
#else
__device__ __forceinline__ f32x4 acc_fetch(const f32x4& v) { return v; }
#endif
__device__ __forceinline__ f32x16 acc_fetch(const f32x16& v) {
  f32x16 o;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const f32x4 part = {v[g * 4 + 0], v[g * 4 + 1], v[g * 4 + 2], v[g * 4 + 3]};
    const f32x4 got = acc_fetch(part);
#pragma unroll
    for (int r = 0; r < 4; ++r) o[g * 4 + r] = got[r];
  }
  return o;
}

// AG: the accumulators live in the accumulation registers (one wavefront per SIMD) and are fetched tile by tile.
template <typename T, typename C, int EPI, bool HOIST = true, bool AG = false, typename AccT>
__device__ __forceinline__ void gemm_epilogue(const GemmArgs& a, AccT (&acc)[C::JF][C::IT], int pid_t, int pid_f,
                                              int expert, int split, int wt, int wf, int frow, int kgrp) {
  typedef Elem<T> E;
  typedef typename E::out_t out_t;
  typedef typename E::out4 out4;
  constexpr int BT = C::BT, BF = C::BF;
  constexpr int ACC_N = (C::TILE == 32) ? 16 : 4;
  // ---- epilogue -------------------------------------------------------------
  // lane holds token column (lane % TILE) of each token tile and, per accumulator
  // group g (TILE==32: 4 groups of 4 regs; TILE==16: one), 4 consecutive features
  // starting at g*8 + kgrp*4 (TILE==32) or kgrp*4 (TILE==16) inside the MFMA tile.
  constexpr int GROUPS = ACC_N / 4;
  // accumulators in the accumulation registers: results are fetched, computed and stored group by group
  constexpr bool kFence = AG;
  // fp8: with HOIST the scales of the lane's weight rows (the same for every token tile) and of its token rows
  // are fetched up front, all loads in flight together, instead of one by one between the stores (which the
  // compiler may not move them across).  That takes JF * ACC_N registers: the persistent kernel, which keeps
  // two address sets alive across its epilogue, does without.
  constexpr int NWS = (E::SCALED && HOIST) ? C::JF * GROUPS * 4 : 1;
  float wscale[NWS];
  float xscale[C::IT];
  int sids[C::IT];
#pragma unroll
  for (int i = 0; i < C::IT; ++i) {
    sids[i] = 0;
    xscale[i] = 1.f;
  }
  if constexpr (EPI != EPI_SILU || E::SCALED) {
#pragma unroll
    for (int i = 0; i < C::IT; ++i) sids[i] = a.sorted[pid_t * BT + wt * C::TT + i * C::TILE + frow];
  }
  float routed[C::IT];  // routed weight of the lane's pair in each token tile (all fetched before the first store)
#pragma unroll
  for (int i = 0; i < C::IT; ++i) {
    routed[i] = 1.f;
    if constexpr (EPI != EPI_SILU)
      if (a.mul_weight && sids[i] < a.num_valid) routed[i] = a.topk_w[sids[i]];
  }
  const float* wsc = nullptr;
  if constexpr (E::SCALED) wsc = a.w_scale + static_cast<int64_t>(expert) * a.w_rows;
  // scale of the weight row behind accumulator register (j, g, r)
  auto w_scale_at = [&](int j, int g, int r) -> float {
    int f;
    if constexpr (EPI == EPI_SILU) {
      constexpr int HJ = C::JF / 2;
      const int fl = pid_f * (BF / 2) + wf * (C::TF / 2) + (j % HJ) * C::TILE + g * 8 + kgrp * 4 + r;
      f = (j / HJ) * a.N + (fl < a.N ? fl : a.N - 1);
    } else {
      const int fl = pid_f * BF + wf * C::TF + j * C::TILE + g * 8 + kgrp * 4 + r;
      f = fl < a.N ? fl : a.N - 1;
    }
    return wsc[f];
  };
  auto w_scale = [&](int j, int g, int r) -> float {
    if constexpr (HOIST) return wscale[(j * GROUPS + g) * 4 + r];
    else return w_scale_at(j, g, r);
  };
  if constexpr (E::SCALED) {
    if constexpr (HOIST) {
#pragma unroll
      for (int j = 0; j < C::JF; ++j)
#pragma unroll
        for (int g = 0; g < GROUPS; ++g)
#pragma unroll
          for (int r = 0; r < 4; ++r) wscale[(j * GROUPS + g) * 4 + r] = w_scale_at(j, g, r);
    }
#pragma unroll
    for (int i = 0; i < C::IT; ++i) {
      if (a.top_k > 0) xscale[i] = sids[i] < a.num_valid ? a.x_scale[sids[i] / a.top_k] : 1.f;
      else xscale[i] = a.x_scale[pid_t * BT + wt * C::TT + i * C::TILE + frow];
    }
  }
#pragma unroll
  for (int i = 0; i < C::IT; ++i) {
    const int slot = pid_t * BT + wt * C::TT + i * C::TILE + frow;
    const int sid = sids[i];
    const float xs = xscale[i];
    if constexpr (EPI == EPI_SILU) {
      constexpr int HJ = C::JF / 2;
      out_t* orow = static_cast<out_t*>(a.out) + static_cast<int64_t>(slot) * a.ldo;
#pragma unroll
      for (int j = 0; j < HJ; ++j) {
        const AccT ga = AG ? acc_fetch(acc[j][i]) : acc[j][i], ua = AG ? acc_fetch(acc[j + HJ][i]) : acc[j + HJ][i];
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
          const int f = pid_f * (BF / 2) + wf * (C::TF / 2) + j * C::TILE + g * 8 + kgrp * 4;
          out4 o;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float gv = ga[g * 4 + r], uv = ua[g * 4 + r];
            if constexpr (E::SCALED) {
              gv *= xs * w_scale(j, g, r);
              uv *= xs * w_scale(j + HJ, g, r);
            }
            o[r] = static_cast<out_t>(silu(gv) * uv);
          }
          if (f + 3 < a.N) *reinterpret_cast<out4*>(orow + f) = o;
          else
            for (int r = 0; r < 4; ++r)
              if (f + r < a.N) orow[f + r] = o[r];
          if constexpr (kFence) __builtin_amdgcn_sched_barrier(0);
        }
      }
    } else {
      if (sid < a.num_valid) {
        const float rw = routed[i] * xs;
#pragma unroll
        for (int j = 0; j < C::JF; ++j) {
          const AccT ca = AG ? acc_fetch(acc[j][i]) : acc[j][i];
#pragma unroll
          for (int g = 0; g < GROUPS; ++g) {
            const int f = pid_f * BF + wf * C::TF + j * C::TILE + g * 8 + kgrp * 4;
            float v[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              v[r] = ca[g * 4 + r] * rw;
              if constexpr (E::SCALED) v[r] *= w_scale(j, g, r);
            }
            if constexpr (EPI == EPI_DOWN) {
              float* orow = static_cast<float*>(a.out) + static_cast<int64_t>(split) * a.split_stride +
                            static_cast<int64_t>(sid) * a.ldo;
              const f32x4 o = {v[0], v[1], v[2], v[3]};
              if (f + 3 < a.N) *reinterpret_cast<f32x4*>(orow + f) = o;
              else
                for (int r = 0; r < 4; ++r)
                  if (f + r < a.N) orow[f + r] = v[r];
            } else {
              out4 o;
#pragma unroll
              for (int r = 0; r < 4; ++r) o[r] = static_cast<out_t>(v[r]);
              if (a.add_div) {  // top-k combine in the epilogue (the launcher requires N % 4 == 0)
                if (f < a.N) atomic_add4(static_cast<out_t*>(a.out) + static_cast<int64_t>(sid / a.add_div) * a.ldo + f, o);
              } else {
                out_t* orow = static_cast<out_t*>(a.out) + static_cast<int64_t>(sid) * a.ldo;
                if (f + 3 < a.N) *reinterpret_cast<out4*>(orow + f) = o;
                else
                  for (int r = 0; r < 4; ++r)
                    if (f + r < a.N) orow[f + r] = o[r];
              }
            }
            if constexpr (kFence) __builtin_amdgcn_sched_barrier(0);
          }
        }
      }
    }
  }
}

template <typename T, typename C, int EPI>
__global__ __launch_bounds__(C::NT, C::MINB) void moe_gemm_kernel(const GemmArgs a) {
  typedef Elem<T> E;
  typedef typename E::out_t out_t;
  typedef typename E::out4 out4;
  typedef typename std::conditional<C::TILE == 32, f32x16, f32x4>::type acc_t;
  constexpr int BT = C::BT, BF = C::BF, CPR = C::CPR, NT = C::NT, FC = E::FC;
  constexpr int EPC = 16 / static_cast<int>(sizeof(T));     // elements per 16-byte chunk
  constexpr int BK = C::BKB / static_cast<int>(sizeof(T));  // elements of K per tile
  constexpr int KS = CPR / (C::KGROUPS * FC);               // MFMA K-steps per tile
  constexpr int ACC_N = (C::TILE == 32) ? 16 : 4;
  static_assert(CPR % (C::KGROUPS * FC) == 0 && KS >= 1, "tile K must be a multiple of the MFMA K");
  static_assert(EPI != EPI_SILU || C::JF % 2 == 0, "gate and up tiles must pair up inside a wave");

  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  u32x4* lds = reinterpret_cast<u32x4*>(lds_raw);
  // LDS map (16-byte units): X slots first, then W slots
  constexpr int NXS = C::STAGES == 0 ? 2 : C::STAGES, WBASE = NXS * C::XCH;

  // ---- tile coordinates ---------------------------------------------------
  // The grid is sized for the worst-case padded length; only the first
  // (npost/BT)*num_f_tiles workgroups have a tile.  Tiles are dealt to the 8 XCDs
  // (workgroup id mod 8) in contiguous, equally sized ranges of the REAL tile
  // count, then walked in groups of group_t token blocks x all feature tiles so
  // co-resident workgroups share weight tiles in their XCD's L2.
  const int npost = a.npost[0];
  const int nt = min(npost / BT, a.num_t_blocks);
  const int total = nt * a.num_f_tiles;
  if (static_cast<int>(blockIdx.x) >= total) return;
  int lin;
  {
    const int pid = blockIdx.x, xcd = pid & 7, idx = pid >> 3;
    const int per = total >> 3, rem = total & 7;
    lin = xcd * per + (xcd < rem ? xcd : rem) + idx;
  }
  const int in_group = a.group_t * a.num_f_tiles;
  const int group_id = lin / in_group;
  const int first_t = group_id * a.group_t;
  const int gsz = min(nt - first_t, a.group_t);
  const int pid_t = first_t + (lin % in_group) % gsz;
  const int pid_f = (lin % in_group) / gsz;
  const int expert = a.expert_ids[pid_t];
  const int split = blockIdx.y;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wt = wave / C::WF, wf = wave % C::WF;

  const T* X = static_cast<const T*>(a.X);
  const T* W = static_cast<const T*>(a.W) + static_cast<int64_t>(expert) * a.w_expert_stride;
  const int k0 = split * a.k_per_split;
  const int k_tiles = min(a.k_per_split, a.K - k0) / BK;

  // X row of a tile row (gathered through the routing arrays) and W row of a tile row
  auto x_src_row = [&](int rr) -> int64_t {
    if (a.top_k > 0) {
      const int sid = a.sorted[pid_t * BT + rr];
      return sid < a.num_valid ? sid / a.top_k : 0;
    }
    return static_cast<int64_t>(pid_t) * BT + rr;
  };
  auto w_src_row = [&](int rr) -> int {
    if constexpr (EPI == EPI_SILU) {
      const int half = rr / (BF / 2), f = pid_f * (BF / 2) + rr % (BF / 2);
      return half * a.N + (f < a.N ? f : a.N - 1);
    } else {
      const int f = pid_f * BF + rr;
      return f < a.N ? f : a.N - 1;
    }
  };

  // ---- per-lane fragment rows ---------------------------------------------
  const int frow = lane % C::TILE;  // row inside an MFMA tile
  const int kgrp = lane / C::TILE;  // which K group of the MFMA this lane feeds
  // All fragment rows of a lane lie a multiple of 16 rows apart, which leaves the swizzle key unchanged: one
  // offset and one key per operand, the fragments at compile-time distances from them (immediate offsets of
  // the LDS reads).
  static_assert(C::TILE % 16 == 0 && (BF / 2) % 16 == 0 && C::TF % 16 == 0 && C::TT % 16 == 0, "fragment rows 16 apart");
  constexpr int HJ_ = C::JF / 2;  // EPI_SILU: first half of the wave's tiles gate rows, second half the matching up rows
  auto wcol = [](int wf_, int j) constexpr -> int {
    if (EPI == EPI_SILU) return (j < HJ_) ? wf_ * (C::TF / 2) + j * C::TILE : BF / 2 + wf_ * (C::TF / 2) + (j - HJ_) * C::TILE;
    return wf_ * C::TF + j * C::TILE;
  };
  const int xrow0 = wt * C::TT + frow, wrow0 = wcol(wf, 0) + frow;
  const int xoff0 = xrow0 * CPR, xkey0 = swizzle<CPR>(xrow0, 0);
  const int woff0 = WBASE + wrow0 * CPR, wkey0 = swizzle<CPR>(wrow0, 0);
#define FR_XD(i_) ((i_) * C::TILE * CPR)
#define FR_WD(j_) ((wcol(0, (j_)) - wcol(0, 0)) * CPR)

  acc_t acc[C::JF][C::IT];
#pragma unroll
  for (int j = 0; j < C::JF; ++j)
#pragma unroll
    for (int i = 0; i < C::IT; ++i)
#pragma unroll
      for (int r = 0; r < ACC_N; ++r) acc[j][i][r] = 0.f;

  // fragments, double-buffered in registers: [buffer][tile][chunk]
  u32x4 xf[2][C::IT][FC], wfr[2][C::JF][FC];
#define FR_READ_FRAGS(xs_, ws_, ks_, fb_)                                               \
  {                                                                                     \
    const u32x4* xt = lds + (xs_) * C::XCH;                                             \
    const u32x4* wtl = lds + (ws_) * C::WCH;                                            \
    _Pragma("unroll") for (int c = 0; c < FC; ++c) {                                    \
      const int kc = ((ks_) * C::KGROUPS + kgrp) * FC + c;                              \
      const u32x4* xp_ = xt + xoff0 + (kc ^ xkey0);                                     \
      const u32x4* wp_ = wtl + woff0 + (kc ^ wkey0);                                    \
      _Pragma("unroll") for (int i = 0; i < C::IT; ++i) xf[fb_][i][c] = xp_[FR_XD(i)];  \
      _Pragma("unroll") for (int j = 0; j < C::JF; ++j) wfr[fb_][j][c] = wp_[FR_WD(j)]; \
    }                                                                                   \
  }
#define FR_MMA(fb_, j0_, j1_)                                                           \
  {                                                                                     \
    _Pragma("unroll") for (int j = (j0_); j < (j1_); ++j)                               \
      _Pragma("unroll") for (int i = 0; i < C::IT; ++i) {                               \
        if constexpr (C::TILE == 32) acc[j][i] = E::m32(wfr[fb_][j], xf[fb_][i], acc[j][i]); \
        else acc[j][i] = E::m16(wfr[fb_][j], xf[fb_][i], acc[j][i]);                    \
      }                                                                                 \
  }

  if constexpr (C::STAGES == 0) {
    // ---- register-staged double buffering ------------------------------------
    const int chunk = tid % CPR;
    const int row0 = tid / CPR;
    constexpr int ROWS_PER_PASS = NT / CPR;
    constexpr bool X_FULL = (C::XCH % NT == 0), W_FULL = (C::WCH % NT == 0);
    const T* xsrc[C::XL];
    int xdst[C::XL];
#pragma unroll
    for (int i = 0; i < C::XL; ++i) {
      const int r = row0 + i * ROWS_PER_PASS;
      const int rr = r < BT ? r : BT - 1;
      xsrc[i] = X + x_src_row(rr) * a.ldx + k0 + chunk * EPC;
      xdst[i] = rr * CPR + swizzle<CPR>(rr, chunk);
    }
    const T* wsrc[C::WL];
    int wdst[C::WL];
#pragma unroll
    for (int i = 0; i < C::WL; ++i) {
      const int r = row0 + i * ROWS_PER_PASS;
      const int rr = r < BF ? r : BF - 1;
      wsrc[i] = W + static_cast<int64_t>(w_src_row(rr)) * a.ldw + k0 + chunk * EPC;
      wdst[i] = WBASE + rr * CPR + swizzle<CPR>(rr, chunk);
    }
    u32x4 xreg[C::XL], wreg[C::WL];
#define FR_LOAD_TILE(kt)                                                              \
  {                                                                                   \
    _Pragma("unroll") for (int i = 0; i < C::XL; ++i)                                 \
      if (X_FULL || row0 + i * ROWS_PER_PASS < BT)                                    \
        xreg[i] = *reinterpret_cast<const u32x4*>(xsrc[i] + (kt) * BK);               \
    _Pragma("unroll") for (int i = 0; i < C::WL; ++i)                                 \
      if (W_FULL || row0 + i * ROWS_PER_PASS < BF)                                    \
        wreg[i] = *reinterpret_cast<const u32x4*>(wsrc[i] + (kt) * BK);               \
  }
#define FR_STORE_TILE(buf)                                                            \
  {                                                                                   \
    _Pragma("unroll") for (int i = 0; i < C::XL; ++i)                                 \
      if (X_FULL || row0 + i * ROWS_PER_PASS < BT) lds[(buf) * C::XCH + xdst[i]] = xreg[i]; \
    _Pragma("unroll") for (int i = 0; i < C::WL; ++i)                                 \
      if (W_FULL || row0 + i * ROWS_PER_PASS < BF) lds[(buf) * C::WCH + wdst[i]] = wreg[i]; \
  }
#define FR_COMPUTE_TILE(buf)                                                          \
  {                                                                                   \
    _Pragma("unroll") for (int ks = 0; ks < KS; ++ks) {                               \
      FR_READ_FRAGS(buf, buf, ks, 0);                                                 \
      FR_MMA(0, 0, C::JF);                                                            \
    }                                                                                 \
  }
    FR_LOAD_TILE(0);
    FR_STORE_TILE(0);
    __syncthreads();
    for (int kt = 0; kt < k_tiles - 1; ++kt) {
      const int buf = kt & 1;
      FR_LOAD_TILE(kt + 1);
      __builtin_amdgcn_sched_barrier(0);  // keep the prefetch ahead of the MFMA block
      FR_COMPUTE_TILE(buf);
      __builtin_amdgcn_sched_barrier(0);
      FR_STORE_TILE(buf ^ 1);
      __syncthreads();
    }
    FR_COMPUTE_TILE((k_tiles - 1) & 1);
#undef FR_LOAD_TILE
#undef FR_STORE_TILE
#undef FR_COMPUTE_TILE
  } else {
    // ---- direct-to-LDS ring --------------------------------------------------
#if defined(__HIP_DEVICE_COMPILE__)  // buffer resources and LDS-DMA builtins exist in the device pass only
    // A wavefront-wide global_load_lds_dwordx4 fills 64 consecutive 16-byte LDS
    // slots (slot = row*CPR + physical chunk), lane L the L-th of them, so each
    // lane fetches the logical chunk that the swizzle maps to its slot.
    typedef __attribute__((address_space(3))) void* lptr_t;
    constexpr int S = C::STAGES, NW = C::NW, XIW = C::XIW, WIW = C::WIW;
    // The NL loads that refill a slot are issued in PARTS groups of PER, one group per K-step.
    constexpr int PARTS = C::SPREAD < 1 ? 1 : (C::SPREAD > KS ? KS : C::SPREAD);
    // With IW == 2 the loads of wavefront w + NW/2 are issued by wavefront w: the two share a SIMD, so while
    // one sits in the load issue stage the other keeps the MFMA pipe busy instead of both stalling together.
    constexpr int IW = C::IW, NLI = XIW + WIW;  // loads per issuing wavefront per tile
    constexpr int PER = (NLI + PARTS - 1) / PARTS, P0 = PER < NLI ? PER : NLI;
    static_assert(IW >= 1 && NW % IW == 0, "issue width");
    static_assert(KS % 2 == 0, "fragment double buffering needs an even number of K-steps per tile");
    static_assert((S - 1) * NLI <= 63, "vmcnt budget");
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    // Loads are buffer-addressed: a scalar resource (base of X, base of this expert's
    // W), one 32-bit byte offset per lane and the K offset of the tile as the scalar
    // offset.  Per-lane 64-bit addresses cost two VALU adds per load and twice the
    // address traffic to the texture unit, and a wavefront that issues a burst of them
    // sits in the issue stage (no MFMAs) until the unit has taken them all.
    // Offsets are 32-bit: slot-addressed token rows are taken relative to the tile's
    // first row; gathered rows and an expert's weights must span less than 4 GiB
    // (checked by the launcher).
    const int64_t xrow0 = a.top_k > 0 ? 0 : static_cast<int64_t>(pid_t) * BT;
    const __amdgpu_buffer_rsrc_t xrs = uniform_rsrc(X + xrow0 * a.ldx, a.x_span ? a.x_span : 0xFFFFFFFFu);
    const __amdgpu_buffer_rsrc_t wrs = uniform_rsrc(W);
    const bool issuer = wave_u < NW / IW;
    const int wstep = a.w_tiled ? (C::BKB / kTileBytes) * kTilePiece : C::BKB;  // bytes from one K tile of W to the next
    unsigned xsrc[XIW], wsrc[WIW];  // byte offsets, [load][virtual wavefront]
#pragma unroll
    for (int ih = 0; ih < XIW; ++ih) {
      const int i = ih / IW, vw = (wave_u + (ih % IW) * (NW / IW)) % NW;
      const int slot = (i * NW + vw) * kWave + lane;
      // (with an odd load count the last index lies beyond the tile for the wavefronts that issue nothing: clamped)
      const int rr = min(slot / CPR, BT - 1), c = swizzle<CPR>(rr, slot % CPR);
      xsrc[ih] = static_cast<unsigned>(((x_src_row(rr) - xrow0) * a.ldx + k0 + c * EPC) * static_cast<int64_t>(sizeof(T)));
      if (a.x_span && a.sorted[pid_t * BT + rr] >= a.num_valid) xsrc[ih] = kSkipOffset;
    }
#pragma unroll
    for (int ih = 0; ih < WIW; ++ih) {
      const int i = ih / IW, vw = (wave_u + (ih % IW) * (NW / IW)) % NW;
      const int slot = (i * NW + vw) * kWave + lane;
      const int rr = slot / CPR, c = swizzle<CPR>(rr, slot % CPR);
      wsrc[ih] = static_cast<unsigned>(w_byte_offset(a.w_tiled, a.ldw, a.K, w_src_row(rr), (k0 + c * EPC) * static_cast<int64_t>(sizeof(T)), sizeof(T)));
    }
    // load q_ of an issuing wavefront of tile tile_ into ring slot slot_.  Weight-tile loads come
    // first: in the prologue they depend only on the expert id, so they are in flight while the
    // sorted ids that the token-tile addresses need are still being fetched.  The IW virtual
    // wavefronts of one load index are adjacent.
#define FR_ISSUE_ONE(tile_, slot_, q_)                                                                     \
  {                                                                                                        \
    const int vw_ = wave_u + ((q_) % IW) * (NW / IW);                                                      \
    if ((q_) < WIW) {                                                                                  \
      __builtin_amdgcn_raw_ptr_buffer_load_lds(                                                            \
          wrs, (lptr_t)(lds_raw + (WBASE + (slot_) * C::WCH) * 16 + (((q_) / IW) * NW + vw_) * (kWave * 16)), \
          16, wsrc[(q_) < WIW ? (q_) : 0], (tile_) * wstep, 0, FR_W_AUX);                                    \
    } else {                                                                                               \
      __builtin_amdgcn_raw_ptr_buffer_load_lds(                                                            \
          xrs, (lptr_t)(lds_raw + (slot_) * (C::XCH * 16) + ((((q_) - WIW) / IW) * NW + vw_) * (kWave * 16)), \
          16, xsrc[(q_) < WIW ? 0 : (q_) - WIW], (tile_) * C::BKB, 0, 0);                          \
    }                                                                                                      \
  }
#define FR_ISSUE_PART(tile_, slot_, p_)                                                                    \
  {                                                                                                        \
    _Pragma("unroll") for (int q = (p_) * PER; q < ((p_) + 1) * PER && q < NLI; ++q) FR_ISSUE_ONE(tile_, slot_, q); \
  }
    // One K-step: NM MFMAs.  The fragments of the NEXT step are read into the other
    // fragment buffer after the first half, so the second half covers the LDS latency.
    // The refill loads of group p_ (if HAVE_) go out one at a time, evenly spaced
    // between the MFMAs.
    constexpr int NM = C::JF * C::IT, RD_AT = (NM + 1) / 2 - 1;
#define FR_KSTEP(fb_, READ_NEXT, HAVE_, tile_, slot_, p_)                                     \
  {                                                                                           \
    _Pragma("unroll") for (int m = 0; m < NM; ++m) {                                          \
      const int j = m / C::IT, i = m % C::IT;                                                 \
      if constexpr (C::TILE == 32) acc[j][i] = E::m32(wfr[fb_][j], xf[fb_][i], acc[j][i]);    \
      else acc[j][i] = E::m16(wfr[fb_][j], xf[fb_][i], acc[j][i]);                            \
      __builtin_amdgcn_sched_barrier(0);                                                      \
      if (m == RD_AT) {                                                                       \
        READ_NEXT;                                                                            \
        __builtin_amdgcn_sched_barrier(0);                                                    \
      }                                                                                       \
      if (HAVE_) {                                                                            \
        _Pragma("unroll") for (int r = 0; r < PER; ++r)                                       \
          if (m == ((2 * r + 1) * NM) / (2 * PER) && (p_) * PER + r < NLI) {                   \
            FR_ISSUE_ONE(tile_, slot_, (p_) * PER + r);                                       \
            __builtin_amdgcn_sched_barrier(0);                                                \
          }                                                                                   \
      }                                                                                       \
    }                                                                                         \
  }
    // Software pipeline.  Tiles are loaded in order; the barrier that publishes tile
    // kt+1 sits before the LAST K-step of tile kt (whose fragments are already in
    // registers).  After it the slot of tile kt is refilled with tile kt+S: group 0 in
    // that last K-step, groups 1.. in the first K-steps of tile kt+1.  vmcnt counts
    // loads in issue order, so "tile kt+1 landed" leaves exactly the S-2 later tiles
    // outstanding.  The prologue leaves tile S-1 in the same half-issued state.  Inside the
    // steady loop tile kt+S exists, so its body is one basic block with a fixed vmcnt and the
    // compiler counts the outstanding LDS reads exactly; the drain finishes the half-issued
    // refill of the last tile and issues nothing more.  ISS_: this wavefront issues loads.
#define FR_PIPELINE(ISS_) \
  { \
_Pragma("unroll") \
    for (int t = 0; t < S; ++t) { \
      if (t < k_tiles) { \
        if (ISS_) FR_ISSUE_PART(t, t, 0); \
        if (t < S - 1) { \
_Pragma("unroll") \
          for (int p = 1; p < PARTS; ++p) if (ISS_) FR_ISSUE_PART(t, t, p); \
        } \
      } \
    } \
    if (k_tiles >= S) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((S - 2) * NLI + P0) : "memory"); \
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); \
    __builtin_amdgcn_s_barrier(); \
    FR_READ_FRAGS(0, 0, 0, 0); \
    __builtin_amdgcn_s_waitcnt(0xC07F); \
    int sl = 0; \
    int kt = 0; \
    for (; kt < k_tiles - S; ++kt) { \
      const int sn = (sl + 1 == S) ? 0 : sl + 1, sp = (sl == 0) ? S - 1 : sl - 1; \
_Pragma("unroll") \
      for (int ks = 0; ks < KS; ++ks) { \
        if (ks + 1 < KS) { \
          FR_KSTEP(ks & 1, FR_READ_FRAGS(sl, sl, ks + 1, (ks + 1) & 1), (ISS_) && ks + 1 < PARTS, kt - 1 + S, sp, ks + 1); \
        } else { \
          asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"((S - 2) * NLI) : "memory"); \
          __builtin_amdgcn_s_barrier(); \
          FR_KSTEP(ks & 1, FR_READ_FRAGS(sn, sn, 0, 0), ISS_, kt + S, sl, 0); \
        } \
      } \
      sl = sn; \
    } \
    if (k_tiles >= S) { \
      const int sp = (sl == 0) ? S - 1 : sl - 1; \
_Pragma("unroll") \
      for (int p = 1; p < PARTS; ++p) if (ISS_) FR_ISSUE_PART(k_tiles - 1, sp, p); \
    } \
    for (; kt < k_tiles - 1; ++kt) { \
      const int sn = (sl + 1 == S) ? 0 : sl + 1; \
_Pragma("unroll") \
      for (int ks = 0; ks < KS; ++ks) { \
        if (ks + 1 < KS) { \
          FR_KSTEP(ks & 1, FR_READ_FRAGS(sl, sl, ks + 1, (ks + 1) & 1), false, 0, 0, 0); \
        } else { \
          asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory"); \
          __builtin_amdgcn_s_barrier(); \
          FR_KSTEP(ks & 1, FR_READ_FRAGS(sn, sn, 0, 0), false, 0, 0, 0); \
        } \
      } \
      sl = sn; \
    } \
_Pragma("unroll") \
    for (int ks = 0; ks < KS; ++ks) { \
      if (ks + 1 < KS) { \
        FR_KSTEP(ks & 1, FR_READ_FRAGS(sl, sl, ks + 1, (ks + 1) & 1), false, 0, 0, 0); \
      } else { \
        FR_KSTEP(ks & 1, {}, false, 0, 0, 0); \
      } \
    } \
  }
    if (IW == 1 || issuer) FR_PIPELINE(true) else FR_PIPELINE(false)
#undef FR_PIPELINE
#undef FR_KSTEP
#undef FR_ISSUE_PART
#undef FR_ISSUE_ONE
#endif
  }
#undef FR_READ_FRAGS
#undef FR_MMA
#undef FR_XD
#undef FR_WD

  gemm_epilogue<T, C, EPI>(a, acc, pid_t, pid_f, expert, split, wt, wf, frow, kgrp);
}

template <typename T, typename C, int EPI>
int launch_gemm(const GemmArgs& a, int splits, hipStream_t st) {
  if (C::LDS_BYTES > 65536) {  // the dynamic LDS limit is a property of the kernel on ONE device
    constexpr int kMaxDevices = 64;
    static bool attr_set[kMaxDevices] = {};  // a race between threads sets the same attribute twice
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail(FR_E_LAUNCH, "grouped GEMM: device %d (%s)", dev, hipGetErrorString(e));
    if (!attr_set[dev]) {
      e = hipFuncSetAttribute(reinterpret_cast<const void*>(&moe_gemm_kernel<T, C, EPI>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
      if (e != hipSuccess) return fail(FR_E_LAUNCH, "hipFuncSetAttribute(%d B LDS): %s", C::LDS_BYTES, hipGetErrorString(e));
      attr_set[dev] = true;
    }
  }
  if (a.setup_only) return FR_OK;
  if (C::STAGES == 0 && a.w_tiled) return fail(FR_E_SHAPE, "prepared weights need a direct-to-LDS tile");
  if (C::STAGES > 0) {  // the ring loads address rows by 32-bit byte offsets
    const int64_t x_rows = a.top_k > 0 ? a.num_valid / a.top_k : C::BT;
    const int64_t w_rows = EPI == EPI_SILU ? 2 * static_cast<int64_t>(a.N) : a.N;
    const int64_t lim = int64_t(1) << 32, es = sizeof(T);
    if (x_rows * a.ldx * es >= lim || w_rows * a.ldw * es >= lim)
      return fail(FR_E_SHAPE, "token rows (%lld x %lld) or one expert's weights (%lld x %lld) span 4 GiB or more",
                  (long long)x_rows, (long long)a.ldx, (long long)w_rows, (long long)a.ldw);
    if (x_rows * a.ldx * es < (int64_t(1) << 31)) {
      GemmArgs b = a;
      b.x_span = static_cast<unsigned>(x_rows * a.ldx * es);
      const unsigned gx = static_cast<unsigned>(a.num_t_blocks) * static_cast<unsigned>(a.num_f_tiles);
      hipLaunchKernelGGL((moe_gemm_kernel<T, C, EPI>), dim3(gx, splits), dim3(C::NT), C::LDS_BYTES, st, b);
      return check_launch("moe_gemm_kernel");
    }
  }
  const unsigned grid_x = static_cast<unsigned>(a.num_t_blocks) * static_cast<unsigned>(a.num_f_tiles);
  hipLaunchKernelGGL((moe_gemm_kernel<T, C, EPI>), dim3(grid_x, splits), dim3(C::NT), C::LDS_BYTES, st, a);
  return check_launch("moe_gemm_kernel");
}

}  // namespace fr
