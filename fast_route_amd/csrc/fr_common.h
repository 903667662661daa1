// Shared host/device helpers for the gfx950 fused-MoE kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "fast_route_hip.h"

namespace fr {

// ---- error reporting (thread local, never throws) -------------------------
char* error_buffer();
int fail(int code, const char* fmt, ...);
int check_launch(const char* what);

// per-row e4m3 quantisation; rows_dev (optional, device) bounds the rows actually touched
// Bytes of the scratch with which a grouped GEMM of this routing block, operand type, K (elements)
// and output feature count N can split the tiles of its last round along K; 0 if it cannot.
// gateup: N counts the activated features (the weight has 2N rows).
int64_t tail_scratch_bytes(int block, int dtype, int64_t K, int64_t N, bool gateup);

int quant_rows(const void* x, int dtype, int64_t rows, const int32_t* rows_dev, int64_t K, int64_t ldx, void* q_out,
               float* scale_out, hipStream_t st);

// the study knobs set through fr_moe_set_tunables (all zero: the library decides)
const fr_moe_tunables& tunables();

// gating + routing arrays in one launch (small batches); see routing.hip
bool route_align_fits(int64_t M, int E, int topk);
// qx (optional): bf16 token rows [M, qK] quantised per row to e4m3 (qq, qscale) by further workgroups of the launch
int route_align_small(const void* logits, int logits_dtype, int64_t M, int E, int topk, int renorm, int block,
                      float* w, int32_t* ids, int32_t* sorted, int32_t* expert_ids, int32_t* npost,
                      const void* qx, int64_t qK, void* qq, float* qscale, hipStream_t st);

// Gate/up projection of a handful of tokens that does the layer's routing itself (see moe_gemv.h).  Returns
// FR_OK, an error, or 1 when the shape is not one it takes (nothing launched: route and project separately).
int gateup_rows_routed(const void* x, const void* w1, const void* logits, int logits_dtype, int64_t M, int64_t H,
                       int64_t F, int E, int topk, int renorm, int block, int dtype, void* act, float* topk_w,
                       int32_t* topk_ids, int32_t* sorted, int32_t* expert_ids, int32_t* npost, hipStream_t st);

// Looks up (once per device) the device address of the static scratch behind fr_fused_moe_noalloc on the current device.
int prepare_static_scratch();

// Down projection + routed weight + top-k combine (what fr_moe_down_combine / fr_moe_down_combine_fp8 launch).  pair_ids:
// the [M, topk] expert ids, or nullptr; with them a pair whose id lies outside [0, E) - it has no slot in the routing
// arrays - contributes nothing to its token's sum (without them its never-written partial row would be added).
int down_impl(const void* act, const float* act_scale, const void* w2, const float* w2_scale,
              const float* topk_weights, const int32_t* sorted, const int32_t* expert_ids, const int32_t* npost,
              int64_t M, int64_t H, int64_t F, int E, int topk, int block, int split_k, int dtype, int out_dtype,
              float* partial, void* out, float* tail_ws, hipStream_t st, const char* who, int w_tiled,
              const int32_t* pair_ids);

#define FR_REQUIRE(cond, code, ...) \
  do {                              \
    if (!(cond)) return ::fr::fail((code), __VA_ARGS__); \
  } while (0)

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline int64_t round_up(int64_t a, int64_t b) { return ceil_div(a, b) * b; }

// ---- device-side scalar types ---------------------------------------------
typedef __bf16 bf16_t;
typedef _Float16 f16_t;

template <typename T>
__device__ __forceinline__ float to_float(T v) { return static_cast<float>(v); }

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
struct __attribute__((aligned(16))) u32x4_t { unsigned x, y, z, w; };

constexpr int kWave = 64;

// ---- cross-lane exchange ----------------------------------------------------
// partner<S>(v): value held by this lane's partner at butterfly step S.  Steps
// 1 and 2 are DPP quad permutes, 4 and 8 DPP mirrors inside a row of 16 lanes
// (an involution that pairs the two halves, which is all an all-reduce needs),
// 16 and 32 go through the LDS crossbar.  All lanes are written (full row/bank masks,
// every source lane valid), so `old` is a don't-care; passing 0 with bound_ctrl lets
// the compiler fold the move into the consuming VALU instruction.
template <int S>
__device__ __forceinline__ int partner_i32(int v) {
  if constexpr (S == 1) return __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true);   // quad_perm [1,0,3,2]
  else if constexpr (S == 2) return __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
  else if constexpr (S == 4) return __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, true); // row_half_mirror
  else if constexpr (S == 8) return __builtin_amdgcn_update_dpp(0, v, 0x140, 0xF, 0xF, true); // row_mirror
  else return __shfl_xor(v, S, kWave);
}
template <int S>
__device__ __forceinline__ float partner_f32(float v) {
  return __int_as_float(partner_i32<S>(__float_as_int(v)));
}

}  // namespace fr
