/* fast_route_hip.h -- C ABI of the MI355X (gfx950) fused-MoE library.
 *
 * Every entry point is what a binding of the reference's hot path calls; the
 * comment on each names the reference interface it replaces
 * (hgl71964/fast-route, paths relative to the reference root).
 *
 * Conventions
 *   - all pointers except `stream` are DEVICE addresses owned by the caller;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *   - every call only enqueues work on `stream`: no allocation, no host
 *     synchronisation, no device-to-host copy.  Under graph capture that holds once the
 *     kernels are set up on the device: the first call of a tile configuration raises its
 *     dynamic-LDS limit and queries its occupancy (set-up calls, not stream work), so a
 *     caller whose first call would be captured calls fr_moe_prepare once per device and
 *     dtype beforehand, or makes one eager call of the same shape;
 *   - return value 0 on success, a negative FR_E_* code otherwise;
 *     fr_last_error_string() gives the thread-local message of the last failure;
 *   - tensors are dense row-major unless a stride argument says otherwise.
 */
#ifndef FAST_ROUTE_HIP_H
#define FAST_ROUTE_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FR_OK 0
#define FR_E_NULL (-1)        /* a required pointer is NULL                     */
#define FR_E_SHAPE (-2)       /* a dimension is out of the supported range      */
#define FR_E_DTYPE (-3)       /* dtype enum not supported by this entry point   */
#define FR_E_ALIGN (-4)       /* pointer / stride not aligned as required       */
#define FR_E_WORKSPACE (-5)   /* workspace too small                            */
#define FR_E_LAUNCH (-6)      /* the HIP runtime rejected a launch              */
#define FR_E_NO_DEVICE (-7)   /* no gfx950 device / code object not loadable    */

typedef enum fr_dtype {
  FR_F16 = 0,
  FR_BF16 = 1,
  FR_F32 = 2,
  FR_FP8_E4M3 = 3, /* OCP e4m3fn */
  FR_I32 = 4,
  FR_I64 = 5
} fr_dtype;

/* Library version (major*10000 + minor*100 + patch). */
int fr_version(void);

/* Message of the last failing call on this thread ("" if none). */
const char* fr_last_error_string(void);

/* ---- gating --------------------------------------------------------------
 * Top-k gating of router logits[M, E] (row stride `ld` elements): stable
 * descending order of the fp32 logits (ties -> lower expert index), softmax
 * over the selected logits (renormalize != 0) or the selected entries of the
 * full softmax (renormalize == 0).  Writes weights_out[M, topk] fp32 and
 * ids_out[M, topk] int32, both contiguous.
 * Replaces: route_kernel's sort+softmax, fast_route/fast_route/ops/stable_route.py:97-121,
 * and vLLM topk_softmax + renormalise, fast_route/fast_route/layers/vllm_route.py:79-87.
 * Limits: 1 <= topk <= E <= 256; logits_dtype in {FR_F16, FR_BF16, FR_F32}. */
int fr_gating_topk(const void* logits, int logits_dtype, int64_t M, int64_t E, int64_t ld,
                   int topk, int renormalize, float* weights_out, int32_t* ids_out, void* stream);

/* Gate-matrix form: logits = hidden[M, H] @ gate[H, E] accumulated in fp32,
 * then fr_gating_topk, in one kernel (no [M, E] round trip).
 * Replaces: fused_route, fast_route/fast_route/ops/stable_route.py:123-178.
 * Limits: E <= 128 (the reference's bound, ops/stable_route.py:134), H % 8 == 0;
 * dtype in {FR_F16, FR_BF16}. */
int fr_route_gate(const void* hidden, const void* gate, int dtype, int64_t M, int64_t H, int64_t E,
                  int topk, int renormalize, float* weights_out, int32_t* ids_out, void* stream);

/* ---- routing arrays ------------------------------------------------------
 * Block-aligned stable counting sort of the n = M*topk flat expert ids.
 *   sorted_token_ids : int32[n + E*(block-1)], fully written; padding = n
 *   expert_ids       : int32[n + E], first num_tokens_post_pad/block entries written
 *   num_tokens_post_pad : int32[1]
 * Replaces: moe_align_block_size, fast_route/fast_route/ops/fused_moe.py:133-175
 * (vLLM ops.moe_align_block_size at :173).
 * ids_dtype in {FR_I32, FR_I64}; 1 <= E <= 1024; block >= 1; ids must lie in [0, E).
 * `workspace` must hold fr_moe_align_workspace_bytes(n, E) bytes (may be 0). */
int64_t fr_moe_align_workspace_bytes(int64_t n, int E);
int fr_moe_align(const void* topk_ids, int ids_dtype, int64_t n, int E, int block,
                 int32_t* sorted_token_ids, int32_t* expert_ids, int32_t* num_tokens_post_pad,
                 void* workspace, int64_t workspace_bytes, void* stream);

/* ---- grouped GEMM, op level ----------------------------------------------
 * For every sorted slot s < num_tokens_post_pad with p = sorted_token_ids[s] < num_valid:
 *   C[p, :] = A[p / top_k, :] @ B[expert_ids[s / block], :, :]^T   (fp32 accumulate)
 * optionally times topk_weights[p], rounded to `dtype`.
 *   A [*, K] (row stride lda), B [E, N, K] dense, C [num_valid, N] dense.
 * Replaces: invoke_fused_moe_kernel / fused_moe_kernel,
 * fast_route/fast_route/ops/fused_moe.py:178-214 and :10-130.
 * Limits: K % 64 == 0 (K % 128 == 0 for block 16), N % 4 == 0, block in {16, 32, 64, 128, 160, 256};
 * dtype in {FR_F16, FR_BF16}. */
int fr_moe_grouped_gemm(const void* A, int64_t lda, const void* B, void* C,
                        const float* topk_weights, const int32_t* sorted_token_ids,
                        const int32_t* expert_ids, const int32_t* num_tokens_post_pad,
                        int64_t sorted_len, int64_t num_valid, int64_t N, int64_t K, int E,
                        int block, int top_k, int mul_routed_weight, int dtype, void* stream);

/* ---- prepared weight layout (optional) -------------------------------------
 * The reference takes w1 [E, 2F, H] and w2 [E, H, F] row-major
 * (fast_route/fast_route/layers/stable_route.py:32-36; gate rows first, up rows second,
 * fast_route/benchmarks/fused_route/activation.py:27-30) and so does every entry point here.
 * A weight tile of a GEMM is then as many 128-byte pieces as it has rows, one row length
 * apart.  fr_moe_prepare_weights re-lays a weight matrix w[E, rows, K] out once, into a
 * buffer `out` of the same size (the caller may free `w` afterwards; not in place):
 * inside an expert, groups of 64 consecutive rows; inside a group, K tiles of 128 bytes per
 * row; inside a K tile the group's 64 rows one after the other - each (row group, K tile)
 * is 8 KB of consecutive memory and a group's whole K range one run.
 * rows % 64 == 0, K * element size % 128 == 0; dtype in {FR_F16, FR_BF16, FR_FP8_E4M3}.
 * Entry points that take a `dtype` argument accept layout flags OR-ed into it: FR_W1_TILED - the
 * gate/up weights (w1; B of fr_moe_grouped_gemm) are in this layout -, FR_W2_TILED - the down
 * weights (w2) are -, FR_W_TILED = both.  fr_moe_gateup_silu looks at FR_W1_TILED,
 * fr_moe_down_combine at FR_W2_TILED, fr_moe_grouped_gemm at either, fr_fused_experts,
 * fr_fused_moe and fr_fused_moe_noalloc at both; the fp8 entry points take the flags in
 * their `out_dtype` (fr_moe_down_combine_fp8: FR_W2_TILED) and `x_dtype` (fr_fused_moe_fp8:
 * FR_W2_TILED) arguments, for codes tiled with dtype FR_FP8_E4M3 (128 elements per K tile).
 * Results are bit-identical to the row-major call when the same kernels run; with FR_W1_TILED
 * (FR_W2_TILED) batches of up to 4 tokens (4 pairs), whose row-major form streams whole weight
 * rows without tiles, take the 16-row tile kernels instead.
 * Measured on the Mixtral shape: the down projection is 2-7 % faster from 512 tokens up and
 * never slower; the gate/up GEMM gains under 1 % from 512 tokens up and loses 2-6 % below
 * (its decode tiles stream 512-byte pieces of the 8 KB weight rows) - prepare w2 always,
 * w1 only for a prefill-only deployment. */
#define FR_W1_TILED 0x100
#define FR_W2_TILED 0x200
#define FR_W_TILED 0x300
int fr_moe_prepare_weights(const void* w, int dtype, int64_t E, int64_t rows, int64_t K, void* out,
                           void* stream);

/* ---- fused expert MLPs ---------------------------------------------------
 * Tile plan chosen from the problem size: the routing block the fused kernels
 * want (pass it to fr_moe_align) and the split-K factor of the down GEMM. */
typedef struct fr_moe_plan {
  int32_t block;      /* routing block = token rows per GEMM tile            */
  int32_t split_k;    /* K splits of the down projection                     */
  int64_t sorted_len; /* n + E*(block-1): length of sorted_token_ids         */
  int64_t workspace_bytes; /* bytes fr_fused_moe / fr_fused_experts need     */
  int64_t tail_bytes; /* bytes of the optional `tail_ws` scratch of the two  */
                      /* GEMM entry points below (0: the plan has no use for */
                      /* it); already counted in workspace_bytes             */
} fr_moe_plan;
int fr_moe_get_plan(int64_t M, int64_t H, int64_t F, int E, int topk, int dtype, fr_moe_plan* plan);

/* Per-device set-up of every grouped-GEMM kernel of `dtype` (FR_F16, FR_BF16, FR_FP8_E4M3) on the
 * CURRENT device: raises the kernels' dynamic-LDS limits and caches the persistent kernels'
 * occupancy, and looks up the address of fr_fused_moe_noalloc's scratch.  The first call of each tile configuration does the same work lazily; a caller whose
 * first call would be under graph capture (set-up calls are not stream work) calls this once per
 * device and dtype beforehand.  Launches nothing.  No counterpart in the reference (Triton compiles
 * and configures its kernels on first use, fast_route/fast_route/layers/stable_route.py:67). */
int fr_moe_prepare(int dtype);

/* Study knobs of the tile plan, process-wide (set them from one thread while no call is in
 * flight; they are read when a call is made, not when its kernels run).  0 in a field leaves
 * that choice to the library.
 *   block      routing block = token rows per GEMM tile: 16, 32, 64, 128, 160 or 256
 *   split_k    K slices of the down projection, 1..64 (1 also switches the last-round split on
 *              where the tile supports it, as the plan itself would)
 *   group_m    token blocks walked together over the feature tiles (L2 sharing of weight tiles),
 *              1..64
 *   no_tail_split  1: never split the last, partly filled round of tiles along K
 *   epilogue_combine  1: with two experts per token and one K slice, the down GEMM adds each pair's
 *              weighted row into a zero-filled `out` with packed atomic adds in its epilogue (the sum of
 *              two rows does not depend on their order) instead of writing the pairs' rows for the
 *              combine kernel.  Off by default: measured slower - 16.7 M four-byte atomics at Mixtral
 *              shape and 4096 tokens cost the down stage 1015 us against 900 us (3650 against 3200 us at
 *              16384 tokens, 149 against 146 us at 16 tokens)
 *   no_quad    1: 256-row tiles of 2-byte operands never take the one-wavefront-per-SIMD kernel
 *              (four wavefronts of 128 x 128 outputs, the default where K has 16 K tiles or more) but the
 *              eight-wavefront one; same results bit for bit, for comparisons and tests
 * fr_moe_get_plan, fr_fused_moe, fr_fused_experts, fr_fused_moe_fp8 and the staged GEMM entry
 * points all see them.  fr_moe_set_tunables(NULL) restores the defaults.
 * The staged entry points read the knobs when they are called, not when the plan was made: a
 * caller that sized `partial` / `tail_ws` from a plan, changed the knobs and then calls the staged
 * GEMMs runs the old sizes with the new group_m / no_tail_split (never out of bounds: `block` and
 * `split_k` are the call's own arguments, and the slices actually run are min(split_k, what K
 * allows at 8 K tiles per slice)).  A study should take a new plan after every change and record
 * fr_moe_get_tunables() next to its timings, as bench.py does.
 * Replaces: the per-GEMM config dictionaries edited by hand in the reference's tile study
 * (block_m / group_m / split_k; block_n and block_k are fixed per block size on this hardware),
 * fast_route/benchmarks/swizzle_moe/v1_moe_fused.py:311-344. */
typedef struct fr_moe_tunables {
  int32_t block;
  int32_t split_k;
  int32_t group_m;
  int32_t no_tail_split;
  int32_t epilogue_combine;
  int32_t no_quad;
} fr_moe_tunables;
int fr_moe_set_tunables(const fr_moe_tunables* t);
int fr_moe_get_tunables(fr_moe_tunables* t);

/* act[s, :] = silu(x[t] @ W1[e, :F]^T) * (x[t] @ W1[e, F:]^T) for every sorted
 * slot s < num_tokens_post_pad that holds a pair (t = sorted_token_ids[s] / topk),
 * written at row s of act[sorted_len, F].  Rows of padding slots are unspecified
 * (the tile kernels fill them from token 0, the decode form for up to 4 tokens
 * leaves them untouched); nothing downstream reads them.
 * Replaces: grouped GEMM 1 + silu_and_mul,
 * fast_route/fast_route/layers/stable_route.py:85-90.
 * `tail_ws`: NULL, or 256-byte aligned device scratch of plan.tail_bytes.  With
 * it the 256-row tiles that only partly fill the last round of workgroups are
 * split along K over the idle ones and summed in a fixed order by a second
 * launch; without it every tile is computed by one workgroup.  Results of the
 * two modes differ by fp32 summation order only. */
int fr_moe_gateup_silu(const void* x, const void* w1, const int32_t* sorted_token_ids,
                       const int32_t* expert_ids, const int32_t* num_tokens_post_pad,
                       int64_t M, int64_t H, int64_t F, int E, int topk, int block, int dtype,
                       void* act, void* tail_ws, void* stream);

/* out[m, :] = sum_j topk_weights[m, j] * (act[slot(m, j)] @ W2[e]^T), the
 * down projection with the routed weight applied in the GEMM epilogue and the
 * top-k combine.  `partial` is scratch of split_k * M*topk * H floats (with
 * split_k == 1 only its first half is used: the pairs' rows are kept in `dtype`).
 * Replaces: grouped GEMM 2 + torch.sum,
 * fast_route/fast_route/layers/stable_route.py:92-102.
 * `tail_ws`: as for fr_moe_gateup_silu (used when split_k == 1). */
int fr_moe_down_combine(const void* act, const void* w2, const float* topk_weights,
                        const int32_t* sorted_token_ids, const int32_t* expert_ids,
                        const int32_t* num_tokens_post_pad, int64_t M, int64_t H, int64_t F, int E,
                        int topk, int block, int split_k, int dtype, float* partial, void* out,
                        void* tail_ws, void* stream);

/* Experts only: routing arrays + both GEMMs + combine, from given top-k
 * weights/ids (the fused_moe(hidden, w1, w2, topk_weights, topk_ids) shape of
 * benchmarks/swizzle_moe/v0_moe_fused.py:219-293). */
int fr_fused_experts(const void* x, const void* w1, const void* w2, const float* topk_weights,
                     const int32_t* topk_ids, int64_t M, int64_t H, int64_t F, int E, int topk,
                     int dtype, void* out, void* workspace, int64_t workspace_bytes, void* stream);

/* Whole layer from router logits[M, E] (dense, `logits_dtype`):
 * gating -> routing arrays -> gate/up GEMM + SiLU*mul -> down GEMM + combine.
 * Replaces: fused_moe, fast_route/fast_route/layers/stable_route.py:10-102 and
 * fast_route/fast_route/layers/vllm_route.py:17-120.  `out` may alias `x`
 * (the reference's inplace=True). */
int fr_fused_moe(const void* x, const void* w1, const void* w2, const void* logits,
                 int logits_dtype, int64_t M, int64_t H, int64_t F, int E, int topk,
                 int renormalize, int dtype, void* out, void* workspace, int64_t workspace_bytes,
                 void* stream);

/* fr_fused_moe without a workspace argument and without any allocation: the layer's
 * scratch (top-k arrays, routing arrays, activated intermediate, partial rows) lives in a
 * 64 MiB device array inside this library, which every GPU the library runs on holds
 * until the process ends.  No counterpart in the reference; it is for callers that
 * cannot allocate: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  Sizes whose fr_moe_get_plan().workspace_bytes exceed 64 MiB are
 * rejected with FR_E_WORKSPACE (Mixtral-8x7B shape: up to 207 tokens).  The array's
 * device address is looked up by fr_moe_prepare, or else on the first call on each device
 * (with that device current): before capturing a call, call fr_moe_prepare or make one
 * eager call on that device.  Nothing in the array has to start at zero.  All calls on one GPU share the
 * array: calls that overlap in time on one GPU (two streams, two threads) race. */
int fr_fused_moe_noalloc(const void* x, const void* w1, const void* w2, const void* logits,
                         int logits_dtype, int64_t M, int64_t H, int64_t F, int E, int topk,
                         int renormalize, int dtype, void* out, void* stream);

/* ---- fp8 (OCP e4m3fn) path -------------------------------------------------
 * No counterpart in the reference (its only fp8 mentions are commented autotune
 * rows, fast_route/fast_route/ops/stable_route.py:20-28); defined by the fp8
 * workload of this build: weights quantised per (expert, output channel),
 * activations per token, fp32 scales, fp32 accumulation on the f8f6f4 MFMAs.
 *
 * Per-row dynamic quantisation: scale[r] = max|x[r,:]|/448 (1 for a zero row),
 * q[r,:] = e4m3(x[r,:]/scale[r]) with round-to-nearest-even.  x is f16/bf16
 * [rows, K] with row stride ldx; q is uint8 [rows, K] dense.  K % 16 == 0.
 * Use it on w1 viewed as [E*2F, H] and w2 as [E*H, F] to prepare weights. */
int fr_quant_e4m3_rows(const void* x, int dtype, int64_t rows, int64_t K, int64_t ldx, void* q_out,
                       float* scale_out, void* stream);

/* fp8 forms of fr_moe_gateup_silu / fr_moe_down_combine: operands are e4m3
 * codes with one fp32 scale per row (x_scale[M], w1_scale[E, 2F], act_scale
 * [sorted_len], w2_scale[E, H]); act is written / read in bf16 resp. e4m3;
 * H and F must be multiples of 256.  `tail_ws` as for fr_moe_down_combine.
 * block 160 (a tile without a plain form for fp8) needs K >= 640 per K slice and E <= 1022; fr_moe_get_plan
 * never hands out a block these calls refuse. */
int fr_moe_gateup_silu_fp8(const void* xq, const float* x_scale, const void* w1q, const float* w1_scale,
                           const int32_t* sorted_token_ids, const int32_t* expert_ids,
                           const int32_t* num_tokens_post_pad, int64_t M, int64_t H, int64_t F, int E,
                           int topk, int block, void* act_bf16, void* stream);
int fr_moe_down_combine_fp8(const void* actq, const float* act_scale, const void* w2q, const float* w2_scale,
                            const float* topk_weights, const int32_t* sorted_token_ids,
                            const int32_t* expert_ids, const int32_t* num_tokens_post_pad, int64_t M,
                            int64_t H, int64_t F, int E, int topk, int block, int split_k, int out_dtype,
                            float* partial, void* out, void* tail_ws, void* stream);

/* Whole fp8 layer from bf16 activations and router logits: gating, routing,
 * per-token quantisation of x, fp8 gate/up GEMM + SiLU*mul (bf16 act), per-row
 * quantisation of act, fp8 down GEMM + routed weight + combine.  Workspace size:
 * fr_moe_get_plan(..., FR_FP8_E4M3, &plan).workspace_bytes. */
int fr_fused_moe_fp8(const void* x, int x_dtype, const void* w1q, const float* w1_scale, const void* w2q,
                     const float* w2_scale, const void* logits, int logits_dtype, int64_t M, int64_t H,
                     int64_t F, int E, int topk, int renormalize, void* out, void* workspace,
                     int64_t workspace_bytes, void* stream);

/* ---- measurement aid -------------------------------------------------------
 * A pure stream of bf16 MFMAs (no loads, no LDS) on every CU: `iters` rounds over 256 accumulator
 * registers per lane and SIMD, `shape` 32 = v_mfma_f32_32x32x16_bf16, 16 = v_mfma_f32_16x16x32_bf16,
 * with one or two wavefronts per SIMD.  operands: 65536 bytes of operand bits (random bf16 draw the
 * power real data draw; zeros do not); sink: 512 floats per CU; counts[2] receives workgroup 0's
 * elapsed shader-clock cycles and ticks of the 100 MHz counter.  The part lowers its clock under MFMA
 * load to hold a power budget; this is the ceiling the roofline fractions of the grouped GEMMs are
 * read against.  No counterpart in the reference. */
int fr_probe_mfma_stream(int shape, int waves_per_simd, int iters, const void* operands, float* sink,
                         int64_t* counts, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FAST_ROUTE_HIP_H */
