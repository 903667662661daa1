"""CPU oracle for the fused MoE layer.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package may import this module: it exists so that the
tests, the smoke check and the bench's CPU-baseline leg have an independent
statement of what the HIP kernels must compute.
"""
from .moe_oracle import (  # noqa: F401
    stable_sort_rows,
    gating_topk,
    gating_topk_softmax_first,
    route_from_gate,
    moe_align_block_size,
    silu_and_mul,
    grouped_gemm,
    moe_experts,
    fused_moe,
    e4m3fn_decode_table,
    e4m3fn_encode,
    quant_e4m3_rows,
    quantize_weights_fp8,
    fused_moe_fp8,
    tile_weights,
    make_inputs,
    zipf_logits,
)
