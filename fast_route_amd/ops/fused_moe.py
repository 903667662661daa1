"""Routing arrays and the op-level grouped GEMM.

Mirrors fast_route/fast_route/ops/fused_moe.py of the reference: same function
names, argument order and meaning; the work is done by the HIP kernels behind
fr_moe_align / fr_moe_grouped_gemm.
"""
from __future__ import annotations

import torch

from .. import _native as N


def moe_align_block_size(topk_ids: torch.Tensor, block_size: int, num_experts: int):
    """Block-aligned stable sort of the flat expert ids
    (reference: ops/fused_moe.py:133-175).

    Returns (sorted_token_ids int32[n + E*(block-1)], expert_ids int32[n + E],
    num_tokens_post_pad int32[1]); padding slots of sorted_token_ids hold n.
    """
    N.require_cuda(topk_ids)
    assert topk_ids.is_contiguous(), "topk_ids must be contiguous"
    n = topk_ids.numel()
    dev = topk_ids.device
    sorted_ids = torch.empty((n + num_experts * (block_size - 1),), dtype=torch.int32, device=dev)
    expert_ids = torch.empty((n + num_experts,), dtype=torch.int32, device=dev)
    num_tokens_post_pad = torch.empty((1,), dtype=torch.int32, device=dev)
    lib = N.lib()
    ws_bytes = lib.fr_moe_align_workspace_bytes(n, num_experts)
    assert ws_bytes >= 0, "num_experts=%d outside [1, 1024]" % num_experts
    ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=dev)
    N.check(lib.fr_moe_align(topk_ids.data_ptr(), N.dtype_code(topk_ids.dtype), n, num_experts, block_size,
                             sorted_ids.data_ptr(), expert_ids.data_ptr(), num_tokens_post_pad.data_ptr(),
                             ws.data_ptr(), ws_bytes, N.stream_ptr(dev)))
    return sorted_ids, expert_ids, num_tokens_post_pad


def invoke_fused_moe_kernel(A: torch.Tensor, B: torch.Tensor, C: torch.Tensor, topk_weights: torch.Tensor,
                            topk_ids: torch.Tensor, sorted_token_ids: torch.Tensor, expert_ids: torch.Tensor,
                            num_tokens_post_padded: torch.Tensor, mul_routed_weight: bool, top_k: int,
                            config: dict) -> None:
    """C[p] = A[p // top_k] @ B[expert(p)]^T (optionally * topk_weights.flat[p])
    for every routed pair p (reference: ops/fused_moe.py:178-214).  C is
    [M, topk, N]; config['BLOCK_SIZE_M'] must be the block the routing arrays
    were aligned to (the other tile keys are accepted and ignored: tile shapes
    are fixed per block size on this hardware)."""
    N.require_cuda(A, B, C, sorted_token_ids, expert_ids, num_tokens_post_padded)
    assert A.dtype in (torch.float16, torch.bfloat16) and B.dtype == A.dtype and C.dtype == A.dtype
    assert B.is_contiguous() and C.is_contiguous(), "B and C must be contiguous"
    assert A.dim() == 2 and A.stride(1) == 1 and B.dim() == 3 and A.shape[1] == B.shape[2], "Incompatible dimensions"
    assert C.shape[-1] == B.shape[1] and C.numel() == topk_ids.numel() * B.shape[1]
    w_ptr = 0
    if mul_routed_weight:
        assert topk_weights.dtype == torch.float32 and topk_weights.is_contiguous(), \
            "topk_weights must be contiguous float32"
        w_ptr = topk_weights.data_ptr()
    block = int(config["BLOCK_SIZE_M"])
    N.check(N.lib().fr_moe_grouped_gemm(
        A.data_ptr(), A.stride(0), B.data_ptr(), C.data_ptr(), w_ptr, sorted_token_ids.data_ptr(),
        expert_ids.data_ptr(), num_tokens_post_padded.data_ptr(), sorted_token_ids.shape[0], topk_ids.numel(),
        B.shape[1], B.shape[2], B.shape[0], block, int(top_k), int(bool(mul_routed_weight)),
        N.dtype_code(A.dtype), N.stream_ptr(A.device)))
