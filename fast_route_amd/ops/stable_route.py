"""Gating ops.  Mirrors fast_route/fast_route/ops/stable_route.py (fused_route)
and the vLLM topk_softmax call of fast_route/fast_route/layers/vllm_route.py:79-84."""
from __future__ import annotations

import torch

from .. import _native as N


def _out_views(topk_weights: torch.Tensor, topk_ids: torch.Tensor, M: int, topk: int):
    """The reference hands in [M, E] scratch and gets [:, :topk] back
    (ops/stable_route.py:169-170).  Here the results are written densely at the
    start of the caller's storage and returned as contiguous [M, topk] views of
    it, so flat-indexed consumers read the right elements."""
    assert topk_weights.is_contiguous() and topk_ids.is_contiguous(), "output buffers must be contiguous"
    assert topk_weights.numel() >= M * topk and topk_ids.numel() >= M * topk, "output buffers too small"
    return topk_weights.view(-1)[: M * topk].view(M, topk), topk_ids.view(-1)[: M * topk].view(M, topk)


def _gating(logits: torch.Tensor, topk: int, renormalize: bool, w_out: torch.Tensor, i_out: torch.Tensor):
    M, E = logits.shape
    assert logits.stride(1) == 1, "router logits must be contiguous along experts"
    w_k = w_out if w_out.dtype == torch.float32 else torch.empty((M, topk), dtype=torch.float32, device=logits.device)
    i_k = i_out if i_out.dtype == torch.int32 else torch.empty((M, topk), dtype=torch.int32, device=logits.device)
    N.check(N.lib().fr_gating_topk(logits.data_ptr(), N.dtype_code(logits.dtype), M, E, logits.stride(0), topk,
                                   int(bool(renormalize)), w_k.data_ptr(), i_k.data_ptr(), N.stream_ptr(logits.device)))
    if w_k is not w_out:
        w_out.copy_(w_k)
    if i_k is not i_out:
        i_out.copy_(i_k)


def topk_softmax(topk_weights: torch.Tensor, topk_ids: torch.Tensor, token_expert_indices, gating_output: torch.Tensor,
                 renormalize: bool = False):
    """softmax over experts + top-k of router logits [M, E] into caller-allocated
    [M, topk] tensors.  `token_expert_indices` is accepted for signature parity
    and left untouched (the reference deletes it unused, layers/vllm_route.py:85)."""
    N.require_cuda(gating_output, topk_weights, topk_ids)
    M, topk = topk_weights.shape
    assert topk_weights.is_contiguous() and topk_ids.is_contiguous() and topk_ids.shape == (M, topk)
    _gating(gating_output, topk, renormalize, topk_weights, topk_ids)
    return topk_weights, topk_ids


def fused_route(hidden_state: torch.Tensor, gate: torch.Tensor, topk: int, topk_weights: torch.Tensor,
                topk_ids: torch.Tensor, renormalize: bool = True):
    """Routing from the gate matrix: logits = hidden_state[M, K] @ gate[K, E] in
    fp32, stable top-k, softmax over the selected logits
    (reference: ops/stable_route.py:123-178).  Unlike the reference,
    renormalize=False and E < 16 are supported."""
    N.require_cuda(hidden_state, gate, topk_weights, topk_ids)
    M, K = hidden_state.shape
    K2, E = gate.shape
    assert K == K2, "Incompatible dimensions"
    assert E <= 128, f"{E} number of experts should be small enough to reside in shared memory"  # ops/stable_route.py:134
    assert hidden_state.dtype in (torch.float16, torch.bfloat16) and gate.dtype == hidden_state.dtype
    w_view, i_view = _out_views(topk_weights, topk_ids, M, topk)
    dev = hidden_state.device
    # the kernels write fp32 weights and int32 ids; buffers of other types (the reference's own recipe passes
    # fp16 weights and int64 ids, tests/test_route.py:30-38) are filled by a cast of dense temporaries
    w_k = w_view if w_view.dtype == torch.float32 else torch.empty((M, topk), dtype=torch.float32, device=dev)
    i_k = i_view if i_view.dtype == torch.int32 else torch.empty((M, topk), dtype=torch.int32, device=dev)
    if K % 8 == 0 and hidden_state.is_contiguous() and gate.is_contiguous():
        N.check(N.lib().fr_route_gate(hidden_state.data_ptr(), gate.data_ptr(), N.dtype_code(hidden_state.dtype),
                                      M, K, E, topk, int(bool(renormalize)), w_k.data_ptr(), i_k.data_ptr(),
                                      N.stream_ptr(dev)))
    else:
        # strided operands or K % 8 != 0 (shapes the reference's asserts refuse anyway): logits accumulated AND kept in
        # fp32, as the reference's kernel keeps its accumulator (ops/stable_route.py:66-97), then the same stable top-k
        logits = torch.matmul(hidden_state.float(), gate.float())
        _gating(logits, topk, renormalize, w_k, i_k)
    if w_k is not w_view:
        w_view.copy_(w_k)
    if i_k is not i_view:
        i_view.copy_(i_k)
    return w_view, i_view
