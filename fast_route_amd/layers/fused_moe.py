"""The fused MoE layer in its router-logits form and the experts-only form."""
from __future__ import annotations

import torch

from .. import _native as N


def _check_layer(hidden_states, w1, w2):
    # same constraints, same messages as the reference (layers/stable_route.py:32-36)
    assert hidden_states.shape[1] == w1.shape[2], "Incompatible dimensions"
    assert hidden_states.is_contiguous(), "Hidden_states must be contiguous"
    assert w1.is_contiguous(), "Expert weights1 must be contiguous"
    assert w2.is_contiguous(), "Expert weights2 must be contiguous"
    assert hidden_states.dtype in [torch.float16, torch.bfloat16]
    assert w1.dtype == hidden_states.dtype and w2.dtype == hidden_states.dtype
    assert w2.shape[0] == w1.shape[0] and w2.shape[1] == w1.shape[2] and 2 * w2.shape[2] == w1.shape[1], \
        "w1 must be [E, 2F, H] and w2 [E, H, F]"
    N.require_cuda(hidden_states, w1, w2)


def plan(M: int, H: int, F: int, E: int, topk: int, dtype, code: int | None = None) -> N.FrMoePlan:
    p = N.FrMoePlan()
    N.check(N.lib().fr_moe_get_plan(M, H, F, E, topk, N.dtype_code(dtype) if code is None else code, p))
    return p


def workspace(M: int, H: int, F: int, E: int, topk: int, dtype, device) -> torch.Tensor:
    """Scratch the layer needs for these shapes (256-byte aligned by torch)."""
    return torch.empty((max(plan(M, H, F, E, topk, dtype).workspace_bytes, 256),), dtype=torch.uint8, device=device)


def prepare_weights(w1: torch.Tensor, w2: torch.Tensor, which: str = "w2"):
    """One-off re-layout of expert weights, from the checkpoint layout the reference takes (w1 [E, 2F, H] with the
    gate rows first, w2 [E, H, F]; layers/stable_route.py:32-36) into tiles of 64 rows x 128 bytes of K, each 8 KB
    of consecutive memory (fr_moe_prepare_weights).  `which`: "w2" (default: the down projection is 2-7 % faster from
    512 tokens up and never slower), "w1" or "both" (the gate/up GEMM gains under 1 % from 512 tokens up and loses
    2-6 % below).  Returns (w1', w2', flags): new tensors of the same shape and dtype for the matrices named - the
    originals of those may be freed -, the others as they came, and the value to pass as `weights_prepared`."""
    N.require_cuda(w1, w2)
    assert which in ("w1", "w2", "both")
    assert w1.is_contiguous() and w2.is_contiguous(), "Expert weights must be contiguous"
    assert w1.dtype in (torch.float16, torch.bfloat16) and w2.dtype == w1.dtype
    E, F2, H = w1.shape
    assert w2.shape == (E, H, F2 // 2), "w1 must be [E, 2F, H] and w2 [E, H, F]"
    assert (F2 // 2) % 64 == 0 and H % 64 == 0, "prepared layout: F and H must be multiples of 64"

    def tile(w):
        t = torch.empty_like(w)
        N.check(N.lib().fr_moe_prepare_weights(w.data_ptr(), N.dtype_code(w.dtype), E, w.shape[1], w.shape[2],
                                               t.data_ptr(), N.stream_ptr(w.device)))
        return t

    flags = 0
    if which in ("w1", "both"):
        w1, flags = tile(w1), flags | N.FR_W1_TILED
    if which in ("w2", "both"):
        w2, flags = tile(w2), flags | N.FR_W2_TILED
    return w1, w2, flags


def _layout_flags(weights_prepared) -> int:
    """weights_prepared: False / 0, True (both matrices), or the flags prepare_weights returned."""
    if weights_prepared is True:
        return N.FR_W_TILED
    flags = int(weights_prepared or 0)
    assert flags & ~N.FR_W_TILED == 0, "weights_prepared: pass what prepare_weights returned"
    return flags


def fused_experts(hidden_states: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, topk_weights: torch.Tensor,
                  topk_ids: torch.Tensor, inplace: bool = False, workspace_buf: torch.Tensor | None = None,
                  weights_prepared=False):
    """out[m] = sum_j topk_weights[m, j] * MLP_{topk_ids[m, j]}(hidden_states[m])
    (the fused_moe(hidden, w1, w2, topk_weights, topk_ids, inplace) entry of
    benchmarks/swizzle_moe/v0_moe_fused.py:219-293)."""
    _check_layer(hidden_states, w1, w2)
    M, H = hidden_states.shape
    E, F2, _ = w1.shape
    topk = topk_ids.shape[1]
    assert topk_weights.shape == topk_ids.shape == (M, topk), "topk shape mismatch"
    tw = topk_weights if (topk_weights.dtype == torch.float32 and topk_weights.is_contiguous()) \
        else topk_weights.float().contiguous()
    ti = topk_ids if (topk_ids.dtype == torch.int32 and topk_ids.is_contiguous()) else topk_ids.int().contiguous()
    ws = workspace_buf if workspace_buf is not None else workspace(M, H, F2 // 2, E, topk, hidden_states.dtype,
                                                                  hidden_states.device)
    out = hidden_states if inplace else torch.empty_like(hidden_states)
    N.check(N.lib().fr_fused_experts(hidden_states.data_ptr(), w1.data_ptr(), w2.data_ptr(), tw.data_ptr(),
                                     ti.data_ptr(), M, H, F2 // 2, E, topk,
                                     N.dtype_code(hidden_states.dtype) | _layout_flags(weights_prepared),
                                     out.data_ptr(), ws.data_ptr(), ws.numel(), N.stream_ptr(hidden_states.device)))
    return out


def fused_moe(hidden_states: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, gating_output: torch.Tensor,
              topk: int, renormalize: bool = True, inplace: bool = False,
              workspace_buf: torch.Tensor | None = None, weights_prepared=False):
    """Whole MoE layer from router logits [M, E]: gating, routing, gate/up GEMM
    with SiLU*mul, down GEMM with routed weight and top-k combine
    (reference layer: layers/stable_route.py:10-102, with the routing input in
    the vLLM 0.4.0 `gating_output` form).  weights_prepared: the flags prepare_weights() returned (True: both matrices prepared)."""
    _check_layer(hidden_states, w1, w2)
    M, H = hidden_states.shape
    E, F2, _ = w1.shape
    assert gating_output.shape == (M, E), "Number of tokens mismatch"
    assert gating_output.is_contiguous(), "gating_output must be contiguous"
    N.require_cuda(gating_output)
    ws = workspace_buf if workspace_buf is not None else workspace(M, H, F2 // 2, E, topk, hidden_states.dtype,
                                                                  hidden_states.device)
    out = hidden_states if inplace else torch.empty_like(hidden_states)
    N.check(N.lib().fr_fused_moe(hidden_states.data_ptr(), w1.data_ptr(), w2.data_ptr(), gating_output.data_ptr(),
                                 N.dtype_code(gating_output.dtype), M, H, F2 // 2, E, topk, int(bool(renormalize)),
                                 N.dtype_code(hidden_states.dtype) | _layout_flags(weights_prepared),
                                 out.data_ptr(), ws.data_ptr(), ws.numel(), N.stream_ptr(hidden_states.device)))
    return out
