"""fp8 (OCP e4m3fn) form of the fused MoE layer.

No counterpart in the reference; it follows the fp8 workload this build is
specified with: weights quantised once per (expert, output channel), bf16
activations quantised per token on the fly, fp32 scales, fp32 accumulation.
"""
from __future__ import annotations

import torch

from .. import _native as N
from .fused_moe import plan


def quantize_rows_e4m3(x: torch.Tensor):
    """Per-row dynamic quantisation of a [rows, K] f16/bf16 tensor.
    Returns (codes uint8 [rows, K], scales float32 [rows]); scale = max|row|/448."""
    N.require_cuda(x)
    assert x.dim() == 2 and x.stride(1) == 1 and x.dtype in (torch.float16, torch.bfloat16)
    rows, K = x.shape
    q = torch.empty((rows, K), dtype=torch.uint8, device=x.device)
    s = torch.empty((rows,), dtype=torch.float32, device=x.device)
    N.check(N.lib().fr_quant_e4m3_rows(x.data_ptr(), N.dtype_code(x.dtype), rows, K, x.stride(0), q.data_ptr(),
                                       s.data_ptr(), N.stream_ptr(x.device)))
    return q, s


def prepare_weights_fp8(w1: torch.Tensor, w2: torch.Tensor):
    """One-off weight preparation: w1 [E, 2F, H] and w2 [E, H, F] (f16/bf16) to
    e4m3 codes of the same shapes plus scales w1_scale [E, 2F], w2_scale [E, H]."""
    assert w1.is_contiguous() and w2.is_contiguous()
    E, F2, H = w1.shape
    w1q, w1s = quantize_rows_e4m3(w1.view(E * F2, H))
    w2q, w2s = quantize_rows_e4m3(w2.view(E * w2.shape[1], w2.shape[2]))
    return w1q.view(E, F2, H), w1s.view(E, F2), w2q.view(w2.shape), w2s.view(E, w2.shape[1])


def fused_moe_fp8(hidden_states: torch.Tensor, w1q: torch.Tensor, w1_scale: torch.Tensor, w2q: torch.Tensor,
                  w2_scale: torch.Tensor, gating_output: torch.Tensor, topk: int, renormalize: bool = True,
                  inplace: bool = False, workspace_buf: torch.Tensor | None = None):
    """Whole layer with fp8 weights: bf16 hidden_states [M, H], e4m3 w1q [E, 2F, H] /
    w2q [E, H, F] with per-row float32 scales, router logits [M, E]."""
    N.require_cuda(hidden_states, w1q, w2q, w1_scale, w2_scale, gating_output)
    assert hidden_states.dtype == torch.bfloat16 and hidden_states.is_contiguous(), "hidden_states must be contiguous bf16"
    assert w1q.dtype == torch.uint8 and w2q.dtype == torch.uint8 and w1q.is_contiguous() and w2q.is_contiguous()
    assert w1_scale.dtype == torch.float32 and w2_scale.dtype == torch.float32
    assert w1_scale.is_contiguous() and w2_scale.is_contiguous()
    M, H = hidden_states.shape
    E, F2, H2 = w1q.shape
    assert H2 == H, "Incompatible dimensions"
    assert w2q.shape == (E, H, F2 // 2) and w1_scale.shape == (E, F2) and w2_scale.shape == (E, H)
    assert gating_output.shape == (M, E) and gating_output.is_contiguous(), "Number of tokens mismatch"
    p = plan(M, H, F2 // 2, E, topk, None, code=N.FR_FP8_E4M3)
    ws = workspace_buf if workspace_buf is not None else torch.empty((max(p.workspace_bytes, 256),), dtype=torch.uint8,
                                                                     device=hidden_states.device)
    out = hidden_states if inplace else torch.empty_like(hidden_states)
    N.check(N.lib().fr_fused_moe_fp8(hidden_states.data_ptr(), N.FR_BF16, w1q.data_ptr(), w1_scale.data_ptr(),
                                     w2q.data_ptr(), w2_scale.data_ptr(), gating_output.data_ptr(),
                                     N.dtype_code(gating_output.dtype), M, H, F2 // 2, E, topk, int(bool(renormalize)),
                                     out.data_ptr(), ws.data_ptr(), ws.numel(), N.stream_ptr(hidden_states.device)))
    return out
