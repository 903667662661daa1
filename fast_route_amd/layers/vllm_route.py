"""Drop-in for fast_route/fast_route/layers/vllm_route.py: the baseline layer
whose routing is `hidden @ gate` followed by softmax/top-k."""
from __future__ import annotations

import torch

from .fused_moe import _check_layer
from .fused_moe import fused_moe as _fused_moe_from_logits


def fused_moe(hidden_states: torch.Tensor, gate: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, topk: int,
              renormalize: bool = True, inplace: bool = False):
    """Reference: layers/vllm_route.py:17-120 (gating GEMM at :78)."""
    _check_layer(hidden_states, w1, w2)
    gating_output = torch.matmul(hidden_states, gate)
    return _fused_moe_from_logits(hidden_states, w1, w2, gating_output, topk, renormalize, inplace)
