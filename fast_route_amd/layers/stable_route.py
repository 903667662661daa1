"""Drop-in for fast_route/fast_route/layers/stable_route.py (gate-matrix form)."""
from __future__ import annotations

import torch

from ..ops.stable_route import fused_route
from .fused_moe import _check_layer, fused_experts


def fused_moe(hidden_states: torch.Tensor, gate: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, topk: int,
              renormalize: bool = True, inplace: bool = False):
    """MoE layer with the routing computed from the gate matrix [H, E]
    (reference: layers/stable_route.py:10-102)."""
    _check_layer(hidden_states, w1, w2)
    M = hidden_states.shape[0]
    dev = hidden_states.device
    topk_weights = torch.empty((M, topk), dtype=torch.float32, device=dev)
    topk_ids = torch.empty((M, topk), dtype=torch.int32, device=dev)
    topk_weights, topk_ids = fused_route(hidden_states, gate, topk, topk_weights, topk_ids, renormalize)
    return fused_experts(hidden_states, w1, w2, topk_weights, topk_ids, inplace)
