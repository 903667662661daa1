"""Stage-by-stage twin of the fused layer that writes a chrome-trace breakdown
(reference: fast_route/fast_route/layers/profile_fused_route.py:15-123).

The reference wraps its five launches in torch.profiler ranges (data_alloc, route,
moe_align, moe_1, silu_and_mul, moe_2) and exports a chrome trace to
./data/fused_breakdown_{M}_{K}_{E}_{N}_{topk}.json.  Here the same stages run through
the op-level C entry points, each bracketed by HIP events on the launch stream, and the
trace holds one complete ("X") event per stage with its GPU duration.  SiLU*mul is fused
into the first grouped GEMM and the top-k sum into the second, so those ranges are named
"moe_1+silu_and_mul" and "moe_2+sum".
"""
from __future__ import annotations

import json
import os

import torch

from .. import _native as N
from ..ops.stable_route import fused_route
from .fused_moe import _check_layer, plan

STAGES = ("data_alloc", "route", "moe_align", "moe_1+silu_and_mul", "moe_2+sum")


def fused_moe(hidden_states: torch.Tensor, gate: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, topk: int,
              renormalize: bool = True, inplace: bool = False, save_dir: str = "./data"):
    """Same signature and result as layers.stable_route.fused_moe; additionally writes
    `fused_breakdown_{M}_{K}_{E}_{N}_{topk}.json` under save_dir and returns the output.
    The per-stage microseconds of the last call are kept in `fused_moe.last_breakdown`."""
    _check_layer(hidden_states, w1, w2)
    M, K = hidden_states.shape
    E, N2, _ = w1.shape
    F = N2 // 2
    dev = hidden_states.device
    lib, st, code = N.lib(), N.stream_ptr(dev), N.dtype_code(hidden_states.dtype)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(len(STAGES) + 1)]

    ev[0].record()
    p = plan(M, K, F, E, topk, hidden_states.dtype)
    n = M * topk
    topk_weights = torch.empty((M, topk), dtype=torch.float32, device=dev)
    topk_ids = torch.empty((M, topk), dtype=torch.int32, device=dev)
    sorted_ids = torch.empty((max(p.sorted_len, 1),), dtype=torch.int32, device=dev)
    expert_ids = torch.empty((n + E,), dtype=torch.int32, device=dev)
    npost = torch.empty((1,), dtype=torch.int32, device=dev)
    align_bytes = lib.fr_moe_align_workspace_bytes(n, E)
    align_ws = torch.empty((max(align_bytes, 256),), dtype=torch.uint8, device=dev)
    act = torch.empty((max(p.sorted_len, 1), F), dtype=hidden_states.dtype, device=dev)
    partial = torch.empty((p.split_k * max(n, 1) * K,), dtype=torch.float32, device=dev)
    tail = torch.empty((p.tail_bytes,), dtype=torch.uint8, device=dev) if p.tail_bytes else None
    tail_ptr = tail.data_ptr() if tail is not None else None
    out = hidden_states if inplace else torch.empty_like(hidden_states)
    ev[1].record()

    topk_weights, topk_ids = fused_route(hidden_states, gate, topk, topk_weights, topk_ids, renormalize)
    ev[2].record()

    N.check(lib.fr_moe_align(topk_ids.data_ptr(), N.FR_I32, n, E, p.block, sorted_ids.data_ptr(),
                             expert_ids.data_ptr(), npost.data_ptr(), align_ws.data_ptr(), align_bytes, st))
    ev[3].record()

    N.check(lib.fr_moe_gateup_silu(hidden_states.data_ptr(), w1.data_ptr(), sorted_ids.data_ptr(),
                                   expert_ids.data_ptr(), npost.data_ptr(), M, K, F, E, topk, p.block, code,
                                   act.data_ptr(), tail_ptr, st))
    ev[4].record()

    N.check(lib.fr_moe_down_combine(act.data_ptr(), w2.data_ptr(), topk_weights.data_ptr(), sorted_ids.data_ptr(),
                                    expert_ids.data_ptr(), npost.data_ptr(), M, K, F, E, topk, p.block, p.split_k,
                                    code, partial.data_ptr(), out.data_ptr(), tail_ptr, st))
    ev[5].record()
    ev[5].synchronize()

    durs = [ev[i].elapsed_time(ev[i + 1]) * 1e3 for i in range(len(STAGES))]  # microseconds
    events, ts = [], 0.0
    for name, d in zip(STAGES, durs):
        events.append({"name": name, "ph": "X", "pid": 0, "tid": 0, "ts": round(ts, 3), "dur": round(d, 3),
                       "cat": "fused_moe", "args": {"M": M, "K": K, "E": E, "N": N2, "topk": topk,
                                                    "block": p.block, "split_k": p.split_k}})
        ts += d
    os.makedirs(save_dir, exist_ok=True)
    save_path = os.path.join(save_dir, f"fused_breakdown_{M}_{K}_{E}_{N2}_{topk}.json")
    with open(save_path, "w") as f:
        json.dump({"traceEvents": events, "displayTimeUnit": "ns"}, f)
    fused_moe.last_breakdown = dict(zip(STAGES, durs))
    fused_moe.last_trace_path = save_path
    return out
