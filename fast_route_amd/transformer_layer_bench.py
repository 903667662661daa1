"""Transformer-layer bench: attention + residual + MoE, to show the MoE share of a layer
(reference caller: benchmarks/fused_route/transformerLayer_bench.py:66-95,156).

The attention block is not part of the MoE path: it is plain PyTorch here (fused QKV
projection, scaled_dot_product_attention with a causal mask, output projection), as the
reference's own Attention module is for this bench.  The MoE is the gate-matrix entry
point of layers/stable_route.py.  Usage:

    python -m fast_route_amd.transformer_layer_bench [-n FFN] [-k HIDDEN] [-e EXPERTS] [--topk K]
        [-b BATCH] [--n_head H] [--head_dim D] [--seqs 32,64,...]

prints one JSON line per sequence length: median / p20 / p80 milliseconds of the whole
layer and of the MoE alone, the MoE share, and the reference's TFLOPS figure
(2*b*seq*n*k + 2*b*seq*seq*n_head*head_dim per layer time).
"""
from __future__ import annotations

import argparse
import json

import torch

from .layers.stable_route import fused_moe


class Attention(torch.nn.Module):
    def __init__(self, hidden: int, n_head: int, head_dim: int, dtype):
        super().__init__()
        self.n_head, self.head_dim = n_head, head_dim
        self.qkv = torch.nn.Linear(hidden, 3 * n_head * head_dim, bias=False, dtype=dtype)
        self.proj = torch.nn.Linear(n_head * head_dim, hidden, bias=False, dtype=dtype)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        b, s, _ = x.shape
        q, k, v = self.qkv(x).view(b, s, 3, self.n_head, self.head_dim).permute(2, 0, 3, 1, 4)
        o = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)
        return self.proj(o.transpose(1, 2).reshape(b, s, self.n_head * self.head_dim))


def transformer_layer(attn, x, gate, w1, w2, topk):
    """out = MoE(attn(x) + x), the reference's fused_route_transformer."""
    h = (attn(x) + x).view(-1, x.shape[-1])
    return fused_moe(h, gate, w1, w2, topk, renormalize=True, inplace=False)


def _quantiles_ms(fn, reps: int, warmup: int):
    for _ in range(warmup):
        fn()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
    for a, b in ev:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    t = sorted(a.elapsed_time(b) for a, b in ev)
    return t[len(t) // 2], t[len(t) // 5], t[(4 * len(t)) // 5]


def run(seq: int, n: int, k: int, e: int, topk: int, b: int, n_head: int, head_dim: int, seed: int = 1337,
        reps: int = 20, warmup: int = 3, dtype=torch.float16, weights=None):
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn((b, seq, k), device="cuda", dtype=dtype, generator=g) / 10
    if weights is None:
        gate = torch.randn((k, e), device="cuda", dtype=dtype, generator=g) / 10
        w1 = torch.randn((e, 2 * n, k), device="cuda", dtype=dtype, generator=g) / 10
        w2 = torch.randn((e, k, n), device="cuda", dtype=dtype, generator=g) / 10
        attn = Attention(k, n_head, head_dim, dtype).to("cuda")
        weights = (gate, w1, w2, attn)
    gate, w1, w2, attn = weights
    with torch.no_grad():
        h = (attn(x) + x).view(-1, k)
        layer = _quantiles_ms(lambda: transformer_layer(attn, x, gate, w1, w2, topk), reps, warmup)
        moe = _quantiles_ms(lambda: fused_moe(h, gate, w1, w2, topk, True, False), reps, warmup)
        out = transformer_layer(attn, x, gate, w1, w2, topk)
    flops = 2.0 * b * seq * n * k + 2.0 * b * seq * seq * n_head * head_dim  # the reference's figure
    rec = {"seq": seq, "batch": b, "layer_ms": round(layer[0], 4), "layer_ms_p20": round(layer[1], 4),
           "layer_ms_p80": round(layer[2], 4), "moe_ms": round(moe[0], 4), "moe_share": round(moe[0] / layer[0], 4),
           "ref_formula_tflops": round(flops * 1e-12 / (layer[0] * 1e-3), 3)}
    return rec, out, weights


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("-n", type=int, default=8192, help="per-expert ffn size")
    ap.add_argument("-k", type=int, default=4096, help="hidden size")
    ap.add_argument("-e", type=int, default=16, help="experts")
    ap.add_argument("--topk", type=int, default=2)
    ap.add_argument("--seed", type=int, default=1337)
    ap.add_argument("-b", type=int, default=1)
    ap.add_argument("--n_head", type=int, default=32)
    ap.add_argument("--head_dim", type=int, default=128)
    ap.add_argument("--seqs", default=",".join(str(2 ** i) for i in range(5, 15)))
    args = ap.parse_args()
    assert torch.cuda.is_available(), "needs an MI355X"
    weights = None
    for seq in [int(s) for s in args.seqs.split(",")]:
        rec, _, weights = run(seq, args.n, args.k, args.e, args.topk, args.b, args.n_head, args.head_dim, args.seed,
                              weights=weights)
        print(json.dumps(rec), flush=True)


if __name__ == "__main__":
    main()
