"""Benchmark of the fused MoE layer on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--tokens M] [--no-sweep] [--no-cpu] [--no-configs]
    python bench.py -n 8192 -k 4096 -e 16 --topk 2 --reference-protocol      (the reference's own sweep, fp16 randn/10)

A step is one pass of the whole layer (gating -> routing arrays -> gate/up GEMM
with SiLU*mul -> down GEMM with routed weight -> top-k combine) over one batch
of M synthetic tokens of the Mixtral-8x7B shape (H4096, F14336, E8, top-2, bf16).
Inputs and weights are resident in HBM before the timed region.  Prints ONE JSON
line: the headline token count (default 4096), the per-stage times measured with
events on the launch stream, the roofline of the dominant kernel, the token sweep
and the CPU baseline (the fp32 PyTorch oracle on the host cores, bounded sample).
Unless --no-configs is given the same line also carries compact records of the other
workloads: the small layer (caches flushed between repetitions), the routing-only stress
case (bit-exact flag), the fine-grained many-expert sweep and the fp8 sweep, each with
its bound, roofline fraction and the error of one point against the CPU oracle.
"""
from __future__ import annotations

import argparse
import hashlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_FP8_TFLOPS = 5000.0   # MI355X dense fp8 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E
SHAPES = {
    "mixtral": dict(H=4096, F=14336, E=8, topk=2, zipf=False, sweep=[1, 16, 64, 256, 512, 1024, 2048, 4096, 16384]),
    "fine": dict(H=2048, F=1408, E=64, topk=6, zipf=True, sweep=[1, 32, 128, 512, 2048, 8192]),
    "small": dict(H=1024, F=3584, E=8, topk=2, zipf=False, sweep=[64]),
    "mixtral22b": dict(H=6144, F=16384, E=8, topk=2, zipf=False, sweep=[1, 16, 128, 1024, 4096]),
}


def layer_flops(M, H, F, topk):
    return 6.0 * M * topk * H * F


def layer_bytes(M, H, F, E, topk, active, bw=2, ba=2):
    """Algorithmic HBM bytes of one layer pass: active experts' weights once,
    tokens in, logits, activated intermediate written and read once, output,
    top-k weights/ids written and read."""
    return (active * 3 * F * H * bw + M * H * ba + M * E * 4 + 2 * M * topk * F * ba + M * H * ba + 16 * M * topk)


class Layer:
    """Device buffers + staged calls through the C ABI for one (shape, M)."""

    def __init__(self, torch, N, shape, M, w1, w2, seed, fp8=None, dtype=None, x_scale=1.0, prepared=False):
        self.torch, self.N, self.M = torch, N, M
        self.tdtype = dtype or torch.bfloat16
        self.code = N.dtype_code(self.tdtype)
        # prepared: the layout flags prepare_weights returned for w1, w2; they ride on the weight-taking calls' dtype
        self.wcode = self.code | int(prepared or 0)
        self.fp8 = fp8  # (w1q, w1_scale, w2q, w2_scale) or None
        self.H, self.F, self.E, self.topk = shape["H"], shape["F"], shape["E"], shape["topk"]
        dev = "cuda"
        g = torch.Generator(device=dev).manual_seed(seed + M)
        self.x = (torch.randn(M, self.H, generator=g, device=dev) * x_scale).to(self.tdtype)
        if shape["zipf"]:
            r = (torch.randperm(self.E, generator=g, device=dev) + 1).double()
            pz = r.pow(-1.2)
            self.logits = (torch.log(pz / pz.sum()).float()[None, :] + torch.randn(M, self.E, generator=g, device=dev))
        else:
            self.logits = torch.randn(M, self.E, generator=g, device=dev)
        self.w1, self.w2 = w1, w2
        self.plan = N.FrMoePlan()
        N.check(N.lib().fr_moe_get_plan(M, self.H, self.F, self.E, self.topk, N.FR_FP8_E4M3 if fp8 else self.code, self.plan))
        p, n = self.plan, M * self.topk
        self.ws = torch.empty(max(p.workspace_bytes, 256), dtype=torch.uint8, device=dev)
        self.out = torch.empty(M, self.H, dtype=self.tdtype, device=dev)
        # staged buffers
        self.tw = torch.empty(n, dtype=torch.float32, device=dev)
        self.ti = torch.empty(n, dtype=torch.int32, device=dev)
        self.sorted = torch.empty(p.sorted_len, dtype=torch.int32, device=dev)
        self.eids = torch.empty(n + self.E, dtype=torch.int32, device=dev)
        self.npost = torch.empty(1, dtype=torch.int32, device=dev)
        self.aws_bytes = N.lib().fr_moe_align_workspace_bytes(n, self.E)
        self.aws = torch.empty(max(self.aws_bytes, 256), dtype=torch.uint8, device=dev)
        self.act = torch.empty(p.sorted_len, self.F, dtype=self.tdtype, device=dev)
        self.partial = torch.empty(p.split_k * n * self.H, dtype=torch.float32, device=dev)
        self.tail = torch.empty(p.tail_bytes, dtype=torch.uint8, device=dev) if p.tail_bytes else None
        if fp8:
            self.xq = torch.empty(M, self.H, dtype=torch.uint8, device=dev)
            self.xs = torch.empty(M, dtype=torch.float32, device=dev)
            self.actq = torch.empty(p.sorted_len, self.F, dtype=torch.uint8, device=dev)
            self.acts = torch.ones(p.sorted_len, dtype=torch.float32, device=dev)
        self.stream = torch.cuda.current_stream().cuda_stream

    def fused(self):
        N = self.N
        if self.fp8:
            w1q, w1s, w2q, w2s = self.fp8
            N.check(N.lib().fr_fused_moe_fp8(self.x.data_ptr(), N.FR_BF16, w1q.data_ptr(), w1s.data_ptr(), w2q.data_ptr(),
                                             w2s.data_ptr(), self.logits.data_ptr(), N.FR_F32, self.M, self.H, self.F, self.E,
                                             self.topk, 1, self.out.data_ptr(), self.ws.data_ptr(), self.ws.numel(), self.stream))
            return
        N.check(N.lib().fr_fused_moe(self.x.data_ptr(), self.w1.data_ptr(), self.w2.data_ptr(), self.logits.data_ptr(),
                                     N.FR_F32, self.M, self.H, self.F, self.E, self.topk, 1, self.wcode,
                                     self.out.data_ptr(), self.ws.data_ptr(), self.ws.numel(), self.stream))

    def staged(self, events=None):
        N, lib, p = self.N, self.N.lib(), self.plan
        rec = (lambda i: events[i].record()) if events else (lambda i: None)
        rec(0)
        N.check(lib.fr_gating_topk(self.logits.data_ptr(), N.FR_F32, self.M, self.E, self.E, self.topk, 1,
                                   self.tw.data_ptr(), self.ti.data_ptr(), self.stream))
        rec(1)
        N.check(lib.fr_moe_align(self.ti.data_ptr(), N.FR_I32, self.M * self.topk, self.E, p.block, self.sorted.data_ptr(),
                                 self.eids.data_ptr(), self.npost.data_ptr(), self.aws.data_ptr(), self.aws_bytes, self.stream))
        rec(2)
        if self.fp8:
            w1q, w1s, w2q, w2s = self.fp8
            N.check(lib.fr_quant_e4m3_rows(self.x.data_ptr(), N.FR_BF16, self.M, self.H, self.H, self.xq.data_ptr(),
                                           self.xs.data_ptr(), self.stream))
            N.check(lib.fr_moe_gateup_silu_fp8(self.xq.data_ptr(), self.xs.data_ptr(), w1q.data_ptr(), w1s.data_ptr(),
                                               self.sorted.data_ptr(), self.eids.data_ptr(), self.npost.data_ptr(), self.M,
                                               self.H, self.F, self.E, self.topk, p.block, self.act.data_ptr(), self.stream))
            rec(3)
            N.check(lib.fr_quant_e4m3_rows(self.act.data_ptr(), N.FR_BF16, p.sorted_len, self.F, self.F, self.actq.data_ptr(),
                                           self.acts.data_ptr(), self.stream))
            N.check(lib.fr_moe_down_combine_fp8(self.actq.data_ptr(), self.acts.data_ptr(), w2q.data_ptr(), w2s.data_ptr(),
                                                self.tw.data_ptr(), self.sorted.data_ptr(), self.eids.data_ptr(),
                                                self.npost.data_ptr(), self.M, self.H, self.F, self.E, self.topk, p.block,
                                                p.split_k, N.FR_BF16, self.partial.data_ptr(), self.out.data_ptr(),
                                                self.tail.data_ptr() if self.tail is not None else None, self.stream))
            rec(4)
            return
        N.check(lib.fr_moe_gateup_silu(self.x.data_ptr(), self.w1.data_ptr(), self.sorted.data_ptr(), self.eids.data_ptr(),
                                       self.npost.data_ptr(), self.M, self.H, self.F, self.E, self.topk, p.block, self.wcode,
                                       self.act.data_ptr(), self.tail.data_ptr() if self.tail is not None else None,
                                       self.stream))
        rec(3)
        N.check(lib.fr_moe_down_combine(self.act.data_ptr(), self.w2.data_ptr(), self.tw.data_ptr(), self.sorted.data_ptr(),
                                        self.eids.data_ptr(), self.npost.data_ptr(), self.M, self.H, self.F, self.E,
                                        self.topk, p.block, p.split_k, self.wcode, self.partial.data_ptr(),
                                        self.out.data_ptr(), self.tail.data_ptr() if self.tail is not None else None,
                                        self.stream))
        rec(4)

    def active_experts(self):
        return int(self.torch.unique(self.ti).numel())


_FLUSH = {}


def flush_caches(torch):
    """Writes 512 MiB: twice the 256 MB Infinity Cache, so nothing of the layer's operands survives in it or in L2."""
    if "buf" not in _FLUSH:
        _FLUSH["buf"] = torch.empty(512 << 20, dtype=torch.uint8, device="cuda")
    _FLUSH["buf"].fill_(1)


def time_layer(torch, layer, steps, warmup, flush=False):
    """flush: the weights fit the Infinity Cache (small workloads); every repetition then starts from cold caches
    (one event pair per repetition, the flush outside it) instead of running back to back."""
    for _ in range(warmup):
        layer.fused()
    torch.cuda.synchronize()
    if flush:
        wall_ms = None
    else:
        t0 = time.perf_counter()
        for _ in range(steps):
            layer.fused()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    # per-step spread (median, 20th and 80th percentile) from one event pair per step
    pe = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for a, b in pe:
        if flush:
            flush_caches(torch)
        a.record()
        layer.fused()
        b.record()
    torch.cuda.synchronize()
    per = sorted(a.elapsed_time(b) * 1e3 for a, b in pe)
    quant = {"p20": per[len(per) // 5], "p50": per[len(per) // 2], "p80": per[(4 * len(per)) // 5]}
    if flush:
        wall_ms = quant["p50"] / 1e3
    # per-stage times: the same kernels launched stage by stage with events on the launch stream
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(5)] for _ in range(steps)]
    layer.staged()
    torch.cuda.synchronize()
    for s in range(steps):
        if flush:
            flush_caches(torch)
        layer.staged(evs[s])
    torch.cuda.synchronize()
    names = ["route", "moe_align", "moe_1+silu_and_mul", "moe_2+sum"]
    stage_us = {nm: sum(evs[s][i].elapsed_time(evs[s][i + 1]) for s in range(steps)) * 1e3 / steps
                for i, nm in enumerate(names)}
    return wall_ms, stage_us, quant


def measure(torch, N, shape, M, w1, w2, steps, warmup, seed, fp8=None, flush=False, dtype=None, x_scale=1.0, prepared=False):
    layer = Layer(torch, N, shape, M, w1, w2, seed, fp8, dtype=dtype, x_scale=x_scale, prepared=prepared)
    if fp8:  # pad rows of act beyond npost are never written: keep them finite for the staged quantisation
        layer.act.zero_()
    wall_ms, stage_us, quant = time_layer(torch, layer, steps, warmup, flush)
    H, F, E, topk = shape["H"], shape["F"], shape["E"], shape["topk"]
    active = layer.active_experts()
    fl = layer_flops(M, H, F, topk)
    by = layer_bytes(M, H, F, E, topk, active, bw=1 if fp8 else 2) + (active * (2 * F + H) * 4 + (M + M * topk) * 4 if fp8 else 0)
    t = wall_ms * 1e-3
    peak = PEAK_FP8_TFLOPS if fp8 else PEAK_BF16_TFLOPS
    t_hbm, t_mfma = by / (PEAK_HBM_GBS * 1e9), fl / (peak * 1e12)
    bound = "hbm" if t_hbm >= t_mfma else "mfma"
    rec = {
        "tokens": M, "us_per_layer": round(wall_ms * 1e3, 2),
        "us_per_layer_p20_p50_p80": [round(quant["p20"], 2), round(quant["p50"], 2), round(quant["p80"], 2)], "tflops": round(fl / t / 1e12, 3),
        "gbps": round(by / t / 1e9, 1), "active_experts": active, "bound": bound,
        "roofline_frac": round(max(t_hbm, t_mfma) / t, 4), "block": layer.plan.block, "split_k": layer.plan.split_k,
        "stage_us": {k: round(v, 2) for k, v in stage_us.items()},
        "ref_2mnk_tflops": round(2.0 * M * F * H / t / 1e12, 3),
    }
    if flush:
        rec["cache_flush"] = "512 MiB written before every timed repetition"
    return rec, layer


def graph_replay_us(torch, layer, reps=20, per_graph=8):
    """Median time of one layer pass when `per_graph` passes are captured into one HIP graph and the graph
    is replayed: what a serving loop that captures its launch-bound steps pays per layer.  The fused entry
    point launches kernels only (no allocation, no memset node), so it is captured as it is."""
    layer.fused()  # first call outside the capture: set-up of the kernels' attributes
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    keep = layer.stream
    with torch.cuda.stream(side):
        layer.stream = side.cuda_stream
        with torch.cuda.graph(graph, stream=side):
            for _ in range(per_graph):
                layer.fused()
        layer.stream = keep
    ref = layer.out.clone()
    times = []
    for _ in range(reps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record(); graph.replay(); b.record()
        torch.cuda.synchronize()
        times.append(a.elapsed_time(b) * 1e3 / per_graph)
    assert torch.equal(layer.out, ref), "graph replay changed the layer's output"
    return round(sorted(times)[len(times) // 2], 2)


def kernel_roofline(shape, rec, fp8=False):
    """Roofline of the dominant kernel (gate/up grouped GEMM + SiLU*mul) from its
    event-measured average duration."""
    M, H, F, topk = rec["tokens"], shape["H"], shape["F"], shape["topk"]
    dur = rec["stage_us"]["moe_1+silu_and_mul"] * 1e-6
    flops = 4.0 * M * topk * H * F
    eb = 1 if fp8 else 2
    byts = rec["active_experts"] * 2 * F * H * eb + M * H * eb + M * topk * F * 2
    peak = PEAK_FP8_TFLOPS if fp8 else PEAK_BF16_TFLOPS
    # which kernel the library picks for the gate/up GEMM: weight rows against token rows for up to 4
    # tokens of 2-byte operands with H = 4096, 5120, 6144, 7168 or 8192, the one-wavefront-per-SIMD kernel for 256-row
    # blocks with a K of 16 K tiles or more, the persistent tile kernel for 64-, 128- and 160-row blocks (and 256-row
    # blocks of 2-byte operands with a short K), the plain tile kernel otherwise
    if not fp8 and M <= 4 and H >= 4096 and H % 512 == 0 and any(H // 512 % c == 0 for c in (5, 6, 7, 8)) and M * H * 2 <= 65536:
        name = "gateup_rows_kernel"
    elif rec["block"] == 256 and H >= (2048 if fp8 else 1024):  # 16 K tiles of 128 bytes per row or more
        name = "moe_gemm_quad_kernel<EPI_SILU>"
    elif rec["block"] in (64, 128, 160) or (rec["block"] == 256 and not fp8):
        name = "moe_gemm_persistent_kernel<EPI_SILU>"
    else:
        name = "moe_gemm_kernel<EPI_SILU>"
    if flops / (peak * 1e12) >= byts / (PEAK_HBM_GBS * 1e9):
        ach = flops / dur / 1e12
        return {"kernel": name, "bound": "mfma", "achieved": round(ach, 2), "peak": peak,
                "unit": "TFLOP/s", "frac": round(ach / peak, 4), "traffic": None,
                "avg_launch_us": round(dur * 1e6, 2), "algorithmic_flops_per_launch": flops}
    ach = byts / dur / 1e9
    return {"kernel": name, "bound": "hbm", "achieved": round(ach, 1), "peak": PEAK_HBM_GBS,
            "unit": "GB/s", "frac": round(ach / PEAK_HBM_GBS, 4), "traffic": None,
            "avg_launch_us": round(dur * 1e6, 2), "algorithmic_bytes_per_launch": byts}


def tunables_now(N):
    """The library's study knobs at the time of the run (all zero = every choice left to the plan)."""
    import ctypes
    t = N.FrMoeTunables()
    N.check(N.lib().fr_moe_get_tunables(ctypes.byref(t)))
    return {name: int(getattr(t, name)) for name, _ in t._fields_}


GEMM_KERNEL_SOURCES = ("moe_gemm_kernel.h", "moe_gemm_persistent.h", "moe_gemm_quad.h", "moe_gemm_tiles.h", "moe_gemv.h", "moe_gemm.hip")


def kernel_sources_sha():
    """Hash of the sources of the grouped-GEMM kernels (tile kernels, their persistent form, the tile table and
    dispatch, the weight-row kernels): ties an offline counter record to the kernels it measured."""
    root = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fast_route_amd", "csrc")
    h = hashlib.sha256()
    for name in GEMM_KERNEL_SOURCES:
        with open(os.path.join(root, name), "rb") as f:
            h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()[:16]


def recorded_traffic(metric, block):
    """HBM bytes per launch of the dominant kernel for this workload, as measured offline with
    rocprofv3 --pmc (FETCH_SIZE and WRITE_SIZE runs, scaled by the copy probe) and recorded
    in profiles/hbm_traffic.json; None when the workload has no record, when the record was taken
    with other GEMM kernel sources than the ones present, or when the plan now picks another
    routing block (i.e. another tile) for this workload than the one that was measured."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "hbm_traffic.json")
    try:
        with open(path) as f:
            doc = json.load(f)
    except (OSError, ValueError):
        return None
    rec = doc.get(metric)
    if not rec or doc.get("kernel_sources_sha") != kernel_sources_sha() or rec.get("block") != block:
        return None
    return rec["traffic_bytes"]


def host_cpu():
    """(threads the CPU legs use, CPU model): the box's CPU share when the environment states one, else every core."""
    n = os.cpu_count() or 1
    try:
        n = min(n, int(os.environ.get("OMP_NUM_THREADS", n)))
    except ValueError:
        pass
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return max(n, 1), model


def cpu_baseline(torch, shape, layer, sample_tokens):
    """fp32 PyTorch oracle on the host cores over the first `sample_tokens` tokens of the same batch."""
    import oracle
    threads, model = host_cpu()
    torch.set_num_threads(threads)
    m = min(sample_tokens, layer.M)
    x, logits = layer.x[:m].cpu(), layer.logits[:m].cpu()
    w1, w2 = layer.w1.cpu(), layer.w2.cpu()
    times, spent = [], 0.0
    while len(times) < 3 and spent < 12.0:  # a bounded sample: up to three passes, about 10 s of CPU work
        t0 = time.perf_counter()
        ref = oracle.fused_moe(x, w1, w2, logits, shape["topk"], True)
        times.append(time.perf_counter() - t0)
        spent += times[-1]
    dt = sorted(times)[len(times) // 2]
    got = layer.out[:m].float().cpu()
    err = (got - ref).abs().max().item()
    return {"value": round(layer_flops(m, shape["H"], shape["F"], shape["topk"]) / dt / 1e12, 4), "unit": "TFLOP/s",
            "cores": threads, "kind": "port", "cpu_model": model, "host_cpus": os.cpu_count(),
            "sample": "fp32 PyTorch oracle, first %d tokens of the M=%d batch, weights upcast per expert, median of %d passes, %.1f s each"
                      % (m, layer.M, len(times), dt),
            "us_per_layer_sample": round(dt * 1e6, 0), "max_abs_err_vs_gpu": err,
            "ref_max_abs": ref.abs().max().item()}


def oracle_error(torch, shape, layer, tokens=48, fp8=None, plain=None):
    """Max-abs error of the layer's last output against the CPU oracle on an evenly spaced sample of tokens.
    plain: (w1, w2) as the reference lays them out, when the layer holds prepared (re-laid-out) weights."""
    import oracle
    layer.fused()
    torch.cuda.synchronize()
    M = layer.M
    idx = torch.arange(M) if M <= tokens else torch.arange(0, M, M // tokens)[:tokens]
    x, logits = layer.x[idx.cuda()].cpu(), layer.logits[idx.cuda()].cpu()
    if fp8:
        # the GPU-prepared codes and scales are bit-identical to the oracle's own (a GPU test holds that):
        # handing them over saves the CPU from quantising 1.4e9 weights
        w1q, w1s, w2q, w2s = fp8
        E, F2, H = w1q.shape
        wq = (w1q.cpu().numpy().reshape(E * F2, H), w1s.cpu().numpy().reshape(-1),
              w2q.cpu().numpy().reshape(E * w2q.shape[1], w2q.shape[2]), w2s.cpu().numpy().reshape(-1))
        ref, _ = oracle.fused_moe_fp8(x, layer.w1.cpu(), layer.w2.cpu(), logits, shape["topk"], True, weights_q=wq)
    else:
        pw1, pw2 = plain if plain is not None else (layer.w1, layer.w2)
        ref = oracle.fused_moe(x, pw1.cpu(), pw2.cpu(), logits, shape["topk"], True)
    got = layer.out[idx.cuda()].float().cpu()
    return {"tokens_checked": int(idx.numel()), "max_abs_err": (got - ref).abs().max().item(),
            "ref_max_abs": ref.abs().max().item(),
            "rel_frobenius_err": ((got - ref).norm() / ref.norm()).item()}


def routing_bench(torch, N, steps, warmup, seed):
    """Routing-only stress workload: 65536 tokens, 64 experts, top-6, Zipf(1.2)-skewed
    logits; gating + block-aligned sort for block in {16, 32, 64, 128}, checked bit-exact
    against the CPU oracle once, then timed."""
    import numpy as np
    import oracle
    M, E, k = 65536, 64, 6
    logits = oracle.zipf_logits(M, E, seed)
    dl = logits.cuda()
    n = M * k
    tw = torch.empty(n, dtype=torch.float32, device="cuda")
    ti = torch.empty(n, dtype=torch.int32, device="cuda")
    lib, st = N.lib(), torch.cuda.current_stream().cuda_stream
    ws_bytes = lib.fr_moe_align_workspace_bytes(n, E)
    ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device="cuda")
    _, ref_ids = oracle.gating_topk(logits, k, True)
    out = []
    for B in (16, 32, 64, 128):
        sl = n + E * (B - 1)
        s_ = torch.empty(sl, dtype=torch.int32, device="cuda")
        e_ = torch.empty(n + E, dtype=torch.int32, device="cuda")
        p_ = torch.empty(1, dtype=torch.int32, device="cuda")

        def gate():
            N.check(lib.fr_gating_topk(dl.data_ptr(), N.FR_F32, M, E, E, k, 1, tw.data_ptr(), ti.data_ptr(), st))

        def align():
            N.check(lib.fr_moe_align(ti.data_ptr(), N.FR_I32, n, E, B, s_.data_ptr(), e_.data_ptr(), p_.data_ptr(),
                                     ws.data_ptr(), ws_bytes, st))
        gate(); align(); torch.cuda.synchronize()
        rs, re_, rn = oracle.moe_align_block_size(ref_ids, B, E)
        exact = bool(torch.equal(ti.cpu().view(M, k), ref_ids) and np.array_equal(s_.cpu().numpy(), rs)
                     and int(p_.cpu()[0]) == int(rn[0]))
        for _ in range(warmup):
            gate(); align()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
        tg = ta = 0.0
        for _ in range(steps):
            ev[0].record(); gate(); ev[1].record(); align(); ev[2].record()
            torch.cuda.synchronize()
            tg += ev[0].elapsed_time(ev[1]); ta += ev[1].elapsed_time(ev[2])
        npost = int(p_.cpu()[0])
        a_bytes = 4 * n + 4 * npost + 4 * (npost // B) + 4
        g_bytes = M * E * 4 + 8 * n
        out.append({"block": B, "bit_exact": exact, "gating_us": round(tg * 1e3 / steps, 2),
                    "align_us": round(ta * 1e3 / steps, 2), "align_ns_per_pair": round(ta * 1e6 / steps / n, 4),
                    "align_gbps": round(a_bytes / (ta * 1e-3 / steps) / 1e9, 2),
                    "gating_gbps": round(g_bytes / (tg * 1e-3 / steps) / 1e9, 1), "npost": npost})
    return out


def make_weights(torch, shape, seed, dtype=None, scale=0.02):
    H, F, E = shape["H"], shape["F"], shape["E"]
    dt = dtype or torch.bfloat16
    g = torch.Generator(device="cuda").manual_seed(seed)
    w1 = (torch.randn(E, 2 * F, H, generator=g, device="cuda") * scale).to(dt)
    w2 = (torch.randn(E, H, F, generator=g, device="cuda") * scale).to(dt)
    return w1, w2


def compact(rec):
    return {k: rec[k] for k in ("tokens", "us_per_layer", "tflops", "gbps", "bound", "roofline_frac", "block", "split_k")}


def other_configs(torch, N, args, mixtral_weights):
    """Compact records of the workloads the headline does not cover."""
    out = {}
    steps, warmup = args.steps, args.warmup
    # small layer: 176 MB of weights fit the 256 MB Infinity Cache -> flush between repetitions
    shape = SHAPES["small"]
    w1, w2 = make_weights(torch, shape, args.seed)
    rec, layer = measure(torch, N, shape, 64, w1, w2, steps, warmup, args.seed, flush=True)
    warm, wlayer = measure(torch, N, shape, 64, w1, w2, steps, warmup, args.seed)
    out["small"] = dict(compact(rec), stage_us=rec["stage_us"], cache_flush=rec["cache_flush"],
                        us_per_layer_back_to_back=warm["us_per_layer"],
                        us_per_layer_graph_replay=graph_replay_us(torch, wlayer),
                        vs_oracle=oracle_error(torch, shape, layer, 64))
    del wlayer
    del w1, w2, layer
    # routing-only stress: gating + block-aligned sort, bit-exact against the oracle
    out["routing_stress"] = {"tokens": 65536, "experts": 64, "topk": 6, "bound": "hbm (latency bound in practice)",
                             "blocks": routing_bench(torch, N, steps, warmup, args.seed)}
    # fine-grained many-expert layer
    shape = SHAPES["fine"]
    w1, w2 = make_weights(torch, shape, args.seed)
    sweep = []
    for M in shape["sweep"]:
        rec, layer = measure(torch, N, shape, M, w1, w2, steps, warmup, args.seed)
        sweep.append(dict(compact(rec), stage_us=rec["stage_us"]))
        if M == 1:  # four launches of a few microseconds each: the launch-bound end
            sweep[-1]["us_per_layer_graph_replay"] = graph_replay_us(torch, layer)
    out["fine"] = {"workload": "H=2048 F=1408 E=64 top-6, Zipf(1.2)-skewed load, bf16", "sweep": sweep,
                   "vs_oracle_M8192": oracle_error(torch, shape, layer)}
    del w1, w2, layer
    # fp8 Mixtral
    from fast_route_amd import prepare_weights_fp8
    shape = SHAPES["mixtral"]
    w1, w2 = mixtral_weights
    fp8 = prepare_weights_fp8(w1, w2)
    sweep = []
    for M in (16, 256, 1024, 4096):
        rec, layer = measure(torch, N, shape, M, w1, w2, steps, warmup, args.seed, fp8)
        sweep.append(dict(compact(rec), stage_us=rec["stage_us"]))
    out["fp8"] = {"workload": "Mixtral shape, e4m3 weights (scale per expert and output channel), bf16 activations quantised per token",
                  "peak_tflops": PEAK_FP8_TFLOPS, "sweep": sweep,
                  "vs_oracle_M4096": oracle_error(torch, shape, layer, 24, fp8=fp8)}
    del fp8, layer
    # Mixtral shape again with the down-projection weights in the prepared layout (prepare_weights, its default)
    from fast_route_amd import prepare_weights
    _, w2p, flags = prepare_weights(w1, w2, "w2")
    sweep = []
    for M in (16, 256, 1024, 4096, 16384):
        rec, layer = measure(torch, N, shape, M, w1, w2p, steps, warmup, args.seed, prepared=flags)
        sweep.append(dict(compact(rec), stage_us=rec["stage_us"]))
    out["prepared_w2"] = {"workload": "Mixtral shape bf16, w2 re-laid-out once by prepare_weights (64-row x 128-byte tiles); w1 as the reference has it",
                          "sweep": sweep, "vs_oracle_M16384": oracle_error(torch, shape, layer, plain=(w1, w2))}
    del w2p, layer
    return out


def reference_protocol(torch, N, args):
    """The reference's own benchmark protocol (benchmarks/fused_route/moe_bench.py:10-38,53,83-99): fp16 operands
    drawn as randn / 10, shape from -n (ffn) -k (hidden) -e --topk, m = 2^0 .. 2^14, the GATE-MATRIX layer
    fused_moe(a, gate, w1, w2, topk, True, False) as the timed call (:92-94; routing GEMM, Python and allocations
    included, as the reference times them), median of the repetitions (its do_bench quantile 0.5), and its "TFLOPS"
    figure 2*m*n*k / t (a sixth of the layer's real work at top-2) next to the real one."""
    from fast_route_amd.layers.stable_route import fused_moe as gate_matrix_layer
    from fast_route_amd.layers.fused_moe import plan
    shape = dict(H=args.k, F=args.n, E=args.e, topk=args.topk, zipf=False)
    w1, w2 = make_weights(torch, shape, args.seed, torch.float16, 0.1)
    g = torch.Generator(device="cuda").manual_seed(args.seed)
    gate = (torch.randn(args.k, args.e, generator=g, device="cuda") / 10).half()
    rows = []
    for m in ([args.tokens] if args.no_sweep else [2 ** i for i in range(15)]):
        a = (torch.randn(m, args.k, generator=g, device="cuda") / 10).half()
        for _ in range(args.warmup):
            gate_matrix_layer(a, gate, w1, w2, args.topk, True, False)
        torch.cuda.synchronize()
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
        for e0, e1 in ev:
            e0.record()
            gate_matrix_layer(a, gate, w1, w2, args.topk, True, False)
            e1.record()
        torch.cuda.synchronize()
        t = sorted(e0.elapsed_time(e1) for e0, e1 in ev)[len(ev) // 2] * 1e-3
        rows.append({"m": m, "us_per_layer": round(t * 1e6, 2), "ref_2mnk_tflops": round(2.0 * m * args.n * args.k / t / 1e12, 3),
                     "tflops": round(layer_flops(m, args.k, args.n, args.topk) / t / 1e12, 3),
                     "block": plan(m, args.k, args.n, args.e, args.topk, torch.float16).block})
    return {"protocol": "fp16, randn/10, n=%d k=%d e=%d topk=%d, gate-matrix layer fused_moe(a, gate, w1, w2, topk, True, False), "
                        "median of %d event-timed calls" % (args.n, args.k, args.e, args.topk, args.steps),
            "ref_2mnk_tflops_is": "2*m*n*k / t, the figure the reference plots (README moe_bench.png)", "rows": rows}


def mfma_stream(torch, N):
    """The part's sustained rate on a pure MFMA stream (fr_probe_mfma_stream): per MFMA shape, wavefronts per SIMD and
    operand data; the shader clock from the ratio of the cycle counter to the 100 MHz counter."""
    lib = N.lib()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    sink = torch.empty(512 * cus, dtype=torch.float32, device="cuda")
    counts = torch.zeros(2, dtype=torch.int64, device="cuda")
    g = torch.Generator(device="cuda").manual_seed(1)
    data = {"random bf16 in [1, 2) with random signs": (torch.rand(32768, generator=g, device="cuda") + 1.0) *
            (torch.randint(0, 2, (32768,), generator=g, device="cuda") * 2 - 1),
            "zeros": torch.zeros(32768, device="cuda")}
    rows = []
    for what, vals in data.items():
        ops = vals.to(torch.bfloat16).contiguous()
        for shape in (32, 16):
            for wps in (1, 2):
                iters = 3000 * (1 if shape == 32 else 1) // 1
                per_iter = (16 if wps == 1 else 8) if shape == 32 else (64 if wps == 1 else 32)  # MFMAs per wavefront and iteration
                best = None
                for _ in range(3):
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    N.check(lib.fr_probe_mfma_stream(shape, wps, iters, ops.data_ptr(), sink.data_ptr(), counts.data_ptr(),
                                                     torch.cuda.current_stream().cuda_stream))
                    e1.record()
                    torch.cuda.synchronize()
                    ms = e0.elapsed_time(e1)
                    cyc, ticks = (int(v) for v in counts.cpu())
                    if best is None or ms < best[0]:
                        best = (ms, cyc, ticks)
                ms, cyc, ticks = best
                mfmas = iters * per_iter                       # per wavefront
                flop = mfmas * 32768.0 * (1 if shape == 32 else 0.5) * 4 * wps * cus
                rows.append({"operands": what, "mfma": "32x32x16" if shape == 32 else "16x16x32", "waves_per_simd": wps,
                             "ms": round(ms, 3), "tflops": round(flop / ms / 1e9, 1),
                             "shader_clock_ghz": round(cyc / (ticks * 10.0), 3),
                             "mfma_pipe_busy": round(mfmas * (32 if shape == 32 else 16) * wps / cyc, 3)})
    return {"metric": "mfma_stream_bf16", "unit": "TFLOP/s", "compute_units": cus, "rows": rows}


def vendor_gemm(torch, tokens, shape, steps):
    """torch.matmul (the vendor's dense GEMM) on the two GEMM shapes of the layer at `tokens` tokens - the same flops,
    no gather, no SiLU, no routed weight: what a dense kernel sustains on this box next to the grouped ones."""
    H, F, topk = shape["H"], shape["F"], shape["topk"]
    g = torch.Generator(device="cuda").manual_seed(3)
    rows = []
    for name, (m, n, k) in {"gate/up": (tokens * topk, 2 * F, H), "down": (tokens * topk, H, F)}.items():
        a = torch.randn(m, k, generator=g, device="cuda").to(torch.bfloat16)
        b = (torch.randn(n, k, generator=g, device="cuda") * 0.02).to(torch.bfloat16)
        for _ in range(3):
            c = a @ b.t()
        torch.cuda.synchronize()
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        for e0, e1 in ev:
            e0.record()
            c = a @ b.t()
            e1.record()
        torch.cuda.synchronize()
        t = sorted(e0.elapsed_time(e1) for e0, e1 in ev)[len(ev) // 2] * 1e-3
        rows.append({"gemm": name, "m": m, "n": n, "k": k, "us": round(t * 1e6, 1), "tflops": round(2.0 * m * n * k / t / 1e12, 1)})
        del a, b, c
    return {"metric": "vendor_dense_gemm_bf16", "unit": "TFLOP/s", "tokens": tokens, "rows": rows}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--tokens", type=int, default=4096, help="headline token count")
    ap.add_argument("--shape", default="mixtral", choices=sorted(SHAPES))
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp8"], help="fp8: e4m3 weights + dynamic per-token activations")
    ap.add_argument("--seed", type=int, default=1337)
    ap.add_argument("--no-sweep", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-configs", action="store_true", help="skip the small / routing / fine-grained / fp8 records")
    ap.add_argument("--cpu-tokens", type=int, default=4096)
    ap.add_argument("--routing", action="store_true", help="also time the routing-only stress workload")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain 1 GiB device copy: the kernel of known size that calibrates "
                         "FETCH_SIZE / WRITE_SIZE when this command runs under rocprofv3 --pmc")
    # the reference's flag names (benchmarks/fused_route/moe_bench.py:10-38)
    ap.add_argument("-n", type=int, default=8192, help="reference protocol: intermediate (ffn) size")
    ap.add_argument("-k", type=int, default=4096, help="reference protocol: hidden size")
    ap.add_argument("-e", type=int, default=16, help="reference protocol: experts")
    ap.add_argument("--topk", type=int, default=2, help="reference protocol: experts per token")
    ap.add_argument("--mfma-stream", action="store_true",
                    help="only run the pure MFMA stream (fr_probe_mfma_stream): sustained rate and shader clock per MFMA shape")
    ap.add_argument("--vendor-gemm", action="store_true",
                    help="only time torch.matmul on the layer's two GEMM shapes at --tokens (dense, no gather): the vendor kernel's rate")
    ap.add_argument("--prepared", default="", choices=["", "w1", "w2", "both"],
                    help="run the workloads with weights re-laid-out by prepare_weights (the w2 default of that call, or both)")
    ap.add_argument("--reference-protocol", action="store_true",
                    help="run the reference's sweep (fp16 randn/10, m = 2^0..2^14 at -n -k -e --topk) instead of the workloads")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build is single-GPU (one MI355X runs the whole layer); --gpus must be 1")

    import torch
    from fast_route_amd import _native as N
    N.lib()
    assert torch.cuda.is_available(), "bench.py needs an MI355X"
    torch.cuda.set_device(0)
    if args.mfma_stream:
        print(json.dumps(mfma_stream(torch, N)))
        return
    if args.vendor_gemm:
        print(json.dumps(vendor_gemm(torch, args.tokens, SHAPES[args.shape], args.steps)))
        return
    if args.reference_protocol:
        print(json.dumps({"metric": "reference_protocol_moe_bench", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
                          "dtype": "f16", "data": "synthetic", **reference_protocol(torch, N, args)}))
        return
    shape = SHAPES[args.shape]
    H, F, E, topk = shape["H"], shape["F"], shape["E"], shape["topk"]
    w1, w2 = make_weights(torch, shape, args.seed)

    fp8 = None
    sweep_ms = shape["sweep"]
    flush = 3 * E * F * H * 2 <= (512 << 20)  # weights that could stay in the Infinity Cache between repetitions
    if args.dtype == "fp8":
        from fast_route_amd import prepare_weights_fp8
        fp8 = prepare_weights_fp8(w1, w2)
        sweep_ms = [16, 256, 1024, 4096] if args.shape == "mixtral" else shape["sweep"]
    prepared = 0
    if args.prepared and fp8 is None:
        from fast_route_amd import prepare_weights
        w1, w2, prepared = prepare_weights(w1, w2, args.prepared)
    # Every point - the headline included - is W warm-up passes and then K timed passes of its own.  The points are
    # taken in the sweep's order (ascending token counts), the headline at its place among them: a process's first
    # launches run on a device whose clocks have not settled yet (a point measured first reads 2-7 % slower than the
    # same point measured later in the same process).  Without the sweep the headline is the only point.
    head = layer = None
    sweep = []
    if not args.no_sweep:
        for M in sweep_ms:
            rec, lay = measure(torch, N, shape, M, w1, w2, args.steps, args.warmup, args.seed, fp8, flush=flush, prepared=prepared)
            sweep.append(rec)
            if M == args.tokens:
                head, layer = rec, lay
            del lay
    if head is None:
        head, layer = measure(torch, N, shape, args.tokens, w1, w2, args.steps, args.warmup, args.seed, fp8, flush=flush, prepared=prepared)
    result = {
        "metric": "moe_layer_tflops_%s_%s_M%d" % (args.shape, args.dtype, args.tokens),
        "value": head["tflops"], "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(head["us_per_layer"] / 1e3, 4), "us_per_layer": head["us_per_layer"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": "%s-shape MoE layer: H=%d F=%d E=%d top-%d, M=%d tokens, %s in / fp32 accumulate"
                               % (args.shape, H, F, E, topk, args.tokens, args.dtype),
                   "tokens": args.tokens, "hidden": H, "ffn": F, "experts": E, "topk": topk, "seed": args.seed,
                   "flops_formula": "6*M*topk*H*F"},
        "native_library": os.path.basename(N.LIB_PATH), "weights_prepared": args.prepared or "no",
        "tunables": tunables_now(N),
        "layer_roofline_frac": head["roofline_frac"], "layer_bound": head["bound"],
        "stage_us": head["stage_us"],
        "roofline": kernel_roofline(shape, head, fp8 is not None),
        "sweep": sweep,
    }
    result["roofline"]["traffic"] = recorded_traffic(result["metric"], head["block"])
    if args.copy_probe:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.mul(src, 1.0, out=dst)  # an elementwise kernel (copy_ would take the DMA engine)
        torch.cuda.synchronize()
        result["copy_probe"] = {"kernel": "torch.mul(src, 1.0, out=dst), fp32", "bytes_read": src.numel() * 4, "bytes_written": dst.numel() * 4, "launches": 3}
    if args.routing:
        result["routing_stress"] = routing_bench(torch, N, args.steps, args.warmup, args.seed)
    if not args.no_cpu and fp8 is None:
        result["cpu_baseline"] = cpu_baseline(torch, shape, layer, args.cpu_tokens)
    default_run = args.shape == "mixtral" and args.dtype == "bf16" and not args.no_sweep
    if default_run and not args.no_configs:
        del layer
        result["configs"] = other_configs(torch, N, args, (w1, w2))
        rp_args = argparse.Namespace(**{**vars(args), "no_sweep": True, "tokens": 4096})
        result["reference_protocol_row"] = reference_protocol(torch, N, rp_args)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
