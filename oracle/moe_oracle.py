"""CPU restatement of the reference's fused-MoE hot path.  TEST INFRASTRUCTURE ONLY.

Every function states the reference lines it follows.  The reference itself
(hgl71964/fast-route) cannot be imported here: its hot-path modules import the
compiled CUDA extensions of vllm==0.4.0.post1 at module top
(fast_route/fast_route/ops/fused_moe.py:6-7) and Triton-3.0 internals
(fast_route/fast_route/ops/stable_argsort.py:5-7).  The third-party arithmetic
(vLLM's moe_align_block_size / silu_and_mul / topk_softmax) is restated from
the reference's own call sites, docstrings and tests.

How each function is pinned (tests/test_oracle_*.py):
  stable_sort_rows        4x4 tie demo of ops/stable_argsort.py:154-159; brute
                          force insertion sort; torch.sort(stable=True).
  gating_topk             equals stable sort + softmax identities; closed forms
                          (E == k, all-equal logits, one-hot logits); agreement
                          of the two orderings (logit / probability).
  moe_align_block_size    docstring known answer ops/fused_moe.py:152-157;
                          brute-force python loop; permutation / monotonicity /
                          single-expert-block invariants.
  silu_and_mul            torch.nn.functional.silu on split halves
                          (benchmarks/fused_route/activation.py:27-30).
  moe_experts             per-(token, slot) brute-force loop on tiny inputs;
                          E=1,k=1,w=1 reduces to a plain SwiGLU MLP; linearity
                          in the routing weights.
  e4m3fn_encode           all 256 codes round-trip; torch.float8_e4m3fn casts;
                          known values (448 saturation, 2**-9 subnormal, ties).
  fused_moe_fp8           parity unpinned by the reference (it has no fp8 path);
                          defined by dequantise -> fp32 oracle.
"""
from __future__ import annotations

import math

import os

import numpy as np
import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------
# gating
# --------------------------------------------------------------------------
def stable_sort_rows(x: torch.Tensor, descending: bool = True):
    """Row-wise stable sort: ties keep the lower column index first, for both
    directions.  Follows the total order of ops/stable_argsort.py:37-50 as
    checked by tests/test_argsort.py:134-145 against torch.sort(stable=True).
    Returns (values, int32 ids)."""
    v, i = torch.sort(x, dim=1, descending=descending, stable=True)
    return v, i.to(torch.int32)


def gating_topk(logits: torch.Tensor, topk: int, renormalize: bool = True):
    """Top-k gating as the reference's fused routing kernel orders it
    (ops/stable_route.py:97-107): stable descending sort of the fp32 LOGITS,
    first `topk` columns, then softmax.  With renormalize the softmax runs over
    the selected logits only (== selected softmax probabilities divided by
    their sum, layers/vllm_route.py:86-87); without it the weights are the
    selected entries of the full softmax.

    Returns (weights fp32 [M, topk], ids int32 [M, topk])."""
    l = logits.detach().to(torch.float32).cpu()
    assert l.dim() == 2 and 1 <= topk <= l.shape[1]
    sv, si = stable_sort_rows(l, descending=True)
    top_v, ids = sv[:, :topk], si[:, :topk].contiguous()
    row_max = sv[:, :1]  # sorted descending: column 0 is the row maximum
    if renormalize:
        ex = torch.exp(top_v - row_max)
        w = ex / ex.sum(dim=1, keepdim=True)
    else:
        w = torch.exp(top_v - row_max) / torch.exp(l - row_max).sum(dim=1, keepdim=True)
    return w.contiguous(), ids


def gating_topk_softmax_first(logits: torch.Tensor, topk: int, renormalize: bool = True):
    """The baseline layer's order of operations (layers/vllm_route.py:78-87 and
    tests/test_route.py:45-65): full fp32 softmax, then stable descending sort
    of the PROBABILITIES, then optional division by the selected sum.  Differs
    from gating_topk only when two distinct logits round to one probability."""
    p = torch.softmax(logits.detach().to(torch.float32).cpu(), dim=-1)
    sv, si = stable_sort_rows(p, descending=True)
    w, ids = sv[:, :topk], si[:, :topk].contiguous()
    if renormalize:
        w = w / w.sum(dim=-1, keepdim=True)
    return w.contiguous(), ids


def route_from_gate(hidden: torch.Tensor, gate: torch.Tensor, topk: int, renormalize: bool = True):
    """Gate-matrix form of the routing op (ops/stable_route.py:123-178):
    logits = hidden @ gate with fp32 accumulation of the half-precision inputs
    (`:66-86`), then gating_topk."""
    logits = hidden.detach().to(torch.float32).cpu() @ gate.detach().to(torch.float32).cpu()
    return gating_topk(logits, topk, renormalize)


# --------------------------------------------------------------------------
# routing arrays
# --------------------------------------------------------------------------
def moe_align_block_size(topk_ids, block_size: int, num_experts: int):
    """Closed form of the block-aligned counting sort the reference obtains from
    vLLM (wrapper ops/fused_moe.py:133-175: output lengths `:161-167`, fill
    value numel `:168`, worked example `:151-159`).

    Flat pair index p = token * topk + slot.  Pairs are stably sorted by expert;
    each expert's run is padded to a multiple of block_size with the value n.

    Returns numpy int32 arrays (sorted_token_ids[n + E*(B-1)], expert_ids of
    length n + E with only the first npost/B entries defined (the rest are set
    to -1 here; the reference leaves them uninitialised), num_tokens_post_pad[1]).
    """
    flat = np.asarray(topk_ids.detach().cpu().numpy() if isinstance(topk_ids, torch.Tensor) else topk_ids)
    flat = flat.reshape(-1).astype(np.int64)
    n, E, B = flat.size, int(num_experts), int(block_size)
    assert n == 0 or (flat.min() >= 0 and flat.max() < E)
    order = np.argsort(flat, kind="stable")
    cnt = np.bincount(flat, minlength=E)
    padded = (cnt + B - 1) // B * B
    start = np.concatenate(([0], np.cumsum(padded)[:-1]))
    src = np.concatenate(([0], np.cumsum(cnt)[:-1]))
    sorted_ids = np.full(n + E * (B - 1), n, dtype=np.int32)
    for e in range(E):
        sorted_ids[start[e]:start[e] + cnt[e]] = order[src[e]:src[e] + cnt[e]]
    npost = int(padded.sum())
    expert_ids = np.full(n + E, -1, dtype=np.int32)
    expert_ids[:npost // B] = np.repeat(np.arange(E, dtype=np.int32), padded // B)
    return sorted_ids, expert_ids, np.array([npost], dtype=np.int32)


# --------------------------------------------------------------------------
# expert MLPs
# --------------------------------------------------------------------------
def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """x[..., :d] is the gate projection, x[..., d:] the up projection
    (benchmarks/fused_route/activation.py:27-30)."""
    d = x.shape[-1] // 2
    return F.silu(x[..., :d]) * x[..., d:]


def grouped_gemm(A, B, topk_weights, topk_ids, mul_routed_weight: bool, top_k: int):
    """One grouped GEMM of the reference (ops/fused_moe.py:10-130 as launched by
    `:178-214`): for every flat pair p, C[p] = A[p // top_k] @ B[expert(p)].T in
    fp32, optionally times topk_weights.flat[p] (`:117-121`).  Returns fp32
    [n, N]; the caller views it as [M, topk, N]."""
    ids = topk_ids.detach().cpu().reshape(-1).long()
    Af, Bf = A.detach().cpu().float(), B.detach().cpu()
    n = ids.numel()
    C = torch.zeros(n, B.shape[1], dtype=torch.float32)
    rows = torch.arange(n) // top_k
    for e in range(B.shape[0]):
        sel = (ids == e).nonzero(as_tuple=True)[0]
        if sel.numel():
            C[sel] = Af[rows[sel]] @ Bf[e].float().T
    if mul_routed_weight:
        C = C * topk_weights.detach().cpu().float().reshape(-1, 1)
    return C


def moe_experts(x, w1, w2, topk_weights, topk_ids, act_dtype=None):
    """The PyTorch reference MoE (benchmarks/swizzle_moe/perf_test_moe.py:17-31)
    evaluated in fp32: out[m] = sum_j w[m,j] * W2[e] @ silu_and_mul(W1[e] @ x[m]),
    e = ids[m,j].  `act_dtype` optionally rounds the activated intermediate the
    way a kernel that stores it in half precision does (the reference stores it
    in the input dtype, layers/stable_route.py:75-77); None keeps pure fp32."""
    xf = x.detach().cpu().float()
    ids = topk_ids.detach().cpu().long()
    wts = topk_weights.detach().cpu().float()
    M, H = xf.shape
    E, F2, _ = w1.shape
    assert w2.shape[0] == E and w2.shape[1] == H and w2.shape[2] * 2 == F2
    out = torch.zeros(M, H, dtype=torch.float32)
    for e in range(E):
        tok, slot = (ids == e).nonzero(as_tuple=True)
        if tok.numel() == 0:
            continue
        h = xf[tok] @ w1[e].detach().cpu().float().T
        a = silu_and_mul(h)
        if act_dtype is not None:
            a = a.to(act_dtype).float()
        y = a @ w2[e].detach().cpu().float().T
        out.index_add_(0, tok, y * wts[tok, slot].unsqueeze(1))
    return out


def fused_moe(hidden_states, w1, w2, gating_output, topk: int, renormalize: bool = True,
              act_dtype=None):
    """Whole layer in the router-logits form: gating_topk -> moe_experts
    (layers/stable_route.py:10-102 with the routing taken from logits)."""
    w, ids = gating_topk(gating_output, topk, renormalize)
    return moe_experts(hidden_states, w1, w2, w, ids, act_dtype=act_dtype)


# --------------------------------------------------------------------------
# fp8 (OCP e4m3fn) -- no counterpart in the reference; parity unpinned there
# --------------------------------------------------------------------------
def e4m3fn_decode_table() -> np.ndarray:
    """float32 value of each of the 256 e4m3fn codes (bias 7, no infinities,
    S.1111.111 is NaN, largest finite 448)."""
    out = np.empty(256, dtype=np.float32)
    for c in range(256):
        s = -1.0 if c & 0x80 else 1.0
        e, m = (c >> 3) & 0xF, c & 7
        if e == 0xF and m == 7:
            out[c] = np.nan
        elif e == 0:
            out[c] = s * m * 2.0 ** -9
        else:
            out[c] = s * (1.0 + m / 8.0) * 2.0 ** (e - 7)
    return out


def _e4m3fn_encode_block(x: np.ndarray) -> np.ndarray:
    sign = (np.signbit(x)).astype(np.uint8) << 7
    a = np.minimum(np.abs(x), np.float32(448.0))  # float32 throughout: every scaling below is by a power of two, hence exact
    # exponent of the quantisation step: normal numbers have 3 mantissa bits,
    # everything below 2**-6 shares the subnormal step 2**-9.  frexp: a = m * 2**e, m in [0.5, 1).
    _, e = np.frexp(a)
    ex = np.maximum(e - 1, -6)
    q = np.rint(np.ldexp(a, 3 - ex))  # numpy rint is round-half-even
    val = np.ldexp(q, ex - 3)  # may carry into the next binade; re-derive fields from val
    _, e2 = np.frexp(val)
    ev = np.maximum(e2 - 1, -6)
    is_sub = val < np.float32(2.0 ** -6)
    mant = np.where(is_sub, np.ldexp(val, 9), (np.ldexp(val, -ev) - np.float32(1.0)) * np.float32(8.0))
    expo = np.where(is_sub, 0, ev + 7)
    code = (expo.astype(np.int32) << 3) | np.rint(mant).astype(np.int32)
    return (code.astype(np.uint8) | sign).astype(np.uint8)


def e4m3fn_encode(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even fp32 -> e4m3fn code (uint8), saturating at +-448.
    Large inputs go through in blocks of rows to bound the temporaries."""
    x = np.asarray(x, dtype=np.float32)
    if x.ndim < 2 or x.size <= (1 << 24):
        return _e4m3fn_encode_block(x)
    out = np.empty(x.shape, dtype=np.uint8)
    rows = max(1, (1 << 22) // max(1, x[0].size))

    def one(r0):
        out[r0:r0 + rows] = _e4m3fn_encode_block(x[r0:r0 + rows])

    from concurrent.futures import ThreadPoolExecutor
    with ThreadPoolExecutor(max_workers=min(16, os.cpu_count() or 1)) as pool:  # numpy releases the GIL inside its loops
        list(pool.map(one, range(0, x.shape[0], rows)))
    return out


def quant_e4m3_rows(x: torch.Tensor):
    """Per-row dynamic quantisation: scale = amax/448 (1.0 for an all-zero row),
    code = e4m3fn(x / scale).  Returns (uint8 codes, fp32 scales[rows])."""
    xf = x.detach().cpu().float().numpy()
    amax = np.abs(xf).max(axis=-1).astype(np.float32)
    scale = np.where(amax > 0, amax / np.float32(448.0), np.float32(1.0)).astype(np.float32)
    codes = e4m3fn_encode((xf / scale[..., None]).astype(np.float32))
    return codes, scale


def quantize_weights_fp8(w1, w2):
    """(w1 codes, w1 scales, w2 codes, w2 scales) per (expert, output channel): what the fp8 layer's
    weight preparation produces; fused_moe_fp8 takes it as `weights_q` to quantise large weights once."""
    E, F2, H = w1.shape
    w1c, w1s = quant_e4m3_rows(w1.reshape(E * F2, H))
    w2c, w2s = quant_e4m3_rows(w2.reshape(E * w2.shape[1], w2.shape[2]))
    return w1c, w1s, w2c, w2s


def fused_moe_fp8(hidden_states, w1, w2, gating_output, topk: int, renormalize: bool = True, weights_q=None):
    """fp8 layer as the fp8 Mixtral workload defines it: weights quantised per (expert,
    output channel), activations per token (both before the gate/up GEMM and
    before the down GEMM), everything dequantised to fp32 and run through the
    fp32 oracle.  Returns (out fp32, dict with the quantised operands)."""
    E, F2, H = w1.shape
    w1c, w1s, w2c, w2s = weights_q if weights_q is not None else quantize_weights_fp8(w1, w2)
    tab = e4m3fn_decode_table()
    Hd = w2.shape[1]

    def dequant(codes, scales):  # uint8 codes index the 256-entry table directly
        return torch.from_numpy(tab[codes] * scales[:, None])

    xc, xs = quant_e4m3_rows(hidden_states)
    xd = dequant(xc, xs)
    wts, ids = gating_topk(gating_output, topk, renormalize)
    M, k = ids.shape
    out = torch.zeros(M, H, dtype=torch.float32)
    idl = ids.long()
    for e in range(E):
        tok, slot = (idl == e).nonzero(as_tuple=True)
        if tok.numel() == 0:
            continue
        w1d = dequant(w1c[e * F2:(e + 1) * F2], w1s[e * F2:(e + 1) * F2])  # one expert at a time bounds the memory
        a = silu_and_mul(xd[tok] @ w1d.T).to(torch.bfloat16)  # kernel stores bf16 then requantises
        del w1d
        ac, asc = quant_e4m3_rows(a)
        ad = dequant(ac, asc)
        w2d = dequant(w2c[e * Hd:(e + 1) * Hd], w2s[e * Hd:(e + 1) * Hd])
        out.index_add_(0, tok, (ad @ w2d.T) * wts[tok, slot].unsqueeze(1))
    return out, {"w1_codes": w1c.reshape(E, F2, H), "w1_scale": w1s.reshape(E, F2),
                 "w2_codes": w2c.reshape(w2.shape), "w2_scale": w2s.reshape(E, -1),
                 "x_codes": xc, "x_scale": xs}


# --------------------------------------------------------------------------
# prepared weight layout (no counterpart in the reference, which keeps w1 [E, 2F, H] / w2 [E, H, F]
# row-major: layers/stable_route.py:32-36): a pure permutation of the elements, restated with a reshape
# --------------------------------------------------------------------------
def tile_weights(w: torch.Tensor, rows_per_group: int = 64, tile_bytes: int = 128) -> torch.Tensor:
    """w [E, rows, K] -> same shape holding [E][rows/64][K tiles][64 rows][tile_bytes / itemsize] flat.
    Pinned in tests/test_oracle.py by an element-by-element loop over the definition."""
    E, rows, K = w.shape
    el = tile_bytes // w.element_size()
    assert rows % rows_per_group == 0 and K % el == 0
    t = w.reshape(E, rows // rows_per_group, rows_per_group, K // el, el).permute(0, 1, 3, 2, 4)
    return t.contiguous().reshape(E, rows, K)


# --------------------------------------------------------------------------
# seeded synthetic inputs (shared by tests, smoke and bench)
# --------------------------------------------------------------------------
def zipf_logits(M: int, E: int, seed: int, s: float = 1.2, tau: float = 1.0) -> torch.Tensor:
    """Router logits with heavily imbalanced expert load: a per-expert bias
    ln(r_e**-s / sum r**-s) * tau, r a seeded permutation of 1..E, plus N(0,1)."""
    g = torch.Generator().manual_seed(seed)
    r = (torch.randperm(E, generator=g) + 1).double()
    pz = r.pow(-s)
    bias = (torch.log(pz / pz.sum()) * tau).float()
    return bias[None, :] + torch.randn(M, E, generator=g)


def make_inputs(M: int, H: int, Fdim: int, E: int, seed: int = 1337, zipf: bool = False,
                w_std: float = 0.02):
    """x ~ N(0,1) [M,H]; logits ~ N(0,1) [M,E] (or Zipf-biased); w1 [E,2F,H] and
    w2 [E,H,F] ~ N(0, w_std); drawn on the CPU in fp32 in that order from one
    generator so every consumer sees the same values."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, H, generator=g)
    logits = torch.randn(M, E, generator=g)
    if zipf:
        logits = zipf_logits(M, E, seed + 1)
    w1 = torch.randn(E, 2 * Fdim, H, generator=g) * w_std
    w2 = torch.randn(E, H, Fdim, generator=g) * w_std
    return x, logits, w1, w2
