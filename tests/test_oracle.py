"""Pins the CPU oracle: reference known answers, brute force, closed forms.

None of these tests restate the oracle's own formula; each one is chosen so a
plausible mistake (wrong tie direction, dropped padding, transposed weight,
swapped gate/up halves) fails it.
"""
import json
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _kat():
    with open(os.path.join(GOLDEN, "reference_known_answers.json")) as f:
        return json.load(f)


# ------------------------------------------------------------------ argsort
def test_argsort_demo_matrix_from_reference():
    k = _kat()["argsort_demo"]
    x = torch.tensor(k["x"], dtype=torch.float16)
    _, ids = oracle.stable_sort_rows(x, descending=False)
    assert ids.tolist() == k["ids_ascending"]
    _, ids = oracle.stable_sort_rows(x, descending=True)
    assert ids.tolist() == k["ids_descending"]


def _insertion_argsort(row, descending):
    """Brute force: insertion sort moves an element only past strictly
    worse ones, hence stable."""
    idx = []
    for j, v in enumerate(row):
        p = len(idx)
        while p > 0 and ((row[idx[p - 1]] < v) if descending else (row[idx[p - 1]] > v)):
            p -= 1
        idx.insert(p, j)
    return idx


@pytest.mark.parametrize("k", [4, 8, 16, 64])
@pytest.mark.parametrize("descending", [False, True])
def test_stable_sort_vs_insertion_sort(k, descending):
    g = torch.Generator().manual_seed(k)
    # few distinct values -> many ties
    x = torch.randint(0, 5, (32, k), generator=g).float()
    _, ids = oracle.stable_sort_rows(x, descending)
    for r in range(x.shape[0]):
        assert ids[r].tolist() == _insertion_argsort(x[r].tolist(), descending)


# ------------------------------------------------------------------- gating
def test_gating_special_cases():
    # E == k: everything selected, renormalised weights == full softmax in sorted order
    l = torch.tensor([[0.5, 2.0, -1.0, 2.0]])
    w, ids = oracle.gating_topk(l, 4, True)
    assert ids.tolist() == [[1, 3, 0, 2]]
    torch.testing.assert_close(w, torch.softmax(l, -1)[:, [1, 3, 0, 2]])
    # all-equal logits: ids 0..k-1, uniform weights
    w, ids = oracle.gating_topk(torch.zeros(3, 8), 2, True)
    assert ids.tolist() == [[0, 1]] * 3
    torch.testing.assert_close(w, torch.full((3, 2), 0.5))
    w, _ = oracle.gating_topk(torch.zeros(3, 8), 2, False)
    torch.testing.assert_close(w, torch.full((3, 2), 0.125))
    # one-hot-ish logits: winner takes ~all of the renormalised weight
    l = torch.full((1, 8), -30.0)
    l[0, 5] = 30.0
    w, ids = oracle.gating_topk(l, 2, True)
    assert ids.tolist() == [[5, 0]]
    assert w[0, 0].item() == pytest.approx(1.0) and w[0, 1].item() == pytest.approx(0.0, abs=1e-20)


@pytest.mark.parametrize("E,k", [(8, 2), (16, 4), (64, 6)])
@pytest.mark.parametrize("renorm", [True, False])
def test_gating_matches_softmax_then_topk(E, k, renorm):
    """Reference test recipe tests/test_route.py:45-65: topk(softmax) renormalised."""
    g = torch.Generator().manual_seed(E * 10 + k)
    l = torch.randn(257, E, generator=g)
    w, ids = oracle.gating_topk(l, k, renorm)
    p = torch.softmax(l, -1)
    rw, rid = torch.topk(p, k)  # no ties in continuous random data
    if renorm:
        rw = rw / rw.sum(-1, keepdim=True)
    assert torch.equal(ids.long(), rid)
    torch.testing.assert_close(w, rw, atol=1e-6, rtol=1e-5)
    w2, ids2 = oracle.gating_topk_softmax_first(l, k, renorm)
    assert torch.equal(ids, ids2)
    torch.testing.assert_close(w, w2, atol=1e-6, rtol=1e-5)
    if renorm:
        torch.testing.assert_close(w.sum(-1), torch.ones(257))


def test_gating_tie_break_prefers_lower_index():
    l = torch.tensor([[1.0, 3.0, 3.0, 0.0, 3.0, 1.0, 1.0, -2.0]]).to(torch.bfloat16)
    _, ids = oracle.gating_topk(l, 4, True)
    assert ids.tolist() == [[1, 2, 4, 0]]


def test_route_from_gate_is_matmul_then_gating():
    g = torch.Generator().manual_seed(3)
    h = (torch.randn(16, 64, generator=g) / 10).half()
    gate = (torch.randn(64, 8, generator=g) / 10).half()
    w, ids = oracle.route_from_gate(h, gate, 2)
    logits = torch.einsum("mk,ke->me", h.double(), gate.double()).float()
    w2, ids2 = oracle.gating_topk(logits, 2)
    assert torch.equal(ids, ids2)
    torch.testing.assert_close(w, w2, atol=1e-6, rtol=1e-5)


# ------------------------------------------------------------------ routing
def test_align_docstring_known_answer():
    k = _kat()["align_docstring"]
    s, e, n = oracle.moe_align_block_size(np.array(k["topk_ids"]), k["block_size"], k["num_experts"])
    npost = k["num_tokens_post_pad"]
    assert n.tolist() == [npost]
    assert s[:npost].tolist() == k["sorted_token_ids_prefix"]
    assert e[: npost // k["block_size"]].tolist() == k["expert_ids_prefix"]
    assert s.shape[0] == 12 + 5 * 3 and e.shape[0] == 12 + 5
    assert (s[npost:] == 12).all()


def _align_bruteforce(flat, B, E):
    n = len(flat)
    out, eids = [], []
    for e in range(E):
        run = [p for p in range(n) if flat[p] == e]
        while len(run) % B:
            run.append(n)
        out += run
        eids += [e] * (len(run) // B)
    return out, eids


@pytest.mark.parametrize("E,k,B", [(8, 2, 16), (64, 6, 32), (5, 3, 4), (16, 1, 128), (3, 2, 1)])
@pytest.mark.parametrize("M", [0, 1, 7, 200])
def test_align_vs_bruteforce(E, k, B, M):
    rng = np.random.default_rng(E * 1000 + k * 10 + M)
    ids = rng.integers(0, E, size=(M, k))
    if M > 3:
        ids[ids == E - 1] = 0  # guarantee an empty expert
    s, e, n = oracle.moe_align_block_size(ids, B, E)
    bs, be = _align_bruteforce(ids.reshape(-1).tolist(), B, E)
    assert n[0] == len(bs)
    assert s[: n[0]].tolist() == bs
    assert e[: n[0] // B].tolist() == be
    assert (s[n[0]:] == M * k).all()
    assert s.shape[0] == M * k + E * (B - 1) and e.shape[0] == M * k + E


def test_align_invariants_zipf():
    l = oracle.zipf_logits(4096, 64, seed=11)
    _, ids = oracle.gating_topk(l, 6)
    n = ids.numel()
    for B in (16, 32, 64, 128):
        s, e, npost = oracle.moe_align_block_size(ids, B, 64)
        npost = int(npost[0])
        assert npost % B == 0 and npost <= n + 64 * (B - 1)
        real = s[:npost][s[:npost] < n]
        assert np.array_equal(np.sort(real), np.arange(n))  # a permutation of all pairs
        flat = ids.reshape(-1).numpy()
        blocks = s[:npost].reshape(-1, B)
        for b in range(blocks.shape[0]):
            r = blocks[b][blocks[b] < n]
            assert r.size > 0  # no all-padding block
            assert (flat[r] == e[b]).all()  # single-expert block
            assert (np.diff(r) > 0).all()  # flat order kept inside an expert
        assert (np.diff(e[: npost // B]) >= 0).all()


# --------------------------------------------------------------- expert MLPs
def test_silu_and_mul_halves():
    x = torch.tensor([[1.0, -2.0, 3.0, 0.5]])
    got = oracle.silu_and_mul(x)
    exp = torch.tensor([[1.0 / (1 + np.exp(-1.0)) * 3.0, -2.0 / (1 + np.exp(2.0)) * 0.5]])
    torch.testing.assert_close(got, exp.float())


def test_moe_experts_vs_per_pair_loops():
    g = torch.Generator().manual_seed(5)
    M, H, Fd, E, k = 6, 16, 8, 4, 2
    x = torch.randn(M, H, generator=g)
    w1 = torch.randn(E, 2 * Fd, H, generator=g) * 0.3
    w2 = torch.randn(E, H, Fd, generator=g) * 0.3
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(M)]).int()
    wts = torch.rand(M, k, generator=g)
    got = oracle.moe_experts(x, w1, w2, wts, ids)
    exp = torch.zeros(M, H, dtype=torch.float64)
    for m in range(M):
        for j in range(k):
            e = int(ids[m, j])
            for h in range(H):
                acc = 0.0
                for f in range(Fd):
                    gte = sum(float(w1[e, f, c]) * float(x[m, c]) for c in range(H))
                    up = sum(float(w1[e, Fd + f, c]) * float(x[m, c]) for c in range(H))
                    acc += float(w2[e, h, f]) * (gte / (1.0 + np.exp(-gte)) * up)
                exp[m, h] += float(wts[m, j]) * acc
    torch.testing.assert_close(got.double(), exp, atol=1e-5, rtol=1e-5)


def test_moe_single_expert_is_swiglu_mlp():
    g = torch.Generator().manual_seed(6)
    x = torch.randn(9, 32, generator=g)
    w1 = torch.randn(1, 48, 32, generator=g) * 0.2
    w2 = torch.randn(1, 32, 24, generator=g) * 0.2
    out = oracle.moe_experts(x, w1, w2, torch.ones(9, 1), torch.zeros(9, 1, dtype=torch.int32))
    gate, up = F.linear(x, w1[0, :24]), F.linear(x, w1[0, 24:])
    torch.testing.assert_close(out, F.linear(F.silu(gate) * up, w2[0]), atol=1e-5, rtol=1e-5)


def test_moe_linear_in_routing_weights_and_grouped_gemm_consistency():
    g = torch.Generator().manual_seed(7)
    x, logits, w1, w2 = oracle.make_inputs(12, 32, 16, 4, seed=7, w_std=0.2)
    wts, ids = oracle.gating_topk(logits, 2)
    a = oracle.moe_experts(x, w1, w2, wts, ids)
    b = oracle.moe_experts(x, w1, w2, 3.0 * wts, ids)
    torch.testing.assert_close(b, 3.0 * a, atol=1e-5, rtol=1e-5)
    # the two op-level grouped GEMMs chained by hand give the layer
    c1 = oracle.grouped_gemm(x, w1, wts, ids, False, 2)
    c2 = oracle.silu_and_mul(c1)
    c3 = oracle.grouped_gemm(c2, w2, wts, ids, True, 1)
    torch.testing.assert_close(c3.view(12, 2, 32).sum(1), a, atol=1e-5, rtol=1e-5)
    full = oracle.fused_moe(x, w1, w2, logits, 2)
    torch.testing.assert_close(full, a)


# ---------------------------------------------------------------------- fp8
def test_e4m3_table_and_roundtrip():
    t = oracle.e4m3fn_decode_table()
    assert t[0x7E] == 448.0 and t[0x01] == 2.0 ** -9 and t[0x08] == 2.0 ** -6 and t[0x38] == 1.0
    assert np.isnan(t[0x7F]) and np.isnan(t[0xFF])
    finite = np.array([c for c in range(256) if c & 0x7F != 0x7F], dtype=np.uint8)
    assert np.array_equal(oracle.e4m3fn_encode(t[finite]), finite)
    tt = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.nan_to_num(t, nan=-7.0), np.nan_to_num(tt, nan=-7.0))


def test_e4m3_encode_known_values_and_torch_cast():
    enc = oracle.e4m3fn_encode
    assert enc(np.float32([448.0, 1e6, -1e6, 0.0])).tolist() == [0x7E, 0x7E, 0xFE, 0x00]
    # ties to even: 1.0625 is halfway between 1.0 (0x38) and 1.125 (0x39) -> even mantissa 0x38
    assert enc(np.float32([1.0625, 1.1875])).tolist() == [0x38, 0x3A]
    # subnormal halfway 2**-10 -> 0 (even), 3*2**-10 -> 2*2**-9
    assert enc(np.float32([2.0 ** -10, 3 * 2.0 ** -10])).tolist() == [0x00, 0x02]
    # carry into the next binade: 1.96 -> 2.0
    assert enc(np.float32([1.96])).tolist() == [0x40]
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.normal(0, 1, 20000), rng.normal(0, 100, 20000), rng.normal(0, 1e-2, 20000)]).astype(np.float32)
    x = np.clip(x, -448, 448)
    got = enc(x)
    ref = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    zero = (got & 0x7F) == 0  # sign of zero is irrelevant
    assert np.array_equal(got[~zero], ref[~zero]) and ((ref[zero] & 0x7F) == 0).all()


def test_quant_rows_and_fp8_layer_close_to_fp32():
    x, logits, w1, w2 = oracle.make_inputs(16, 64, 32, 4, seed=9, w_std=0.1)
    c, s = oracle.quant_e4m3_rows(x)
    t = oracle.e4m3fn_decode_table()
    deq = t[c] * s[:, None]
    assert np.abs(deq - x.numpy()).max() <= np.abs(x.numpy()).max() * 2.0 ** -4
    assert (np.abs(t[c]).max(axis=1) == 448.0).all()
    out8, _ = oracle.fused_moe_fp8(x, w1, w2, logits, 2)
    out32 = oracle.fused_moe(x, w1, w2, logits, 2)
    rel = (out8 - out32).norm() / out32.norm()
    assert rel < 0.08


def test_reciprocal_fma_quotient_is_correctly_rounded():
    """The fp8 row quantisation divides by the row scale with y = RN(1/s), q = RN(x*y),
    r = RN(x - s*q) (one FMA), RN(q + r*y) (another) for rows whose max|x| lies in [2^-40, 2^40].
    Exact rational arithmetic: for bf16/fp16 values x with |x| >= 2^-70 (smaller ones encode as
    zero whatever their last bit) the result is the correctly rounded fp32 quotient x/s."""
    from fractions import Fraction as F
    rng = np.random.default_rng(5)

    def rn32(fr):
        c = np.float32(float(fr))
        best = None
        for cand in (np.nextafter(c, np.float32(-np.inf)), c, np.nextafter(c, np.float32(np.inf))):
            key = (abs(F(float(cand)) - fr), int(np.float32(cand).view(np.uint32)) & 1)
            if best is None or key < best[0]:
                best = (key, np.float32(cand))
        return best[1]

    def grid(n, kind):
        if kind == "bf16":
            v = (rng.integers(0, 1 << 16, n, dtype=np.uint32) << 16).view(np.float32)
        else:
            v = rng.integers(0, 1 << 16, n, dtype=np.uint16).view(np.float16).astype(np.float32)
        return v[np.isfinite(v)]

    checked = 0
    for kind in ("bf16", "f16"):
        xs = grid(60000, kind)
        xs = xs[np.abs(xs) >= 2.0 ** -70]
        am = np.abs(grid(60000, kind))
        am = am[(am >= 2.0 ** -40) & (am <= 2.0 ** 40)]
        for x, a in list(zip(xs, am))[:6000]:
            if abs(x) > a:
                x, a = np.float32(np.copysign(a, x)), np.float32(abs(x))
                if not (2.0 ** -40 <= a <= 2.0 ** 40):
                    continue
            s = rn32(F(float(a)) / 448)
            y = rn32(1 / F(float(s)))
            q = rn32(F(float(x)) * F(float(y)))
            r = rn32(F(float(x)) - F(float(s)) * F(float(q)))
            got = rn32(F(float(q)) + F(float(r)) * F(float(y)))
            assert got.view(np.uint32) == rn32(F(float(x)) / F(float(s))).view(np.uint32), (kind, x, a)
            checked += 1
    assert checked > 8000


def test_fp8_layer_oracle_against_independent_per_pair_loop():
    """oracle.fused_moe_fp8 restated pair by pair on torch.float8_e4m3fn casts and torch.topk:
    scale per ROW (weight output channel, token, activated row), bf16 rounding of the activated
    row before it is quantised again, routed weight after the down projection.  A per-tensor scale,
    a skipped bf16 rounding or a skipped re-quantisation each move the result by far more than the
    fp32 summation-order difference allowed here."""
    def q(t):  # per-row e4m3 quantise + dequantise with fp32 scale amax/448
        amax = t.abs().amax(dim=-1, keepdim=True)
        s = torch.where(amax > 0, amax / 448.0, torch.ones_like(amax))
        return (t / s).to(torch.float8_e4m3fn).float() * s

    def layer(x, logits, w1, w2, k, mistake=None):
        M, H = x.shape
        E, F2, _ = w1.shape
        Fd = F2 // 2
        if mistake == "per_tensor_scale":
            s1, s2 = w1.abs().max() / 448.0, w2.abs().max() / 448.0
            w1q, w2q = (w1 / s1).to(torch.float8_e4m3fn).float() * s1, (w2 / s2).to(torch.float8_e4m3fn).float() * s2
        else:
            w1q, w2q = q(w1.reshape(E * F2, H)).reshape(E, F2, H), q(w2.reshape(E * H, Fd)).reshape(E, H, Fd)
        xq = q(x)
        pw, pid = torch.topk(torch.softmax(logits.float(), -1), k)  # no ties in these random logits
        pw = pw / pw.sum(-1, keepdim=True)
        want = torch.zeros(M, H)
        for m in range(M):
            for j in range(k):
                e = int(pid[m, j])
                h = w1q[e] @ xq[m]
                a = torch.nn.functional.silu(h[:Fd]) * h[Fd:]
                if mistake != "no_bf16_rounding":
                    a = a.bfloat16().float()
                if mistake != "no_requantisation":
                    a = q(a[None, :])[0]
                want[m] += float(pw[m, j]) * (w2q[e] @ a)
        return want

    for seed, (M, H, Fd, E, k) in enumerate([(7, 32, 16, 4, 2), (5, 64, 32, 3, 3), (9, 16, 48, 8, 1)]):
        x, logits, w1, w2 = oracle.make_inputs(M, H, Fd, E, seed=40 + seed, w_std=0.1)
        x, w1, w2 = x.bfloat16().float(), w1.bfloat16().float(), w2.bfloat16().float()
        got, _ = oracle.fused_moe_fp8(x, w1, w2, logits, k, True)
        want = layer(x, logits, w1, w2, k)
        tol = 1e-5 * want.abs().max()
        assert (got - want).abs().max() <= tol, (got - want).abs().max()
        for mistake in ("per_tensor_scale", "no_bf16_rounding", "no_requantisation"):
            assert (got - layer(x, logits, w1, w2, k, mistake)).abs().max() > 20 * tol, mistake


def test_tile_weights_is_the_stated_permutation():
    """oracle.tile_weights against the layout's definition, element by element: element (e, row, k) lands at flat
    offset ((row // 64) * ktiles + k // el) * 64 * el + (row % 64) * el + k % el of expert e."""
    import oracle
    torch.manual_seed(5)
    for dtype, el in ((torch.bfloat16, 64), (torch.uint8, 128)):
        E, rows, K = 2, 128, 2 * el
        w = torch.arange(E * rows * K, dtype=torch.int32).reshape(E, rows, K) % 251
        w = w.to(dtype)
        t = oracle.tile_weights(w).reshape(E, -1)
        ktiles = K // el
        for e in range(E):
            for row in (0, 1, 63, 64, 65, 127):
                for k in (0, 1, el - 1, el, K - 1):
                    off = ((row // 64) * ktiles + k // el) * 64 * el + (row % 64) * el + k % el
                    assert t[e, off] == w[e, row, k], (e, row, k)
        # a permutation: nothing lost, nothing duplicated
        assert torch.equal(torch.sort(t.flatten().int())[0], torch.sort(w.flatten().int())[0])
