"""GPU parity: gating kernels vs the CPU oracle.  ids bit-exact, weights to 1e-6."""
import sys

import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu
W_ATOL = 2e-6  # fp32 softmax weights in [0, 1]: a few ulp of expf/divide


def _say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


def _run_gating(logits_dev, topk, renorm):
    from fast_route_amd.ops.stable_route import topk_softmax
    M = logits_dev.shape[0]
    w = torch.empty((M, topk), dtype=torch.float32, device="cuda")
    ids = torch.empty((M, topk), dtype=torch.int32, device="cuda")
    topk_softmax(w, ids, None, logits_dev, renormalize=renorm)
    torch.cuda.synchronize()
    return w.cpu(), ids.cpu()


@pytest.mark.parametrize("E,topk", [(8, 2), (16, 4), (64, 6), (1, 1), (3, 2), (5, 5), (24, 3), (100, 7), (256, 8)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("renorm", [True, False])
def test_gating_parity(native, E, topk, dtype, renorm):
    for M in (1, 63, 1000, 2500):
        _say(f"gating E={E} k={topk} dtype={dtype} renorm={renorm} M={M}")
        g = torch.Generator().manual_seed(E * 131 + topk * 7 + M)
        logits = torch.randn(M, E, generator=g).to(dtype)  # bf16/fp16 rounding creates exact ties
        w, ids = _run_gating(logits.cuda(), topk, renorm)
        rw, rid = oracle.gating_topk(logits, topk, renorm)
        assert torch.equal(ids, rid), "gating ids differ"
        torch.testing.assert_close(w, rw, atol=W_ATOL, rtol=0)


def test_gating_ties_and_special_rows(native):
    _say("gating special rows")
    rows = [
        [0.0] * 8,                                   # all equal -> ids 0..k-1
        [1.0, 3.0, 3.0, 0.0, 3.0, 1.0, 1.0, -2.0],   # three-way tie
        [-30.0, -30.0, -30.0, -30.0, -30.0, 30.0, -30.0, -30.0],
        [5.0, 4.0, 3.0, 2.0, 1.0, 0.0, -1.0, -2.0],
        [-2.0, -1.0, 0.0, 1.0, 2.0, 3.0, 4.0, 5.0],
        [-0.0, 0.0, -0.0, 0.0, -1.0, 0.0, -0.0, -1.0],  # signed zeros are one value: ties by index
    ]
    logits = torch.tensor(rows)
    for k in (1, 2, 4, 8):
        for renorm in (True, False):
            w, ids = _run_gating(logits.cuda(), k, renorm)
            rw, rid = oracle.gating_topk(logits, k, renorm)
            assert torch.equal(ids, rid)
            torch.testing.assert_close(w, rw, atol=W_ATOL, rtol=0)
    w, ids = _run_gating(logits.cuda(), 4, True)
    assert ids[0].tolist() == [0, 1, 2, 3] and ids[1].tolist() == [1, 2, 4, 0]


@pytest.mark.parametrize("E,topk", [(32, 5), (64, 6), (64, 16), (64, 40), (128, 8), (256, 8), (48, 3)])
def test_gating_ties_many_experts(native, E, topk):
    """Rows built from a handful of distinct values, so every round of the selection has
    ties inside a lane, across lanes and across the vectors of a lane; +0 / -0 tie too.
    (topk = 40 exceeds the result slots of the few-lanes-per-token form: fallback path.)"""
    _say(f"gating ties E={E} topk={topk}")
    g = torch.Generator().manual_seed(E * 131 + topk)
    vals = torch.tensor([0.0, -0.0, 1.5, -1.5, 3.0, 0.25])
    logits = vals[torch.randint(0, len(vals), (1300, E), generator=g)]  # long enough for the few-lanes-per-token form
    logits[0] = 0.0
    logits[1] = torch.arange(E, dtype=torch.float32) % 3
    logits[2] = -torch.arange(E, dtype=torch.float32)
    for renorm in (True, False):
        w, ids = _run_gating(logits.cuda(), topk, renorm)
        rw, rid = oracle.gating_topk(logits, topk, renorm)
        assert torch.equal(ids, rid)
        torch.testing.assert_close(w, rw, atol=W_ATOL, rtol=0)
    # a row stride that is not a multiple of 4 takes the one-logit-per-lane path
    wide = torch.zeros(1300, E + 3)
    wide[:, :E] = logits
    w2, ids2 = _run_gating(wide.cuda()[:, :E], topk, True)
    assert torch.equal(ids2, oracle.gating_topk(logits, topk, True)[1])


def test_gating_reference_route_test_recipe(native):
    """tests/test_route.py:12-77 of the reference: weights vs topk(softmax(h@gate)), atol 1e-2."""
    for seed in range(3):
        for m, topk in ((128, 2), (512, 4)):
            _say(f"route recipe seed={seed} m={m} topk={topk}")
            torch.manual_seed(seed)
            h = (torch.randn((m, 4096)) / 10).half()
            gate = (torch.randn((4096, 16)) / 10).half()
            from fast_route_amd.ops.stable_route import fused_route
            tw = torch.empty(m, 16, dtype=torch.float32, device="cuda")
            ti = torch.empty(m, 16, dtype=torch.int32, device="cuda")
            w, ids = fused_route(h.cuda(), gate.cuda(), topk, tw, ti, True)
            torch.cuda.synchronize()
            score = h.float() @ gate.float()
            rw, rid = torch.topk(torch.softmax(score, -1), topk)
            rw = rw / rw.sum(-1, keepdim=True)
            torch.testing.assert_close(w.cpu(), rw, atol=1e-2, rtol=0)
            ow, oid = oracle.route_from_gate(h, gate, topk)
            torch.testing.assert_close(w.cpu(), ow, atol=1e-4, rtol=0)
            # ids can only differ where fp32 accumulation order flips a near-tie
            assert (ids.cpu() != oid).float().mean() < 0.01


@pytest.mark.parametrize("E,topk,H", [(8, 2, 1024), (64, 6, 2048), (16, 4, 520), (5, 2, 64)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_route_gate_fused_gemm(native, E, topk, H, dtype):
    from fast_route_amd.ops.stable_route import fused_route
    for M in (1, 70, 300):
        _say(f"route_gate E={E} k={topk} H={H} dtype={dtype} M={M}")
        g = torch.Generator().manual_seed(E + H + M)
        h = (torch.randn(M, H, generator=g) / 4).to(dtype)
        gate = (torch.randn(H, E, generator=g) / 4).to(dtype)
        tw = torch.empty(M, topk, dtype=torch.float32, device="cuda")
        ti = torch.empty(M, topk, dtype=torch.int32, device="cuda")
        w, ids = fused_route(h.cuda(), gate.cuda(), topk, tw, ti, True)
        torch.cuda.synchronize()
        logits = h.double() @ gate.double()
        ow, oid = oracle.gating_topk(logits.float(), topk, True)
        # fp32 MFMA accumulation vs float64 reference: ids may flip only at near-ties
        flips = (ids.cpu() != oid)
        assert flips.float().mean() < 0.02
        ok = ~flips.any(dim=1)
        torch.testing.assert_close(w.cpu()[ok], ow[ok], atol=1e-4, rtol=0)


@pytest.mark.parametrize("E,topk,H", [(8, 2, 264), (64, 6, 256), (24, 3, 512), (128, 8, 256), (100, 6, 512)])
def test_route_gate_large_batch(native, E, topk, H):
    """From 16384 tokens on the kernel takes its unsplit form (64 or 128 tokens per workgroup,
    every wavefront the whole K range of its own tokens); 16500 tokens leave a ragged last
    workgroup."""
    from fast_route_amd.ops.stable_route import fused_route
    M = 16500
    _say(f"route_gate large batch E={E} k={topk} H={H}")
    g = torch.Generator().manual_seed(E * 7 + H)
    h = (torch.randn(M, H, generator=g) / 4).to(torch.bfloat16)
    gate = (torch.randn(H, E, generator=g) / 4).to(torch.bfloat16)
    tw = torch.empty(M, topk, dtype=torch.float32, device="cuda")
    ti = torch.empty(M, topk, dtype=torch.int32, device="cuda")
    w, ids = fused_route(h.cuda(), gate.cuda(), topk, tw, ti, True)
    torch.cuda.synchronize()
    ow, oid = oracle.gating_topk((h.double() @ gate.double()).float(), topk, True)
    flips = (ids.cpu() != oid)
    assert flips.float().mean() < 0.02
    ok = ~flips.any(dim=1)
    torch.testing.assert_close(w.cpu()[ok], ow[ok], atol=1e-4, rtol=0)


@pytest.mark.parametrize("E,topk,H", [(16, 2, 4096), (128, 4, 1024), (100, 3, 512)])
def test_fused_route_half_and_int64_buffers(native, E, topk, H):
    """The reference's own recipe hands fused_route fp16 weight and int64 id buffers of [M, E]
    (tests/test_route.py:30-38) and allows up to 128 experts (ops/stable_route.py:130-134):
    both must give the fp32-logit result, not one rounded to the operand type first."""
    from fast_route_amd.ops.stable_route import fused_route
    for M in (3, 257):
        _say(f"fused_route fp16/int64 buffers E={E} k={topk} H={H} M={M}")
        g = torch.Generator().manual_seed(E * 31 + H + M)
        h = (torch.randn(M, H, generator=g) / 10).half()
        gate = (torch.randn(H, E, generator=g) / 10).half()
        tw = torch.empty(M, E, dtype=torch.float16, device="cuda")
        ti = torch.empty(M, E, dtype=torch.int64, device="cuda")
        w, ids = fused_route(h.cuda(), gate.cuda(), topk, tw, ti, True)
        torch.cuda.synchronize()
        assert w.dtype == torch.float16 and ids.dtype == torch.int64 and w.shape == ids.shape == (M, topk)
        ow, oid = oracle.gating_topk((h.double() @ gate.double()).float(), topk, True)
        flips = (ids.cpu() != oid.long())
        assert flips.float().mean() < 0.02   # fp32 against float64 logits: near-ties only
        ok = ~flips.any(dim=1)
        torch.testing.assert_close(w.cpu().float()[ok], ow[ok], atol=1e-3, rtol=0)  # fp16 storage of the weights
