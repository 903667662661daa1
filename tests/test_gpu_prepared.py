"""GPU parity of the prepared (pre-tiled) weight layout: the re-layout itself bit-exact against the oracle's
permutation, and every layer / GEMM entry point bit-identical to its row-major call wherever the same kernels
run (from 5 tokens up), within the layer tolerance against the fp32 oracle below that."""
import sys

import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu


def _say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


def ref_scale(t):
    return t.float().abs().max().cpu()


def _inputs(M, H, Fd, E, seed, dtype, zipf=False):
    x, logits, w1, w2 = oracle.make_inputs(M, H, Fd, E, seed=seed, zipf=zipf)
    return x.to(dtype), logits, w1.to(dtype), w2.to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_prepare_weights_matches_the_oracle_permutation(native, dtype):
    from fast_route_amd import prepare_weights
    _say(f"prepare_weights {dtype}")
    _, _, w1, w2 = _inputs(1, 256, 192, 3, 7, dtype)
    w1p, w2p, flags = prepare_weights(w1.cuda(), w2.cuda(), "both")
    torch.cuda.synchronize()
    assert flags == 0x300
    assert torch.equal(w1p.cpu().view(torch.int16), oracle.tile_weights(w1).view(torch.int16))
    assert torch.equal(w2p.cpu().view(torch.int16), oracle.tile_weights(w2).view(torch.int16))


def test_prepare_weights_fp8_codes(native):
    """The byte-wise form (128 elements per K tile) through the C ABI."""
    from fast_route_amd import _native as N
    _say("prepare_weights fp8 codes")
    w = torch.randint(0, 255, (2, 128, 384), dtype=torch.uint8)
    wd = w.cuda()
    out = torch.empty_like(wd)
    N.check(N.lib().fr_moe_prepare_weights(wd.data_ptr(), N.FR_FP8_E4M3, 2, 128, 384, out.data_ptr(), N.stream_ptr(wd.device)))
    torch.cuda.synchronize()
    assert torch.equal(out.cpu(), oracle.tile_weights(w))


def test_prepare_weights_rejects_what_it_cannot_tile(native):
    from fast_route_amd import _native as N
    w = torch.zeros(1, 96, 64, dtype=torch.bfloat16, device="cuda")
    out = torch.empty_like(w)
    with pytest.raises(AssertionError):
        N.check(N.lib().fr_moe_prepare_weights(w.data_ptr(), N.FR_BF16, 1, 96, 64, out.data_ptr(), None))   # rows % 64
    with pytest.raises(AssertionError):
        N.check(N.lib().fr_moe_prepare_weights(w.data_ptr(), N.FR_BF16, 1, 64, 96, out.data_ptr(), None))   # K tiles
    with pytest.raises(AssertionError):
        N.check(N.lib().fr_moe_prepare_weights(w.data_ptr(), N.FR_BF16, 1, 64, 64, w.data_ptr(), None))     # in place


@pytest.mark.parametrize("M", [1, 3, 5, 16, 40, 100, 300, 700, 3000])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("which", ["w2", "both"])
def test_layer_with_prepared_weights(native, M, dtype, which):
    """Small layer shape at token counts that hit every tile plan (16 ... 256-row blocks)."""
    from fast_route_amd import fused_moe, prepare_weights
    _say(f"prepared layer M={M} {dtype} {which}")
    x, logits, w1, w2 = _inputs(M, 1024, 3584, 8, 1337, dtype)
    xd, ld, w1d, w2d = x.cuda(), logits.cuda(), w1.cuda(), w2.cuda()
    w1p, w2p, flags = prepare_weights(w1d, w2d, which)
    assert (w1p.data_ptr() == w1d.data_ptr()) == (which == "w2")
    out_p = fused_moe(xd, w1p, w2p, ld, 2, True, weights_prepared=flags)
    out_r = fused_moe(xd, w1d, w2d, ld, 2, True)
    torch.cuda.synchronize()
    if M > 4:  # same kernels, same order of every sum
        assert torch.equal(out_p, out_r), f"M={M}: prepared and row-major outputs differ"
    if M == 3000:  # the plan keeps this width on 128-row blocks: the 256-row tiles (32x32x16 MFMA form) by override
        import fast_route_amd as fr
        with fr.tunables(block=256):
            out_p2 = fused_moe(xd, w1p, w2p, ld, 2, True, weights_prepared=flags)
            out_r2 = fused_moe(xd, w1d, w2d, ld, 2, True)
            torch.cuda.synchronize()
        assert torch.equal(out_p2, out_r2), "256-row blocks: prepared and row-major outputs differ"
        assert (out_p2.float() - out_p.float()).abs().max().cpu() <= 2.0 ** -6 * ref_scale(out_p)
    ref = oracle.fused_moe(x, w1, w2, logits, 2, True)
    err = (out_p.float().cpu() - ref).abs().max()
    assert err <= 2.0 ** -6 * ref.abs().max(), f"M={M}: max abs err {err:.3e}"


@pytest.mark.parametrize("M", [32, 512, 2500])
def test_fine_grained_layer_with_prepared_weights(native, M):
    from fast_route_amd import fused_moe, prepare_weights
    _say(f"prepared fine-grained layer M={M}")
    x, logits, w1, w2 = _inputs(M, 512, 384, 64, 99, torch.bfloat16, zipf=True)
    xd, ld, w1d, w2d = x.cuda(), logits.cuda(), w1.cuda(), w2.cuda()
    w1p, w2p, flags = prepare_weights(w1d, w2d, "both")
    out_p = fused_moe(xd, w1p, w2p, ld, 6, True, weights_prepared=flags)
    out_r = fused_moe(xd, w1d, w2d, ld, 6, True)
    torch.cuda.synchronize()
    assert torch.equal(out_p, out_r)


def test_fused_experts_and_inplace_with_prepared_weights(native):
    from fast_route_amd import fused_experts, prepare_weights
    _say("prepared fused_experts, inplace")
    x, logits, w1, w2 = _inputs(200, 1024, 3584, 8, 3, torch.bfloat16)
    tw, ti = oracle.gating_topk(logits, 2, True)
    xd, w1d, w2d = x.cuda(), w1.cuda(), w2.cuda()
    w1p, w2p, flags = prepare_weights(w1d, w2d, "both")
    ref = fused_experts(xd, w1d, w2d, tw.cuda(), ti.cuda())
    xin = xd.clone()
    got = fused_experts(xin, w1p, w2p, tw.cuda(), ti.cuda(), inplace=True, weights_prepared=flags)
    torch.cuda.synchronize()
    assert got.data_ptr() == xin.data_ptr()
    assert torch.equal(got, ref)


def test_mixtral_width_with_prepared_weights(native):
    """Full Mixtral width (H 4096, F 14336) on two experts: 512-byte K tiles of the 16- and 32-row gate/up GEMMs,
    the 64-row tiles, the persistent 128-, 160- and 256-row tiles with their last-round split."""
    from fast_route_amd import fused_moe, prepare_weights
    H, Fd, E = 4096, 14336, 2
    g = torch.Generator().manual_seed(11)
    w1 = (torch.randn(E, 2 * Fd, H, generator=g) * 0.02).to(torch.bfloat16).cuda()
    w2 = (torch.randn(E, H, Fd, generator=g) * 0.02).to(torch.bfloat16).cuda()
    w1p, w2p, flags = prepare_weights(w1, w2, "both")
    for M in (6, 20, 40, 150, 520, 600, 1300):  # 520 / 600: 160-row blocks; 1300: 256-row blocks (16x16x32 form)
        _say(f"prepared Mixtral width M={M}")
        x = torch.randn(M, H, generator=g).to(torch.bfloat16).cuda()
        logits = torch.randn(M, E, generator=g).cuda()
        out_p = fused_moe(x, w1p, w2p, logits, 2, True, weights_prepared=flags)
        out_r = fused_moe(x, w1, w2, logits, 2, True)
        torch.cuda.synchronize()
        assert torch.equal(out_p, out_r), f"M={M}"


def test_fp8_layer_with_prepared_down_weights(native):
    """fp8 layer with the e4m3 codes of w2 tiled (flag in the activation dtype argument): bit-identical."""
    from fast_route_amd import _native as N, prepare_weights_fp8
    from fast_route_amd.layers.fused_moe import plan
    _say("prepared fp8 down weights")
    M, H, Fd, E = 300, 1024, 3584, 8
    x, logits, w1, w2 = _inputs(M, H, Fd, E, 21, torch.bfloat16)
    xd, ld = x.cuda(), logits.cuda()
    w1q, w1s, w2q, w2s = prepare_weights_fp8(w1.cuda(), w2.cuda())
    w2t = torch.empty_like(w2q)
    N.check(N.lib().fr_moe_prepare_weights(w2q.data_ptr(), N.FR_FP8_E4M3, E, H, Fd, w2t.data_ptr(), N.stream_ptr(xd.device)))
    p = plan(M, H, Fd, E, 2, None, code=N.FR_FP8_E4M3)
    ws = torch.empty(p.workspace_bytes, dtype=torch.uint8, device="cuda")
    outs = []
    for wq, xcode in ((w2q, N.FR_BF16), (w2t, N.FR_BF16 | N.FR_W2_TILED)):
        out = torch.empty_like(xd)
        N.check(N.lib().fr_fused_moe_fp8(xd.data_ptr(), xcode, w1q.data_ptr(), w1s.data_ptr(), wq.data_ptr(), w2s.data_ptr(),
                                         ld.data_ptr(), N.FR_F32, M, H, Fd, E, 2, 1, out.data_ptr(), ws.data_ptr(),
                                         ws.numel(), N.stream_ptr(xd.device)))
        outs.append(out)
    torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1])
