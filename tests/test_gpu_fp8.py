"""GPU parity of the fp8 (e4m3fn) path.  The reference has no fp8 code, so the
oracle here is this build's own definition (dequantise -> fp32), see oracle/moe_oracle.py."""
import sys

import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu


def _say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_row_quantisation_bit_exact(native, dtype):
    from fast_route_amd import quantize_rows_e4m3
    # rows of up to 16384 elements are held in registers by a workgroup (2, 4 or 8 chunks per thread, the last
    # one partly filled); longer rows take the two-pass kernel
    for rows, K, std in ((1, 16, 1.0), (37, 1024, 1.0), (130, 4096, 0.02), (16, 14336, 3.0), (9, 5008, 1.0),
                         (3, 9008, 0.5), (4, 16384, 1.0), (5, 16400, 1.0)):
        _say(f"quant rows={rows} K={K} std={std} {dtype}")
        g = torch.Generator().manual_seed(rows * 7 + K)
        x = (torch.randn(rows, K, generator=g) * std).to(dtype)
        if rows > 2:
            x[1].zero_()                      # all-zero row -> scale 1, codes 0
            x[2, 5] = 448.0 if dtype == torch.bfloat16 else 400.0
        q, s = quantize_rows_e4m3(x.cuda())
        torch.cuda.synchronize()
        rq, rs = oracle.quant_e4m3_rows(x)
        assert np.array_equal(s.cpu().numpy(), rs), "scales differ"
        got, ref = q.cpu().numpy(), rq
        zero = (ref & 0x7F) == 0              # the sign of a zero code is not significant
        assert np.array_equal(got[~zero], ref[~zero]) and ((got[zero] & 0x7F) == 0).all(), "codes differ"


@pytest.mark.parametrize("M", [16, 64, 200, 700, 2048])
def test_fp8_layer_vs_oracle(native, M):
    """fp8 workload shape family (E8 top2) at reduced width; every tile plan is hit.
    Tolerance: the GPU and the oracle quantise the same bf16 activations, so they
    differ only by fp32 summation order, occasional 1-ulp flips of the bf16
    intermediate (and hence a few fp8 codes): ||out-ref||_F <= 1e-2 ||ref||_F and
    max|out-ref| <= 2**-5 max|ref|."""
    from fast_route_amd import fused_moe_fp8, prepare_weights_fp8
    _say(f"fp8 layer M={M}")
    H, Fd, E, k = 512, 1024, 8, 2
    x, logits, w1, w2 = oracle.make_inputs(M, H, Fd, E, seed=77)
    x, w1, w2 = x.bfloat16(), w1.bfloat16(), w2.bfloat16()
    w1q, w1s, w2q, w2s = prepare_weights_fp8(w1.cuda(), w2.cuda())
    out = fused_moe_fp8(x.cuda(), w1q, w1s, w2q, w2s, logits.cuda(), k, True)
    torch.cuda.synchronize()
    ref, parts = oracle.fused_moe_fp8(x, w1, w2, logits, k, True)
    # the prepared weights are bit-identical to the oracle's
    assert np.array_equal(w1s.cpu().numpy(), parts["w1_scale"]) and np.array_equal(w2s.cpu().numpy(), parts["w2_scale"])
    z = (parts["w1_codes"] & 0x7F) == 0
    assert np.array_equal(w1q.cpu().numpy()[~z], parts["w1_codes"][~z])
    o = out.float().cpu()
    assert torch.isfinite(o).all()
    rel = (o - ref).norm() / ref.norm()
    err = (o - ref).abs().max()
    assert rel <= 1e-2, f"rel F error {rel:.3e}"
    assert err <= 2.0 ** -5 * ref.abs().max(), f"max abs err {err:.3e}"
    # and it stays close to the unquantised fp32 layer (quantisation noise only)
    full = oracle.fused_moe(x, w1, w2, logits, k, True)
    assert (o - full).norm() / full.norm() < 0.08


def test_fp8_layer_with_64_row_blocks(native):
    """H = 4096 with 40 pairs per expert: the plan takes 64-row routing blocks for fp8 too."""
    from fast_route_amd import fused_moe_fp8, prepare_weights_fp8
    from fast_route_amd.layers.fused_moe import plan
    _say("fp8 layer with 64-row blocks")
    M, H, Fd, E, k = 160, 4096, 1024, 8, 2
    from fast_route_amd import _native as N
    assert plan(M, H, Fd, E, k, None, code=N.FR_FP8_E4M3).block == 64
    x, logits, w1, w2 = oracle.make_inputs(M, H, Fd, E, seed=64)
    x, w1, w2 = x.bfloat16(), w1.bfloat16(), w2.bfloat16()
    w1q, w1s, w2q, w2s = prepare_weights_fp8(w1.cuda(), w2.cuda())
    out = fused_moe_fp8(x.cuda(), w1q, w1s, w2q, w2s, logits.cuda(), k, True)
    torch.cuda.synchronize()
    ref, _ = oracle.fused_moe_fp8(x, w1, w2, logits, k, True)
    o = out.float().cpu()
    assert torch.isfinite(o).all()
    assert (o - ref).norm() / ref.norm() <= 1e-2
    assert (o - ref).abs().max() <= 2.0 ** -5 * ref.abs().max()


def test_fp8_mixtral_shape_sampled(native):
    """Full fp8 workload shape (H4096 F14336 E8 top2), M in {16, 128, 256, 512, 1024, 4096} (512 and 1024: 160-row blocks): sampled tokens vs the
    oracle.  At M=4096 the down projection runs the persistent form with its last round of tiles
    split along K."""
    from fast_route_amd import fused_moe_fp8, prepare_weights_fp8
    H, Fd, E, k = 4096, 14336, 8, 2
    g = torch.Generator(device="cuda").manual_seed(5)
    w1 = (torch.randn(E, 2 * Fd, H, generator=g, device="cuda") * 0.02).bfloat16()
    w2 = (torch.randn(E, H, Fd, generator=g, device="cuda") * 0.02).bfloat16()
    w1q, w1s, w2q, w2s = prepare_weights_fp8(w1, w2)
    w1c, w2c = w1.cpu(), w2.cpu()
    wq = oracle.quantize_weights_fp8(w1c, w2c)  # once: 1.4e9 weights through the CPU encoder
    for M in (16, 128, 256, 512, 1024, 4096):
        _say(f"fp8 mixtral M={M}")
        x = torch.randn(M, H, generator=g, device="cuda").bfloat16()
        logits = torch.randn(M, E, generator=g, device="cuda")
        out = fused_moe_fp8(x, w1q, w1s, w2q, w2s, logits, k, True)
        torch.cuda.synchronize()
        sample = torch.arange(0, M, max(1, M // 12))[:12]
        ref, _ = oracle.fused_moe_fp8(x[sample].cpu(), w1c, w2c, logits[sample].cpu(), k, True, weights_q=wq)
        o = out[sample].float().cpu()
        assert (o - ref).norm() / ref.norm() <= 1e-2
        # same quantised operands on both sides: what is left is accumulation order and the bf16 rounding of
        # the activated row (which can flip an e4m3 code of its re-quantisation) and of the output: the bound of the other fp8 tests
        assert (o - ref).abs().max() <= 2.0 ** -5 * ref.abs().max(), f"M={M}: max abs err {(o - ref).abs().max():.3e} of {ref.abs().max():.3e}"
        out2 = fused_moe_fp8(x, w1q, w1s, w2q, w2s, logits, k, True)
        assert torch.equal(out, out2)


def test_fp8_down_projection_tail_split(native, rows256):
    """Routing built so that the down projection has 8 token blocks x 2 feature tiles of 256 rows
    over K = 4096: two tiles per XCD, each cut into 8 K slices whose sum the fix-up kernel scales
    (activation-row scale x weight-row scale x routed weight) and rounds."""
    from fast_route_amd import fused_moe_fp8, prepare_weights_fp8
    from fast_route_amd.layers.fused_moe import plan
    from fast_route_amd import _native as N
    _say("fp8 tail split")
    H, Fd, E, k, M = 512, 4096, 2, 1, 2048
    p = plan(M, H, Fd, E, k, torch.bfloat16, code=N.FR_FP8_E4M3)
    assert p.block == 256 and p.tail_bytes > 0 and p.split_k == 1
    g = torch.Generator().manual_seed(91)
    x = torch.randn(M, H, generator=g).bfloat16()
    w1 = (torch.randn(E, 2 * Fd, H, generator=g) * 0.02).bfloat16()
    w2 = (torch.randn(E, H, Fd, generator=g) * 0.02).bfloat16()
    ids = torch.cat([torch.zeros(1280, dtype=torch.long), torch.ones(768, dtype=torch.long)])[torch.randperm(M, generator=g)]
    logits = torch.full((M, E), -4.0)
    logits[torch.arange(M), ids] = 4.0
    w1q, w1s, w2q, w2s = prepare_weights_fp8(w1.cuda(), w2.cuda())
    out = fused_moe_fp8(x.cuda(), w1q, w1s, w2q, w2s, logits.cuda(), k, True)
    torch.cuda.synchronize()
    ref, _ = oracle.fused_moe_fp8(x, w1, w2, logits, k, True)
    o = out.float().cpu()
    assert torch.isfinite(o).all()
    assert (o - ref).norm() / ref.norm() <= 1e-2
    assert (o - ref).abs().max() <= 2.0 ** -5 * ref.abs().max()


def test_fp8_one_wavefront_per_simd_tile_equals_the_eight_wavefront_tile(native):
    """fp8 on 256-row blocks with 16 K tiles (2048 elements) or more runs on four wavefronts of 128 x 128 outputs
    (moe_gemm_quad_kernel, 32x32x64 MFMAs); the no_quad knob sends the call to the eight-wavefront kernels.  Same
    MFMA shape and K order: equal bit for bit, and within the fp8 bounds of the oracle.  Sixteen experts with a mix
    of full, under-half and over-half blocks (half tiles), 2304 and 2560 elements of K (18 and 20 K tiles); top-2
    routing by logits."""
    import fast_route_amd as fr
    from fast_route_amd import fused_moe_fp8, prepare_weights_fp8
    _say("fp8 quad tile vs eight-wavefront tile")
    H, Fd, E, k, M = 2304, 2560, 16, 2, 2600
    g = torch.Generator().manual_seed(93)
    x = torch.randn(M, H, generator=g).bfloat16()
    w1 = (torch.randn(E, 2 * Fd, H, generator=g) * 0.02).bfloat16()
    w2 = (torch.randn(E, H, Fd, generator=g) * 0.02).bfloat16()
    logits = torch.randn(M, E, generator=g) + torch.linspace(2.0, -2.0, E)  # skewed loads: 1 .. 3 blocks per expert
    w1q, w1s, w2q, w2s = prepare_weights_fp8(w1.cuda(), w2.cuda())
    try:
        with fr.tunables(block=256):
            quad = fused_moe_fp8(x.cuda(), w1q, w1s, w2q, w2s, logits.cuda(), k, True)
        with fr.tunables(block=256, no_quad=True):
            eight = fused_moe_fp8(x.cuda(), w1q, w1s, w2q, w2s, logits.cuda(), k, True)
        torch.cuda.synchronize()
    finally:
        fr.reset_tunables()
    assert torch.equal(quad, eight), "the two 256-row fp8 kernels differ"
    ref, _ = oracle.fused_moe_fp8(x, w1, w2, logits, k, True)
    o = quad.float().cpu()
    assert torch.isfinite(o).all()
    assert (o - ref).norm() / ref.norm() <= 1e-2
    assert (o - ref).abs().max() <= 2.0 ** -5 * ref.abs().max()


def test_fp8_random_shapes_against_oracle(native):
    """Sixteen seeded random fp8 layer shapes against the oracle (same tolerance as above)."""
    from fast_route_amd import fused_moe_fp8, prepare_weights_fp8
    rng = np.random.default_rng(8)
    for case in range(16):
        E = int(rng.choice([1, 2, 4, 8, 16, 64]))
        k = int(rng.integers(1, min(E, 6) + 1))
        H = int(rng.choice([256, 512, 1024, 4096]))
        Fd = int(rng.choice([256, 512, 768]))
        M = int(rng.choice([1, 2, 5, 17, 40, 100, 160, 257, 500]))
        _say(f"fp8 random case {case}: M={M} H={H} F={Fd} E={E} k={k}")
        x, logits, w1, w2 = oracle.make_inputs(M, H, Fd, E, seed=500 + case)
        x, w1, w2 = x.bfloat16(), w1.bfloat16(), w2.bfloat16()
        w1q, w1s, w2q, w2s = prepare_weights_fp8(w1.cuda(), w2.cuda())
        out = fused_moe_fp8(x.cuda(), w1q, w1s, w2q, w2s, logits.cuda(), k, True)
        torch.cuda.synchronize()
        ref, _ = oracle.fused_moe_fp8(x, w1, w2, logits, k, True)
        o = out.float().cpu()
        assert torch.isfinite(o).all()
        assert (o - ref).norm() / ref.norm() <= 1e-2, f"case {case}"
        assert (o - ref).abs().max() <= 2.0 ** -5 * ref.abs().max(), f"case {case}"
