"""GPU parity: grouped GEMMs, fused epilogues and the whole layer vs the fp32 oracle.

Tolerance (stated once, used everywhere below): operands are bf16/fp16, products
accumulate in fp32, the activated intermediate is stored in the operand dtype and
the output is rounded once to the operand dtype.  Against the pure-fp32 oracle
evaluated on the same rounded operands we require
    max|out - ref| <= 2**-6 * max|ref|      (a few output ulps at the largest magnitude)
    ||out - ref||_F <= 6e-3 * ||ref||_F     (bf16; 1.5e-3 for fp16)
"""
import sys

import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu


def _say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


def _assert_close(out, ref, dtype, what=""):
    out, ref = out.float().cpu(), ref.float()
    assert torch.isfinite(out).all(), what + ": non-finite output"
    scale = ref.abs().max().clamp(min=1e-30)
    err = (out - ref).abs().max()
    rel_f = (out - ref).norm() / ref.norm().clamp(min=1e-30)
    lim_f = 6e-3 if dtype == torch.bfloat16 else 1.5e-3
    assert err <= 2.0 ** -6 * scale, f"{what}: max abs err {err:.3e} vs scale {scale:.3e}"
    assert rel_f <= lim_f, f"{what}: relative Frobenius error {rel_f:.3e}"


def _inputs(M, H, Fd, E, seed, dtype, zipf=False):
    x, logits, w1, w2 = oracle.make_inputs(M, H, Fd, E, seed=seed, zipf=zipf)
    return x.to(dtype), logits, w1.to(dtype), w2.to(dtype)


@pytest.mark.parametrize("M", [1, 16, 64, 200, 512, 2048])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_small_layer_config(native, M, dtype):
    """Small layer (H1024 F3584 E8 top2) at token counts that hit every tile plan."""
    from fast_route_amd import fused_moe
    _say(f"layer C1 M={M} dtype={dtype}")
    x, logits, w1, w2 = _inputs(M, 1024, 3584, 8, 1337, dtype)
    out = fused_moe(x.cuda(), w1.cuda(), w2.cuda(), logits.cuda(), 2, True)
    torch.cuda.synchronize()
    ref = oracle.fused_moe(x, w1, w2, logits, 2, True)
    _assert_close(out, ref, dtype, f"C1 M={M}")


@pytest.mark.parametrize("M", [1, 32, 128, 700])
def test_fine_grained_config(native, M):
    """Fine-grained many-expert shape family (E64 top6, Zipf-skewed load), reduced H/F for CPU oracle time."""
    from fast_route_amd import fused_moe
    _say(f"layer C4-like M={M}")
    x, logits, w1, w2 = _inputs(M, 512, 384, 64, 99, torch.bfloat16, zipf=True)
    out = fused_moe(x.cuda(), w1.cuda(), w2.cuda(), logits.cuda(), 6, True)
    torch.cuda.synchronize()
    ref = oracle.fused_moe(x, w1, w2, logits, 6, True)
    _assert_close(out, ref, torch.bfloat16, f"C4 M={M}")


def test_fine_grained_full_width(native):
    """The fine-grained workload at its real H2048 / F1408 / E64 / top-6 with Zipf-skewed load, every token
    count of its sweep: all tokens against the oracle up to 512, a sample of 48 tokens above."""
    from fast_route_amd import fused_moe
    H, Fd, E, k = 2048, 1408, 64, 6
    _, _, w1, w2 = _inputs(1, H, Fd, E, 5, torch.bfloat16)
    w1d, w2d = w1.cuda(), w2.cuda()
    for M in (1, 32, 128, 512, 2048, 8192):
        _say(f"layer C4 full width M={M}")
        g = torch.Generator().manual_seed(500 + M)
        x = torch.randn(M, H, generator=g).bfloat16()
        logits = oracle.zipf_logits(M, E, 600 + M)
        out = fused_moe(x.cuda(), w1d, w2d, logits.cuda(), k, True)
        torch.cuda.synchronize()
        assert torch.isfinite(out.float()).all()
        sample = torch.arange(M) if M <= 512 else torch.arange(0, M, M // 48)[:48]
        ref = oracle.fused_moe(x[sample], w1, w2, logits[sample], k, True)
        _assert_close(out[sample], ref, torch.bfloat16, f"C4 full M={M}")


def test_layer_edge_cases(native):
    from fast_route_amd import fused_moe, fused_experts
    dtype = torch.bfloat16
    x, logits, w1, w2 = _inputs(96, 256, 128, 8, 3, dtype)
    _say("edge: all tokens to one expert")
    ids = torch.full((96, 1), 5, dtype=torch.int32)
    wts = torch.rand(96, 1)
    out = fused_experts(x.cuda(), w1.cuda(), w2.cuda(), wts.cuda(), ids.cuda())
    _assert_close(out, oracle.moe_experts(x, w1, w2, wts, ids), dtype, "one expert")
    _say("edge: topk == E, renormalize False")
    out = fused_moe(x.cuda(), w1.cuda(), w2.cuda(), logits.cuda(), 8, False)
    _assert_close(out, oracle.fused_moe(x, w1, w2, logits, 8, False), dtype, "topk==E")
    _say("edge: inplace")
    xd = x.cuda().clone()
    out = fused_moe(xd, w1.cuda(), w2.cuda(), logits.cuda(), 2, True, inplace=True)
    assert out.data_ptr() == xd.data_ptr()
    _assert_close(out, oracle.fused_moe(x, w1, w2, logits, 2, True), dtype, "inplace")
    _say("edge: M == 0")
    out = fused_moe(x[:0].cuda(), w1.cuda(), w2.cuda(), logits[:0].cuda(), 2, True)
    assert out.shape == (0, 256)
    _say("edge: int64 ids / fp16 weights accepted by fused_experts")
    w, ids = oracle.gating_topk(logits, 2)
    out = fused_experts(x.cuda(), w1.cuda(), w2.cuda(), w.half().cuda(), ids.long().cuda())
    _assert_close(out, oracle.moe_experts(x, w1, w2, w.half().float(), ids), dtype, "dtype coercion")


@pytest.mark.parametrize("M", [4, 40])
def test_hidden_size_not_multiple_of_long_row_tile(native, M):
    """H = 384 is a multiple of 128 but not of 256: the decode gate/up GEMM must take the
    short-row tile instead of the 512-byte-row one."""
    from fast_route_amd import fused_moe
    _say(f"layer H=384 M={M}")
    x, logits, w1, w2 = _inputs(M, 384, 256, 8, 5, torch.bfloat16)
    out = fused_moe(x.cuda(), w1.cuda(), w2.cuda(), logits.cuda(), 2, True)
    torch.cuda.synchronize()
    _assert_close(out, oracle.fused_moe(x, w1, w2, logits, 2, True), torch.bfloat16, f"H=384 M={M}")


def test_token_matrix_of_4gib_is_refused(native):
    """Tile loads address rows by 32-bit byte offsets: a gathered token matrix of 4 GiB
    or more is refused before anything is launched (no memory of that size is touched)."""
    from fast_route_amd import _native as N
    H, Fd, E, k, block = 256, 128, 2, 1, 16
    M = (1 << 32) // (H * 2)  # M*H*2 bytes == 4 GiB exactly
    dummy = torch.zeros(1 << 16, dtype=torch.int32, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    rc = N.lib().fr_moe_gateup_silu(dummy.data_ptr(), dummy.data_ptr(), dummy.data_ptr(), dummy.data_ptr(),
                                    dummy.data_ptr(), M, H, Fd, E, k, block, N.FR_BF16, dummy.data_ptr(), None, st)
    assert rc == -2, rc
    assert b"4 GiB" in N.lib().fr_last_error_string()
    torch.cuda.synchronize()


def test_layer_rejects_bad_arguments(native):
    from fast_route_amd import fused_moe
    x, logits, w1, w2 = _inputs(8, 256, 128, 8, 3, torch.bfloat16)
    with pytest.raises(AssertionError, match="Incompatible dimensions"):
        fused_moe(x[:, :128].contiguous().cuda(), w1.cuda(), w2.cuda(), logits.cuda(), 2)
    with pytest.raises(AssertionError, match="Hidden_states must be contiguous"):
        fused_moe(x.cuda().t().contiguous().t(), w1.cuda(), w2.cuda(), logits.cuda(), 2)
    with pytest.raises(AssertionError):
        fused_moe(x.float().cuda(), w1.cuda(), w2.cuda(), logits.cuda(), 2)
    with pytest.raises(AssertionError):
        fused_moe(x.cuda(), w1.cuda(), w2.cuda(), logits.cuda(), 9)  # topk > E


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_layer_with_64_row_blocks(native, dtype):
    """26 to 52 pairs per expert with H >= 4096: the plan takes 64-row routing blocks (one block per
    expert, K of the down projection cut into slices)."""
    from fast_route_amd import fused_moe
    from fast_route_amd.layers.fused_moe import plan
    _say(f"layer with 64-row blocks {dtype}")
    M, H, Fd, E, k = 160, 4096, 1024, 8, 2
    p = plan(M, H, Fd, E, k, dtype)
    assert p.block == 64 and p.split_k >= 2
    x, logits, w1, w2 = _inputs(M, H, Fd, E, 64, dtype)
    out = fused_moe(x.cuda(), w1.cuda(), w2.cuda(), logits.cuda(), k, True)
    torch.cuda.synchronize()
    _assert_close(out, oracle.fused_moe(x, w1, w2, logits, k, True), dtype, "64-row blocks")


@pytest.mark.parametrize("block", [16, 32, 64, 128, 160, 256])
def test_op_level_chain_matches_reference_layer_recipe(native, block):
    """The reference layer spelled with its own ops (layers/stable_route.py:82-102):
    align -> grouped GEMM -> silu_and_mul -> grouped GEMM * weight -> sum."""
    from fast_route_amd.ops.fused_moe import invoke_fused_moe_kernel, moe_align_block_size
    _say(f"op chain block={block}")
    dtype = torch.bfloat16
    M, H, Fd, E, k = 150, 256, 384, 8, 2
    x, logits, w1, w2 = _inputs(M, H, Fd, E, 21, dtype)
    w, ids = oracle.gating_topk(logits, k)
    xd, w1d, w2d, wd, idd = x.cuda(), w1.cuda(), w2.cuda(), w.cuda(), ids.cuda()
    cfg = {"BLOCK_SIZE_M": block, "BLOCK_SIZE_N": 64, "BLOCK_SIZE_K": 32, "GROUP_SIZE_M": 8}
    s, e, npost = moe_align_block_size(idd, block, E)
    c1 = torch.empty((M, k, 2 * Fd), dtype=dtype, device="cuda")
    invoke_fused_moe_kernel(xd, w1d, c1, wd, idd, s, e, npost, False, k, cfg)
    ref1 = oracle.grouped_gemm(x, w1, w, ids, False, k)
    _assert_close(c1.view(M * k, -1), ref1, dtype, "gemm1")
    c2 = (torch.nn.functional.silu(c1[..., :Fd].float()) * c1[..., Fd:].float()).to(dtype).view(M * k, Fd)
    c3 = torch.empty((M, k, H), dtype=dtype, device="cuda")
    invoke_fused_moe_kernel(c2, w2d, c3, wd, idd, s, e, npost, True, 1, cfg)
    out = c3.float().sum(dim=1)
    torch.cuda.synchronize()
    _assert_close(out, oracle.moe_experts(x, w1, w2, w, ids), dtype, "op chain")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_block_256_several_tiles_per_workgroup(native, dtype):
    """With more 256x256 tiles than resident workgroups the 2-byte kernel walks several
    tiles per workgroup, the next tile's first loads issued during the current tile's last
    K tiles: 27 token blocks x 16 feature tiles = 432 tiles for at most 256 workgroups,
    so the grid mixes workgroups with one tile and with two."""
    from fast_route_amd import fused_moe
    from fast_route_amd.ops.fused_moe import invoke_fused_moe_kernel, moe_align_block_size
    _say(f"block 256, several tiles per workgroup, {dtype}")
    M, H, Fd, E, k, block = 3000, 512, 2048, 4, 2, 256
    x, logits, w1, w2 = _inputs(M, H, Fd, E, 33, dtype)
    w, ids = oracle.gating_topk(logits, k)
    xd, w1d, w2d, wd, idd = x.cuda(), w1.cuda(), w2.cuda(), w.cuda(), ids.cuda()
    cfg = {"BLOCK_SIZE_M": block, "BLOCK_SIZE_N": 64, "BLOCK_SIZE_K": 32, "GROUP_SIZE_M": 8}
    s, e, npost = moe_align_block_size(idd, block, E)
    c1 = torch.empty((M, k, 2 * Fd), dtype=dtype, device="cuda")
    invoke_fused_moe_kernel(xd, w1d, c1, wd, idd, s, e, npost, False, k, cfg)
    _assert_close(c1.view(M * k, -1), oracle.grouped_gemm(x, w1, w, ids, False, k), dtype, "gemm1")
    c2 = (torch.nn.functional.silu(c1[..., :Fd].float()) * c1[..., Fd:].float()).to(dtype).view(M * k, Fd)
    c3 = torch.empty((M, k, H), dtype=dtype, device="cuda")
    invoke_fused_moe_kernel(c2, w2d, c3, wd, idd, s, e, npost, True, 1, cfg)
    torch.cuda.synchronize()
    _assert_close(c3.float().sum(dim=1), oracle.moe_experts(x, w1, w2, w, ids), dtype, "op chain")
    # the fused layer at the same size takes the same kernels through its own plan
    out = fused_moe(xd, w1d, w2d, logits.cuda(), k, True)
    torch.cuda.synchronize()
    _assert_close(out, oracle.fused_moe(x, w1, w2, logits, k, True), dtype, "layer")


@pytest.mark.parametrize("rows", [256, 160])
@pytest.mark.parametrize("case", ["gate_up_after_whole_tile", "down_first_unit", "with_and_without_scratch"])
def test_last_round_of_tiles_split_along_k(native, rows, case):
    """256-row (and 160-row) tiles that only partly fill the last round of workgroups are cut along K over
    the idle ones and summed by a second launch.  Routing is constructed so that the tile
    counts are exact (k = 1, every expert a whole number of `rows`-token blocks):
    gate_up_after_whole_tile - 17 blocks x 16 feature tiles = 272 tiles, 34 per XCD: one whole
      round of 32 and 2 tiles cut into 8 K slices each (K = 4096 is 64 K tiles);
    down_first_unit - 8 blocks x 2 feature tiles over F = 4096: 2 tiles per XCD in 8 slices
      each, the slice being the workgroup's first and only unit;
    with_and_without_scratch - the two GEMM entry points with and without the scratch agree
      to fp32 summation order (same bf16 result up to one rounding)."""
    from fast_route_amd import _native as N, fused_experts
    from fast_route_amd.layers.fused_moe import plan
    import fast_route_amd as fr
    _say(f"tail split {case} rows={rows}")
    dtype = torch.bfloat16
    if case == "down_first_unit":
        H, Fd, E, blocks = 512, 4096, 2, (5, 3)
    else:
        H, Fd, E, blocks = 4096, 2048, 3, (9, 0, 8)
    M = rows * sum(blocks)
    g = torch.Generator().manual_seed(77)
    x = torch.randn(M, H, generator=g).to(dtype)
    w1 = (torch.randn(E, 2 * Fd, H, generator=g) * 0.02).to(dtype)
    w2 = (torch.randn(E, H, Fd, generator=g) * 0.02).to(dtype)
    ids = torch.cat([torch.full((rows * b,), e, dtype=torch.int32) for e, b in enumerate(blocks)])
    ids = ids[torch.randperm(M, generator=g)].view(M, 1)
    w = (torch.rand(M, 1, generator=g) + 0.5).float()
    with fr.tunables(block=rows):  # the plan itself keeps a short gate/up K on smaller blocks
        p = plan(M, H, Fd, E, 1, dtype)
    assert p.block == rows and p.tail_bytes > 0 and p.split_k == 1
    xd, w1d, w2d, wd, idd = x.cuda(), w1.cuda(), w2.cuda(), w.cuda(), ids.cuda()
    if case != "with_and_without_scratch":
        with fr.tunables(block=rows):
            out = fused_experts(xd, w1d, w2d, wd, idd)
        torch.cuda.synchronize()
        _assert_close(out, oracle.moe_experts(x, w1, w2, w, ids), dtype, case)
        return
    from fast_route_amd.ops.fused_moe import moe_align_block_size
    lib, st = N.lib(), torch.cuda.current_stream().cuda_stream
    s, e, npost = moe_align_block_size(idd, rows, E)
    tail = torch.empty(p.tail_bytes, dtype=torch.uint8, device="cuda")
    res = []
    for tptr in (None, tail.data_ptr()):
        act = torch.zeros(s.numel(), Fd, dtype=dtype, device="cuda")
        partial = torch.empty(M * H, dtype=torch.float32, device="cuda")
        out = torch.empty(M, H, dtype=dtype, device="cuda")
        N.check(lib.fr_moe_gateup_silu(xd.data_ptr(), w1d.data_ptr(), s.data_ptr(), e.data_ptr(), npost.data_ptr(), M, H,
                                       Fd, E, 1, rows, N.FR_BF16, act.data_ptr(), tptr, st))
        N.check(lib.fr_moe_down_combine(act.data_ptr(), w2d.data_ptr(), wd.data_ptr(), s.data_ptr(), e.data_ptr(),
                                        npost.data_ptr(), M, H, Fd, E, 1, rows, 1, N.FR_BF16, partial.data_ptr(),
                                        out.data_ptr(), tptr, st))
        torch.cuda.synchronize()
        res.append((act.float().cpu(), out.float().cpu()))
    (act0, out0), (act1, out1) = res
    assert not torch.equal(act0, act1), "the scratch changed nothing: the split path did not run"
    # one bf16 rounding apart at most (2^-8 relative), on values whose fp32 sums differ in the last bits
    assert ((act0 - act1).abs() <= 2.0 ** -7 * act0.abs().clamp(min=1e-3)).all()
    assert ((out0 - out1).abs() <= 2.0 ** -6 * out0.abs().max()).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,H,E,k", [(1, 4096, 8, 2), (2, 4096, 8, 2), (3, 4096, 8, 2), (4, 4096, 8, 2), (4, 8192, 4, 2),
                                      (2, 4096, 16, 6), (1, 8192, 8, 8), (3, 5120, 4, 2), (2, 6144, 8, 2), (4, 7168, 4, 3)])
def test_decode_gate_up_by_rows(native, M, H, E, k, dtype):
    """Up to four tokens with H = 4096, 5120, 6144, 7168 or 8192 (rows of 5 to 8 rounds' chunks): the gate/up
    projection streams each weight row
    past the routing block's token rows (dot products, no tiles) and leaves the same activation
    layout to the down projection.  H = 8192 with four tokens fills the token-row buffer."""
    from fast_route_amd import fused_moe
    _say(f"decode rows M={M} H={H} E={E} k={k} {dtype}")
    x, logits, w1, w2 = _inputs(M, H, 384, E, 100 + M + k, dtype)
    out = fused_moe(x.cuda(), w1.cuda(), w2.cuda(), logits.cuda(), k, True)
    torch.cuda.synchronize()
    _assert_close(out, oracle.fused_moe(x, w1, w2, logits, k, True), dtype, f"rows M={M} H={H}")


@pytest.mark.parametrize("block", [16, 32, 64, 128])
def test_decode_gate_up_by_rows_matches_tiles(native, block):
    """The same three tokens through the gate/up entry point with H = 4096 (rows, for blocks up to
    64 slots; 128-slot blocks keep the tiles) and, zero-extended to H = 4224 (not a multiple of
    4096: tiles), give the same activations up to the summation order; an expert chosen twice by
    one token puts more rows into a block than there are tokens, which costs the row form a second
    pass over that block."""
    from fast_route_amd import _native as N
    from fast_route_amd.ops.fused_moe import moe_align_block_size
    _say(f"decode rows vs tiles block={block}")
    dtype = torch.bfloat16
    M, H, Fd, E, k = 3, 4096, 256, 4, 2
    g = torch.Generator().manual_seed(block)
    x = torch.randn(M, H, generator=g).to(dtype)
    w1 = (torch.randn(E, 2 * Fd, H, generator=g) * 0.02).to(dtype)
    ids = torch.tensor([[1, 1], [1, 3], [0, 1]], dtype=torch.int32)   # expert 1: 4 rows from 3 tokens
    lib, st = N.lib(), torch.cuda.current_stream().cuda_stream
    s, e, npost = moe_align_block_size(ids.cuda(), block, E)
    acts = []
    for pad in (0, 128):
        xd = torch.nn.functional.pad(x, (0, pad)).contiguous().cuda()
        w1d = torch.nn.functional.pad(w1, (0, pad)).contiguous().cuda()
        act = torch.zeros(s.numel(), Fd, dtype=dtype, device="cuda")
        N.check(lib.fr_moe_gateup_silu(xd.data_ptr(), w1d.data_ptr(), s.data_ptr(), e.data_ptr(), npost.data_ptr(), M,
                                       H + pad, Fd, E, k, block, N.FR_BF16, act.data_ptr(), None, st))
        torch.cuda.synchronize()
        acts.append(act.float().cpu())
    # reference: every real slot's row (the tile kernel also fills the padding slots of a block, with
    # values nobody reads; the row form leaves them alone)
    sc = s.cpu()
    ref = torch.zeros_like(acts[0])
    real = torch.zeros(ref.shape[0], dtype=torch.bool)
    for slot in range(int(npost.item())):
        sid = int(sc[slot])
        if sid < M * k:
            gu = x[sid // k].float() @ w1[int(ids.view(-1)[sid])].float().T
            ref[slot] = torch.nn.functional.silu(gu[:Fd]) * gu[Fd:]
            real[slot] = True
    assert int(real.sum()) == M * k
    for a in acts:
        assert ((a - ref).abs() <= 2.0 ** -7 * ref.abs() + 1e-3)[real].all()
    if block <= 64:
        assert acts[0][~real].abs().sum() == 0


@pytest.mark.parametrize("M", [2, 16, 1536])
def test_layer_under_graph_capture(native, M):
    """The whole layer (router logits form) captured into a HIP graph after one warm-up call and
    replayed three times, with eager work and synchronisations between the replays and new inputs
    written into the captured buffers: every replay equals the eager result bit for bit.  M=2
    (with H = 4096) takes the gate/up projection by weight rows, M=16
    takes the decode kernels and the fused route+align launch, M=1536 the persistent kernels with
    their split last round and fix-up launches."""
    from fast_route_amd import _native as N
    from fast_route_amd.layers.fused_moe import plan
    _say(f"graph capture M={M}")
    dtype = torch.bfloat16
    H, Fd, E, k = (4096, 512, 4, 2) if M == 2 else (1024, 2048, 4, 2)
    x, logits, w1, w2 = _inputs(M, H, Fd, E, 55, dtype)
    xd, ld, w1d, w2d = x.cuda(), logits.cuda(), w1.cuda(), w2.cuda()
    p = plan(M, H, Fd, E, k, dtype)
    ws = torch.empty(max(p.workspace_bytes, 256), dtype=torch.uint8, device="cuda")
    out = torch.empty(M, H, dtype=dtype, device="cuda")
    lib = N.lib()

    def call(stream):
        N.check(lib.fr_fused_moe(xd.data_ptr(), w1d.data_ptr(), w2d.data_ptr(), ld.data_ptr(), N.FR_F32, M, H, Fd, E, k, 1,
                                 N.FR_BF16, out.data_ptr(), ws.data_ptr(), ws.numel(), stream))

    call(torch.cuda.current_stream().cuda_stream)  # warm-up: per-kernel attributes are set on first use
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        call(torch.cuda.current_stream().cuda_stream)
    for rep in range(3):
        gen = torch.Generator().manual_seed(100 + rep)
        xd.copy_(torch.randn(M, H, generator=gen).to(dtype))
        ld.copy_(torch.randn(M, E, generator=gen))
        call(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        eager = out.clone()
        out.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {rep} differs from the eager result"
    _assert_close(out, oracle.fused_moe(xd.cpu(), w1, w2, ld.cpu(), k, True), dtype, "graph replay")


@pytest.mark.parametrize("block", [128, 160, 256])
def test_grouped_gemm_with_blocks_in_any_order(native, block):
    """The op-level GEMM only needs every block to belong to one expert; routing arrays whose
    blocks are not in ascending expert order (here: reversed) are legal input.  The persistent
    kernels walk tiles expert by expert through a table built from an ascending expert_ids and
    must fall back to a plain walk when it is not."""
    from fast_route_amd.ops.fused_moe import invoke_fused_moe_kernel, moe_align_block_size
    _say(f"grouped GEMM, blocks reversed, block={block}")
    dtype = torch.bfloat16
    M, H, Fd, E, k = 1200, 512, 768, 6, 2
    x, logits, w1, w2 = _inputs(M, H, Fd, E, 41, dtype)
    w, ids = oracle.gating_topk(logits, k)
    xd, w1d, wd, idd = x.cuda(), w1.cuda(), w.cuda(), ids.cuda()
    s, e, npost = moe_align_block_size(idd, block, E)
    nb = int(npost.item()) // block
    s2, e2 = s.clone(), e.clone()
    s2[: nb * block] = s[: nb * block].view(nb, block).flip(0).reshape(-1)
    e2[:nb] = e[:nb].flip(0)
    cfg = {"BLOCK_SIZE_M": block, "BLOCK_SIZE_N": 64, "BLOCK_SIZE_K": 32, "GROUP_SIZE_M": 8}
    c1 = torch.empty((M, k, 2 * Fd), dtype=dtype, device="cuda")
    invoke_fused_moe_kernel(xd, w1d, c1, wd, idd, s2, e2, npost, False, k, cfg)
    torch.cuda.synchronize()
    _assert_close(c1.view(M * k, -1), oracle.grouped_gemm(x, w1, w, ids, False, k), dtype, "reversed blocks")


def test_stable_and_vllm_route_layers(native):
    """Gate-matrix entry points of both reference layers."""
    from fast_route_amd.layers import stable_route, vllm_route
    _say("gate-matrix layers")
    dtype = torch.bfloat16
    M, H, Fd, E, k = 80, 512, 256, 16, 2
    x, _, w1, w2 = _inputs(M, H, Fd, E, 8, dtype)
    gate = (torch.randn(H, E, generator=torch.Generator().manual_seed(1)) / 8).to(dtype)
    a = stable_route.fused_moe(x.cuda(), gate.cuda(), w1.cuda(), w2.cuda(), k, True)
    b = vllm_route.fused_moe(x.cuda(), gate.cuda(), w1.cuda(), w2.cuda(), k, True)
    torch.cuda.synchronize()
    # routing decided from fp32 logits on device; take the device's own selection for the oracle
    from fast_route_amd.ops.stable_route import fused_route
    tw = torch.empty(M, k, dtype=torch.float32, device="cuda")
    ti = torch.empty(M, k, dtype=torch.int32, device="cuda")
    w, ids = fused_route(x.cuda(), gate.cuda(), k, tw, ti, True)
    ref = oracle.moe_experts(x, w1, w2, w.cpu(), ids.cpu())
    _assert_close(a, ref, dtype, "stable_route layer")
    # the baseline layer rounds logits to bf16 before gating: compare on tokens routed identically
    lw, lid = oracle.gating_topk(torch.matmul(x.cuda(), gate.cuda()).cpu(), k, True)
    same = (lid == ids.cpu()).all(dim=1)
    assert same.float().mean() > 0.8
    refb = oracle.moe_experts(x, w1, w2, lw, lid)
    _assert_close(b, refb, dtype, "vllm_route layer")


def test_profile_twin_matches_layer_and_writes_trace(native, tmp_path):
    """layers/profile_fused_route.py: same result as the fused layer, bit for bit (same
    kernels, same plan), and a chrome trace with one complete event per stage."""
    import json
    from fast_route_amd.layers import profile_fused_route, stable_route
    _say("profile twin")
    dtype = torch.bfloat16
    M, H, Fd, E, k = 96, 512, 256, 8, 2
    x, _, w1, w2 = _inputs(M, H, Fd, E, 12, dtype)
    gate = (torch.randn(H, E, generator=torch.Generator().manual_seed(2)) / 8).to(dtype)
    ref = stable_route.fused_moe(x.cuda(), gate.cuda(), w1.cuda(), w2.cuda(), k, True)
    out = profile_fused_route.fused_moe(x.cuda(), gate.cuda(), w1.cuda(), w2.cuda(), k, True, save_dir=str(tmp_path))
    torch.cuda.synchronize()
    assert torch.equal(out, ref)
    # and against the oracle: routing from fp64 logits; tokens whose fp32 near-tie flipped an id are left out
    ow, oid = oracle.route_from_gate(x, gate, k)
    from fast_route_amd.ops.stable_route import fused_route
    tw = torch.empty(M, k, dtype=torch.float32, device="cuda")
    ti = torch.empty(M, k, dtype=torch.int32, device="cuda")
    _, ids = fused_route(x.cuda(), gate.cuda(), k, tw, ti, True)
    same = (ids.cpu() == oid).all(dim=1)
    assert same.float().mean() > 0.95
    want = oracle.moe_experts(x, w1, w2, ow, oid)
    _assert_close(out[same.cuda()], want[same], dtype, "profile twin vs oracle")
    path = tmp_path / f"fused_breakdown_{M}_{H}_{E}_{2 * Fd}_{k}.json"
    trace = json.loads(path.read_text())
    names = [e["name"] for e in trace["traceEvents"]]
    assert names == list(profile_fused_route.STAGES)
    assert all(e["ph"] == "X" and e["dur"] > 0 for e in trace["traceEvents"])
    ts = [e["ts"] for e in trace["traceEvents"]]
    assert ts == sorted(ts)


def test_transformer_layer_bench_runs_and_matches_its_parts(native):
    """fast_route_amd.transformer_layer_bench: the layer is attention + residual + the
    gate-matrix MoE; its output equals the MoE entry point applied to attn(x) + x."""
    from fast_route_amd import transformer_layer_bench as tb
    from fast_route_amd.layers.stable_route import fused_moe
    _say("transformer layer bench")
    rec, out, (gate, w1, w2, attn) = tb.run(seq=64, n=256, k=512, e=8, topk=2, b=2, n_head=4, head_dim=64,
                                            reps=3, warmup=1)
    assert out.shape == (2 * 64, 512) and torch.isfinite(out.float()).all()
    assert 0.0 < rec["moe_share"] <= 1.0 and rec["layer_ms"] > 0 and rec["layer_ms_p20"] <= rec["layer_ms_p80"]
    g = torch.Generator(device="cuda").manual_seed(1337)
    x = torch.randn((2, 64, 512), device="cuda", dtype=torch.float16, generator=g) / 10
    with torch.no_grad():
        h = (attn(x) + x).view(-1, 512)
        again = fused_moe(h, gate, w1, w2, 2, True, False)
    assert torch.equal(out, again)
    # against the oracle: the MoE of the layer's own attention output, routed and multiplied on the CPU
    hc, gc = h.cpu(), gate.cpu()
    ow, oid = oracle.route_from_gate(hc, gc, 2)
    from fast_route_amd.ops.stable_route import fused_route
    tw = torch.empty(h.shape[0], 2, dtype=torch.float32, device="cuda")
    ti = torch.empty(h.shape[0], 2, dtype=torch.int32, device="cuda")
    _, ids = fused_route(h, gate, 2, tw, ti, True)
    same = (ids.cpu() == oid).all(dim=1)
    assert same.float().mean() > 0.95
    want = oracle.moe_experts(hc, w1.cpu(), w2.cpu(), ow, oid)
    _assert_close(out[same.cuda()], want[same], torch.float16, "transformer layer vs oracle")


def test_mixtral_shape_sampled_tokens_and_properties(native):
    """Mixtral-8x7B shape at full size (H4096 F14336 E8 top2), every token count of its sweep:
    oracle on a sample of tokens and determinism; at 16 and 4096 tokens also the size-independent
    properties (batch independence, linearity in the routed weights) on all tokens."""
    from fast_route_amd import fused_moe, fused_experts
    dtype = torch.bfloat16
    H, Fd, E, k = 4096, 14336, 8, 2
    g = torch.Generator(device="cuda").manual_seed(1337)
    w1 = (torch.randn(E, 2 * Fd, H, generator=g, device="cuda") * 0.02).to(dtype)
    w2 = (torch.randn(E, H, Fd, generator=g, device="cuda") * 0.02).to(dtype)
    w1c, w2c = w1.cpu(), w2.cpu()
    for M in (1, 16, 64, 256, 1024, 4096, 16384):
        _say(f"mixtral full width M={M}")
        x = torch.randn(M, H, generator=g, device="cuda").to(dtype)
        logits = torch.randn(M, E, generator=g, device="cuda")
        out = fused_moe(x, w1, w2, logits, k, True)
        torch.cuda.synchronize()
        assert torch.isfinite(out.float()).all()
        sample = torch.arange(0, M, max(1, M // 24))[:24]
        ref = oracle.fused_moe(x[sample].cpu(), w1c, w2c, logits[sample].cpu(), k, True)
        _assert_close(out[sample], ref, dtype, f"mixtral M={M} sample")
        # determinism: same call, same bits
        out2 = fused_moe(x, w1, w2, logits, k, True)
        assert torch.equal(out, out2)
        if M not in (16, 4096):
            continue
        # a token's output does not depend on which other tokens share the batch
        half = fused_moe(x[: M // 2].contiguous(), w1, w2, logits[: M // 2].contiguous(), k, True)
        _assert_close(half, out[: M // 2].float().cpu(), dtype, "batch independence")
        # linearity in the routed weights: doubling them doubles the output (exact in binary fp)
        from fast_route_amd.ops.stable_route import topk_softmax
        w = torch.empty((M, k), dtype=torch.float32, device="cuda")
        ids = torch.empty((M, k), dtype=torch.int32, device="cuda")
        topk_softmax(w, ids, None, logits, renormalize=True)
        a = fused_experts(x, w1, w2, w, ids)
        b = fused_experts(x, w1, w2, 2 * w, ids)
        assert torch.equal(a, out) and torch.equal(b.float(), 2 * a.float())


@pytest.mark.parametrize("m", [1, 33, 222, 1024])
def test_reference_end_to_end_recipe(native, m):
    """The reference's own end-to-end check replayed (benchmarks/swizzle_moe/perf_test_moe.py:34-73):
    fp16 operands drawn as randn / 10, routing = torch.topk(softmax(randn score)), no renormalisation,
    experts-only entry point, torch_moe as the expectation, assert_close(atol=1e-2, rtol=0).
    Widths are scaled down from the reference's n=14336 / k=4096 to keep the CPU expectation quick."""
    from fast_route_amd import fused_experts
    n, k, e, topk = 1024, 512, 8, 2
    _say(f"reference recipe m={m} n={n} k={k} e={e} topk={topk}")
    torch.manual_seed(3227)  # the reference's seed for this check
    a = (torch.randn((m, k)) / 10).half()
    w1 = (torch.randn((e, 2 * n, k)) / 10).half()
    w2 = (torch.randn((e, k, n)) / 10).half()
    score = torch.softmax(torch.randn((m, e)), dim=-1)
    topk_weight, topk_ids = torch.topk(score, topk)
    out = fused_experts(a.cuda(), w1.cuda(), w2.cuda(), topk_weight.cuda(), topk_ids.cuda(), inplace=False)
    torch.cuda.synchronize()
    want = oracle.moe_experts(a, w1, w2, topk_weight, topk_ids)
    torch.testing.assert_close(out.float().cpu(), want, atol=1e-2, rtol=0)


@pytest.mark.parametrize("E,k,H,Fd", [(8, 2, 256, 4096), (8, 2, 512, 5120), (16, 6, 256, 4096), (8, 8, 128, 8192),
                                      (4, 1, 384, 14336), (64, 6, 256, 16384)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_decode_down_projection_by_rows(native, E, k, H, Fd, dtype):
    """At most 4 routed pairs and weight rows of 4096..16384 elements (multiples of 512): the down
    projection streams weight rows past the activated rows and sums a token's pairs itself - no partial
    buffer, no combine launch.  Token counts on both sides of that limit (up to 8 pairs), against the
    oracle; the same bits on every run."""
    from fast_route_amd import fused_moe, fused_experts
    for M in range(1, 8 // k + 1):
        _say(f"down by rows E={E} k={k} H={H} F={Fd} {dtype} M={M}")
        x, logits, w1, w2 = _inputs(M, H, Fd, E, 77 + M, dtype)
        xd, w1d, w2d, ld = x.cuda(), w1.cuda(), w2.cuda(), logits.cuda()
        out = fused_moe(xd, w1d, w2d, ld, k, True)
        torch.cuda.synchronize()
        _assert_close(out, oracle.fused_moe(x, w1, w2, logits, k, True), dtype, f"down by rows M={M}")
        for _ in range(3):
            assert torch.equal(fused_moe(xd, w1d, w2d, ld, k, True), out)
    if k == 2 and E >= 4:
        _say("down by rows: a token naming one expert twice, another token sharing it")
        ids = torch.tensor([[3, 3], [3, 1], [0, 2]], dtype=torch.int32)
        wts = torch.tensor([[0.25, 0.5], [0.7, 0.3], [0.9, 0.1]])
        x, _, w1, w2 = _inputs(3, H, Fd, E, 5, dtype)
        out = fused_experts(x.cuda(), w1.cuda(), w2.cuda(), wts.cuda(), ids.cuda())
        _assert_close(out, oracle.moe_experts(x, w1, w2, wts, ids), dtype, "down by rows, repeated expert")


def test_tunables_and_prepare(native):
    """Plan overrides (routing block, K slices, walk group, no last-round split) change the kernels a layer takes,
    never its result beyond fp32 summation order; fr_moe_prepare sets every kernel up without launching."""
    import fast_route_amd as fr
    from fast_route_amd import fused_moe
    dtype = torch.bfloat16
    fr.prepare(dtype)
    fr.prepare(torch.float16)
    fr.prepare("fp8")
    torch.cuda.synchronize()
    x, logits, w1, w2 = _inputs(300, 512, 1024, 8, 21, dtype)
    xd, w1d, w2d, ld = x.cuda(), w1.cuda(), w2.cuda(), logits.cuda()
    ref = oracle.fused_moe(x, w1, w2, logits, 2, True)
    base = fused_moe(xd, w1d, w2d, ld, 2, True)
    _assert_close(base, ref, dtype, "library plan")
    try:
        for kw in ({"block": 16}, {"block": 32, "split_k": 3}, {"block": 64, "group_m": 1}, {"block": 128, "split_k": 2},
                   {"block": 256, "no_tail_split": True}, {"block": 256, "group_m": 3}, {"split_k": 4}, {"group_m": 64},
                   {"block": 160}, {"block": 160, "split_k": 2}):
            _say(f"tunables {kw}")
            with fr.tunables(**kw):
                out = fused_moe(xd, w1d, w2d, ld, 2, True)
            torch.cuda.synchronize()
            _assert_close(out, ref, dtype, f"tunables {kw}")
            assert (out.float() - base.float()).abs().max() <= 2.0 ** -7 * ref.abs().max()
    finally:
        fr.reset_tunables()
    assert torch.equal(fused_moe(xd, w1d, w2d, ld, 2, True), base)


@pytest.mark.parametrize("block,kind", [(128, "bf16"), (160, "bf16"), (256, "bf16"), (128, "fp8"), (160, "fp8"), (256, "fp8")])
def test_persistent_tiles_alternating_half_empty_and_full_blocks(native, block, kind):
    """The persistent 128-, 160- and 256-row kernels let the wavefronts of a block's upper half skip their fragment
    reads and MFMAs when that half holds only padding, and pick the fragments up again when their next block
    has rows.  64 experts with one routing block each, a seeded mix of full blocks and blocks filled to less
    than half, 8 feature tiles per block: every workgroup walks several units and meets both transitions."""
    import fast_route_amd as fr
    from fast_route_amd import fused_experts, fused_moe_fp8, prepare_weights_fp8
    E, H, Fd = 64, 512, 1024
    if (block, kind) == (160, "fp8"):
        H = 1024  # that tile has no plain form: five K tiles of 128 bytes per K slice at least
    rng = np.random.default_rng(block)
    counts = np.where(rng.random(E) < 0.5, block, rng.integers(1, block // 2 + 1, E))
    ids = torch.from_numpy(np.repeat(np.arange(E), counts)).int()
    ids = ids[torch.from_numpy(rng.permutation(ids.numel()))].view(-1, 1)
    M = ids.shape[0]
    _say(f"persistent half/full blocks block={block} {kind} M={M}")
    x, _, w1, w2 = _inputs(M, H, Fd, E, 31 + block, torch.bfloat16)
    try:
        with fr.tunables(block=block):
            if kind == "bf16":
                wts = torch.rand(M, 1) + 0.5
                out = fused_experts(x.cuda(), w1.cuda(), w2.cuda(), wts.cuda(), ids.cuda())
                torch.cuda.synchronize()
                _assert_close(out, oracle.moe_experts(x, w1, w2, wts, ids), torch.bfloat16, "half/full blocks")
            else:
                logits = torch.full((M, E), -20.0)
                logits[torch.arange(M), ids.view(-1).long()] = 20.0
                w1q, w1s, w2q, w2s = prepare_weights_fp8(w1.cuda(), w2.cuda())
                out = fused_moe_fp8(x.cuda(), w1q, w1s, w2q, w2s, logits.cuda(), 1, True)
                torch.cuda.synchronize()
                ref, _ = oracle.fused_moe_fp8(x, w1, w2, logits, 1, True)
                o = out.float().cpu()
                assert torch.isfinite(o).all()
                assert (o - ref).norm() / ref.norm() <= 1e-2 and (o - ref).abs().max() <= 2.0 ** -5 * ref.abs().max()
    finally:
        fr.reset_tunables()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_one_wavefront_per_simd_tile_equals_the_eight_wavefront_tile(native, dtype):
    """256-row blocks with 16 K tiles or more run on four wavefronts of 128 x 128 outputs (moe_gemm_quad_kernel);
    the no_quad knob sends the same call to the eight-wavefront kernel.  Same MFMA shape and K order: outputs equal
    bit for bit, and both match the oracle.  64 experts with a seeded mix of full, under-half and over-half blocks,
    16 / 8 feature tiles: every workgroup walks several units (hand-over of the ring), meets all-padding halves,
    and the last round of tiles is split along K (32 K tiles in the gate/up GEMM)."""
    import fast_route_amd as fr
    from fast_route_amd import fused_experts, fused_moe
    E, H, Fd = 64, 2048, 2048
    rng = np.random.default_rng(5)
    counts = np.where(rng.random(E) < 0.4, 256, rng.integers(1, 200, E))
    ids = torch.from_numpy(np.repeat(np.arange(E), counts)).int()
    ids = ids[torch.from_numpy(rng.permutation(ids.numel()))].view(-1, 1)
    M = ids.shape[0]
    _say(f"quad tile vs eight-wavefront tile {dtype} M={M}")
    x, _, w1, w2 = _inputs(M, H, Fd, E, 77, dtype)
    wts = torch.rand(M, 1) + 0.5
    xd, w1d, w2d, wd, idd = x.cuda(), w1.cuda(), w2.cuda(), wts.cuda(), ids.cuda()
    try:
        with fr.tunables(block=256):
            quad = fused_experts(xd, w1d, w2d, wd, idd)
        with fr.tunables(block=256, no_quad=True):
            eight = fused_experts(xd, w1d, w2d, wd, idd)
        with fr.tunables(block=256, no_tail_split=True):
            whole = fused_experts(xd, w1d, w2d, wd, idd)
        torch.cuda.synchronize()
        assert torch.equal(quad, eight), "the two 256-row kernels differ"
        _assert_close(quad, oracle.moe_experts(x, w1, w2, wts, ids), dtype, "quad tile, experts only")
        _assert_close(whole, oracle.moe_experts(x, w1, w2, wts, ids), dtype, "quad tile, no tail split")
        # the layer with gating: top-2 of 8 experts, token rows gathered by sorted id, padding rows not fetched
        x2, logits, w1b, w2b = _inputs(1500, 1024, 1024, 8, 78, dtype)
        with fr.tunables(block=256):
            a = fused_moe(x2.cuda(), w1b.cuda(), w2b.cuda(), logits.cuda(), 2, True)
        with fr.tunables(block=256, no_quad=True):
            b = fused_moe(x2.cuda(), w1b.cuda(), w2b.cuda(), logits.cuda(), 2, True)
        torch.cuda.synchronize()
        assert torch.equal(a, b), "the two 256-row kernels differ (layer with gating)"
        _assert_close(a, oracle.fused_moe(x2, w1b, w2b, logits, 2, True), dtype, "quad tile, layer")
        # widths that are no multiples of 256: 18 and 22 K tiles, the down projection's last feature tile half wide;
        # three experts, one of them without a token
        x3, logits3, w1c, w2c = _inputs(900, 1152, 1408, 3, 79, dtype)
        logits3[:, 1] = -30.0
        with fr.tunables(block=256):
            c = fused_moe(x3.cuda(), w1c.cuda(), w2c.cuda(), logits3.cuda(), 2, True)
        with fr.tunables(block=256, no_quad=True):
            d = fused_moe(x3.cuda(), w1c.cuda(), w2c.cuda(), logits3.cuda(), 2, True)
        torch.cuda.synchronize()
        assert torch.equal(c, d), "the two 256-row kernels differ (odd widths)"
        _assert_close(c, oracle.fused_moe(x3, w1c, w2c, logits3, 2, True), dtype, "quad tile, odd widths")
    finally:
        fr.reset_tunables()


@pytest.mark.parametrize("E,k,H", [(8, 2, 4096), (64, 6, 4096), (100, 3, 4096), (256, 8, 4096), (4, 4, 4096), (16, 1, 4096),
                                   (64, 6, 2048), (8, 2, 3072), (16, 4, 2560)])
@pytest.mark.parametrize("ldtype", [torch.float32, torch.bfloat16])
def test_decode_layer_routes_inside_the_gate_up_launch(native, E, k, H, ldtype):
    """Up to 4 tokens with H >= 2048: fused_moe's gate/up launch gates the tokens and sorts the pairs itself.
    Its result must equal, bit for bit, the experts-only entry point fed with the gating kernel's weights and ids
    (the same gating core, the same routing order), and match the oracle; exact ties in the logits included."""
    from fast_route_amd import fused_moe, fused_experts
    from fast_route_amd.ops.stable_route import topk_softmax
    Fd, dtype = 256, torch.bfloat16
    _, _, w1, w2 = _inputs(1, H, Fd, E, 9, dtype)
    w1d, w2d = w1.cuda(), w2.cuda()
    for M in (1, 2, 3, 4):
        if M * k > 32:
            continue
        for renorm in (True, False):
            _say(f"routed decode E={E} k={k} H={H} {ldtype} M={M} renorm={renorm}")
            g = torch.Generator().manual_seed(E * 100 + k * 10 + M)
            x = torch.randn(M, H, generator=g).to(dtype)
            logits = torch.randn(M, E, generator=g).to(ldtype)
            if E >= 4:
                logits[0, : min(E, 5)] = logits[0, 0]  # a run of equal logits: lower index first
            out = fused_moe(x.cuda(), w1d, w2d, logits.cuda(), k, renorm)
            torch.cuda.synchronize()
            w = torch.empty((M, k), dtype=torch.float32, device="cuda")
            ids = torch.empty((M, k), dtype=torch.int32, device="cuda")
            topk_softmax(w, ids, None, logits.cuda(), renormalize=renorm)
            ow, oid = oracle.gating_topk(logits, k, renorm)
            assert torch.equal(ids.cpu(), oid)
            same = fused_experts(x.cuda(), w1d, w2d, w, ids)
            assert torch.equal(out, same), "routing inside the gate/up launch differs from the routing kernels"
            _assert_close(out, oracle.fused_moe(x, w1, w2, logits, k, renorm), dtype, f"routed decode M={M}")


def test_random_shapes_against_oracle(native):
    """Forty seeded random layer shapes (token count, widths, expert count, top-k, dtype, renormalisation)
    against the oracle: every plan boundary gets neighbours on both sides sooner or later."""
    from fast_route_amd import fused_moe
    rng = np.random.default_rng(20240607)
    for case in range(40):
        E = int(rng.choice([1, 2, 3, 4, 8, 16, 60, 64]))
        k = int(rng.integers(1, min(E, 8) + 1))
        H = int(rng.choice([128, 256, 384, 512, 1024, 2048, 3072, 4096]))
        Fd = int(rng.choice([128, 256, 384, 640]))
        M = int(rng.choice([1, 2, 3, 4, 5, 7, 17, 33, 100, 257, 600]) if rng.random() < 0.7 else rng.integers(1, 700))
        dtype = torch.bfloat16 if rng.random() < 0.7 else torch.float16
        renorm = bool(rng.random() < 0.7)
        _say(f"random case {case}: M={M} H={H} F={Fd} E={E} k={k} {dtype} renorm={renorm}")
        x, logits, w1, w2 = _inputs(M, H, Fd, E, 1000 + case, dtype, zipf=bool(rng.random() < 0.3))
        out = fused_moe(x.cuda(), w1.cuda(), w2.cuda(), logits.cuda(), k, renorm)
        torch.cuda.synchronize()
        _assert_close(out, oracle.fused_moe(x, w1, w2, logits, k, renorm), dtype, f"random case {case}")


@pytest.mark.parametrize("M,E,k,H,Fd", [(2, 8, 2, 512, 4096), (3, 8, 2, 512, 1024), (300, 8, 2, 512, 1024), (700, 8, 2, 512, 1024),
                                        (200, 64, 6, 512, 384)])
def test_out_of_range_expert_ids_are_dropped_pairs(native, M, E, k, H, Fd):
    """Expert ids outside [0, E) (masked pairs of an expert-parallel caller) get no slot in the routing arrays
    and contribute nothing: the oracle's per-expert masks never match them either (perf_test_moe.py:22-27).
    Covers the decode kernels, the combine in the GEMM epilogue (top-2) and the combine kernel (top-6);
    with every pair masked the output is exactly zero."""
    from fast_route_amd import fused_experts
    dtype = torch.bfloat16
    _say(f"masked ids M={M} E={E} k={k}")
    x, logits, w1, w2 = _inputs(M, H, Fd, E, 31, dtype)
    tw, ti = oracle.gating_topk(logits, k, True)
    g = torch.Generator().manual_seed(M)
    drop = torch.rand(M, k, generator=g) < 0.3
    ti = ti.clone()
    ti[drop] = torch.where(torch.rand(int(drop.sum()), generator=g) < 0.5, -1, E + 3).int()
    xd, w1d, w2d = x.cuda(), w1.cuda(), w2.cuda()
    out = fused_experts(xd, w1d, w2d, tw.cuda(), ti.cuda())
    torch.cuda.synchronize()
    _assert_close(out, oracle.moe_experts(x, w1, w2, tw, ti), dtype, f"masked ids M={M}")
    none = torch.full_like(ti, -1)
    out0 = fused_experts(xd, w1d, w2d, tw.cuda(), none.cuda())
    torch.cuda.synchronize()
    assert torch.count_nonzero(out0) == 0, "all pairs masked: output must be zero"


@pytest.mark.parametrize("E", [8, 100, 256])
@pytest.mark.parametrize("M", [3, 40])
def test_nan_logit_rows_do_not_reach_the_weights(native, E, M):
    """A token whose router logits are all NaN has no valid expert (with more than 64 experts the gating core
    leaves an id outside [0, E) behind): its pairs are dropped by the routing - also by the routing done inside
    the decode gate/up launch - instead of indexing the weights, and the other tokens are unaffected."""
    from fast_route_amd import fused_moe
    dtype = torch.bfloat16
    _say(f"NaN logits E={E} M={M}")
    x, logits, w1, w2 = _inputs(M, 2048, 256, E, 13, dtype)
    logits = logits.clone()
    logits[1, :] = float("nan")
    out = fused_moe(x.cuda(), w1.cuda(), w2.cuda(), logits.cuda(), 2, True)
    torch.cuda.synchronize()
    keep = [m for m in range(M) if m != 1]
    ref = oracle.fused_moe(x[keep], w1, w2, logits[keep], 2, True)
    _assert_close(out[keep], ref, dtype, f"NaN logits E={E}")
    if E > 64:
        assert torch.count_nonzero(out[1]) == 0


@pytest.mark.parametrize("M", [40, 300, 3000])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_top2_combine_in_the_epilogue_is_deterministic(native, M, dtype):
    """The epilogue_combine knob: top-2 layers add the two weighted rows of a token into a zero-filled output
    with packed atomics.  The result may not depend on which pair arrives first: same bits on every run, also
    in place, and the same bits as the combine kernel forms from the same two rounded rows."""
    import fast_route_amd as fr
    from fast_route_amd import fused_moe
    _say(f"top-2 epilogue combine M={M} {dtype}")
    x, logits, w1, w2 = _inputs(M, 512, 1024, 8, 17, dtype)
    xd, w1d, w2d, ld = x.cuda(), w1.cuda(), w2.cuda(), logits.cuda()
    with fr.tunables(split_k=1):
        by_kernel = fused_moe(xd, w1d, w2d, ld, 2, True)
    with fr.tunables(split_k=1, epilogue_combine=True):
        first = fused_moe(xd, w1d, w2d, ld, 2, True)
        for _ in range(4):
            assert torch.equal(fused_moe(xd, w1d, w2d, ld, 2, True), first)
        xin = xd.clone()
        assert torch.equal(fused_moe(xin, w1d, w2d, ld, 2, True, inplace=True), first)
    torch.cuda.synchronize()
    _assert_close(first, oracle.fused_moe(x, w1, w2, logits, 2, True), dtype, f"top-2 M={M}")
    assert torch.equal(first, by_kernel), "epilogue combine and combine kernel round differently"


_FIRST_CALL_CAPTURE = r'''
import sys
sys.path.insert(0, sys.argv[1])
import torch
import fast_route_amd as fr
from fast_route_amd import _native as N
from fast_route_amd.layers.fused_moe import plan

dtype, lib = torch.bfloat16, N.lib()
fr.prepare(dtype)                      # every kernel set up, the no-alloc scratch resolved: nothing left to do lazily
gen = torch.Generator().manual_seed(9)
cases = []
for M, H, Fd, E, k in ((2, 4096, 512, 4, 2), (16, 1024, 2048, 4, 2), (1536, 1024, 2048, 4, 2)):
    x = torch.randn(M, H, generator=gen).to(dtype).cuda()
    logits = torch.randn(M, E, generator=gen).cuda()
    w1 = (torch.randn(E, 2 * Fd, H, generator=gen) * 0.02).to(dtype).cuda()
    w2 = (torch.randn(E, H, Fd, generator=gen) * 0.02).to(dtype).cuda()
    p = plan(M, H, Fd, E, k, dtype)
    ws = torch.empty(max(p.workspace_bytes, 256), dtype=torch.uint8, device="cuda")
    out, out_na = torch.zeros(M, H, dtype=dtype, device="cuda"), torch.zeros(M, H, dtype=dtype, device="cuda")
    na = p.workspace_bytes <= (64 << 20)

    def call(stream, x=x, w1=w1, w2=w2, logits=logits, M=M, H=H, Fd=Fd, E=E, k=k, out=out, out_na=out_na, ws=ws, na=na):
        N.check(lib.fr_fused_moe(x.data_ptr(), w1.data_ptr(), w2.data_ptr(), logits.data_ptr(), N.FR_F32, M, H, Fd, E, k, 1,
                                 N.FR_BF16, out.data_ptr(), ws.data_ptr(), ws.numel(), stream))
        if na:
            N.check(lib.fr_fused_moe_noalloc(x.data_ptr(), w1.data_ptr(), w2.data_ptr(), logits.data_ptr(), N.FR_F32, M, H, Fd,
                                             E, k, 1, N.FR_BF16, out_na.data_ptr(), stream))
    cases.append((M, call, out, out_na, na))
torch.cuda.synchronize()
graphs = []
for M, call, out, out_na, na in cases:  # the captured calls are this process's first launches of these kernels
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        call(torch.cuda.current_stream().cuda_stream)
    graphs.append(g)
for (M, call, out, out_na, na), g in zip(cases, graphs):
    for rep in range(2):
        out.zero_(); out_na.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        got, got_na = out.clone(), out_na.clone()
        out.zero_(); out_na.zero_()
        call(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        assert torch.count_nonzero(got) > 0
        assert torch.equal(got, out), "M=%d replay %d: captured first call differs from the eager call" % (M, rep)
        if na:
            assert torch.equal(got_na, out_na) and torch.equal(got_na, got), "M=%d: no-alloc entry under capture" % M
print("FIRST-CALL-CAPTURE-OK")
'''


def test_first_call_under_graph_capture_after_prepare(native):
    """What fr_moe_prepare exists for: in a fresh process, after fr_moe_prepare and nothing else, the whole layer -
    through fr_fused_moe and through fr_fused_moe_noalloc - is captured as the process's FIRST launch of its
    kernels (weight-row decode kernels, decode tiles with the fused route+align launch, persistent tiles with
    their last-round split) and replays to the bits of the eager calls made afterwards."""
    import os
    import subprocess
    _say("first call captured after fr_moe_prepare (fresh process)")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, "-c", _FIRST_CALL_CAPTURE, root], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                          text=True, timeout=110)
    assert proc.returncode == 0 and "FIRST-CALL-CAPTURE-OK" in proc.stdout, proc.stdout[-3000:]
