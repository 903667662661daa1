"""fr_fused_moe_noalloc (scratch in a device array of the library, no allocation) against
fr_fused_moe with a caller's workspace: bit-identical outputs, two calls in a row, the second
on a smaller input; sizes beyond the static scratch are refused."""
import sys

import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu


def _say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


def _both(N, x, w1, w2, logits, topk):
    M, H = x.shape
    E, F2, _ = w1.shape
    lib, st = N.lib(), torch.cuda.current_stream().cuda_stream
    plan = N.FrMoePlan()
    N.check(lib.fr_moe_get_plan(M, H, F2 // 2, E, topk, N.FR_BF16, plan))
    ws = torch.empty(max(plan.workspace_bytes, 256), dtype=torch.uint8, device="cuda")
    ref = torch.empty_like(x)
    N.check(lib.fr_fused_moe(x.data_ptr(), w1.data_ptr(), w2.data_ptr(), logits.data_ptr(), N.FR_F32, M, H, F2 // 2, E,
                             topk, 1, N.FR_BF16, ref.data_ptr(), ws.data_ptr(), ws.numel(), st))
    out = torch.full_like(x, float("nan"))
    N.check(lib.fr_fused_moe_noalloc(x.data_ptr(), w1.data_ptr(), w2.data_ptr(), logits.data_ptr(), N.FR_F32, M, H,
                                     F2 // 2, E, topk, 1, N.FR_BF16, out.data_ptr(), st))
    torch.cuda.synchronize()
    return out, ref


def test_noalloc_matches_workspace_entry_twice(native):
    from fast_route_amd import _native as N
    H, F, E, topk = 1024, 3584, 8, 2
    _, _, w1, w2 = oracle.make_inputs(1, H, F, E, seed=11)
    w1d, w2d = w1.bfloat16().cuda(), w2.bfloat16().cuda()
    for M in (96, 5):  # the second call is smaller: whatever the first left in the scratch must not matter
        _say(f"noalloc M={M} H={H} F={F} E={E} topk={topk}")
        x, logits, _, _ = oracle.make_inputs(M, H, F, E, seed=100 + M)
        xd, ld = x.bfloat16().cuda(), logits.cuda()
        out, ref = _both(N, xd, w1d, w2d, ld, topk)
        assert torch.equal(out, ref), "no-alloc entry differs from fr_fused_moe (max |d| %g)" % (
            (out.float() - ref.float()).abs().max().item())
        want = oracle.fused_moe(x.bfloat16(), w1.bfloat16(), w2.bfloat16(), logits, topk, True)
        err = (out.float().cpu() - want).abs().max().item()
        assert err <= 2.0 ** -6 * want.abs().max().item(), err


def test_noalloc_rejects_sizes_beyond_its_scratch(native):
    from fast_route_amd import _native as N
    _say("noalloc size limit")
    lib = N.lib()
    # Mixtral shape, 4096 tokens: hundreds of MB of scratch; refused before any pointer is touched
    rc = lib.fr_fused_moe_noalloc(256, 256, 256, 256, N.FR_F32, 4096, 4096, 14336, 8, 2, 1, N.FR_BF16, 256, None)
    assert rc == -5, rc
    assert b"static scratch" in lib.fr_last_error_string()
