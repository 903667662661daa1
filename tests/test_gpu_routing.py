"""GPU parity: block-aligned routing arrays, bit-exact against the CPU oracle."""
import sys

import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu


def _say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


def _check(ids: torch.Tensor, B: int, E: int):
    from fast_route_amd.ops.fused_moe import moe_align_block_size
    s, e, npost = moe_align_block_size(ids.cuda(), B, E)
    torch.cuda.synchronize()
    rs, re_, rn = oracle.moe_align_block_size(ids, B, E)
    n = ids.numel()
    assert s.shape[0] == n + E * (B - 1) and e.shape[0] == n + E and s.dtype == torch.int32
    npost = int(npost.cpu()[0])
    assert npost == int(rn[0])
    assert np.array_equal(s.cpu().numpy(), rs), "sorted_token_ids differ"  # includes padding and tail == n
    assert np.array_equal(e.cpu().numpy()[: npost // B], re_[: npost // B]), "expert_ids differ"


def test_align_reference_docstring_example(native):
    _say("align docstring example")
    ids = torch.tensor([[2, 3, 4], [1, 2, 4], [1, 3, 4], [1, 2, 3]], dtype=torch.int32)
    from fast_route_amd.ops.fused_moe import moe_align_block_size
    s, e, n = moe_align_block_size(ids.cuda(), 4, 5)
    assert s.cpu()[:16].tolist() == [3, 6, 9, 12, 0, 4, 10, 12, 1, 7, 11, 12, 2, 5, 8, 12]
    assert e.cpu()[:4].tolist() == [1, 2, 3, 4] and n.cpu().tolist() == [16]


@pytest.mark.parametrize("E,k", [(8, 2), (64, 6), (5, 3), (16, 1), (256, 8), (300, 4), (1024, 2)])
@pytest.mark.parametrize("B", [16, 32, 64, 128, 1, 4])
def test_align_small_and_ragged(native, E, k, B):
    for M in (0, 1, 7, 64, 333, 2500):
        _say(f"align E={E} k={k} B={B} M={M}")
        rng = np.random.default_rng(E * 7 + k * 3 + B + M)
        ids = rng.integers(0, E, size=(M, k)).astype(np.int32)
        if M > 3:
            ids[ids == E - 1] = 0  # an empty expert
        _check(torch.from_numpy(ids), B, E)


@pytest.mark.parametrize("dtype", [torch.int32, torch.int64])
def test_align_all_to_one_expert_and_id_dtypes(native, dtype):
    _say(f"align single expert dtype={dtype}")
    ids = torch.full((1000, 2), 3, dtype=dtype)
    _check(ids, 64, 8)
    ids = torch.arange(4000, dtype=dtype).reshape(2000, 2) % 8
    _check(ids, 16, 8)


@pytest.mark.parametrize("B", [16, 32, 64, 128])
def test_align_routing_stress_config(native, B):
    """65536 tokens, 64 experts, top-6, Zipf(1.2)-skewed load: the multi-launch path."""
    _say(f"align stress B={B}")
    logits = oracle.zipf_logits(65536, 64, seed=2024)
    _, ids = oracle.gating_topk(logits, 6)
    counts = torch.bincount(ids.reshape(-1).long(), minlength=64)
    assert counts.max() > 8 * counts.min().clamp(min=1)  # really imbalanced
    _check(ids, B, 64)
    # also through int64 ids and after the GPU's own gating of the same logits
    from fast_route_amd.ops.stable_route import topk_softmax
    w = torch.empty((65536, 6), dtype=torch.float32, device="cuda")
    gi = torch.empty((65536, 6), dtype=torch.int32, device="cuda")
    topk_softmax(w, gi, None, logits.cuda(), renormalize=True)
    assert torch.equal(gi.cpu(), ids)
    _check(ids.long(), B, 64)


def test_align_medium_sizes_cross_path_boundary(native):
    for n_tokens in (1024, 1025, 1365, 1366, 2730, 2731, 8192, 20000):  # 6144 / 6150 pairs straddle the one-workgroup limit
        _say(f"align boundary M={n_tokens}")
        rng = np.random.default_rng(n_tokens)
        ids = rng.integers(0, 64, size=(n_tokens, 6)).astype(np.int32)
        _check(torch.from_numpy(ids), 32, 64)
