"""CPU-only: the C-ABI library loads and exports every symbol the header declares."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "fast_route_hip.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fr_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_expected_entry_points():
    names = _declared()
    for must in ("fr_gating_topk", "fr_moe_align", "fr_moe_grouped_gemm", "fr_moe_gateup_silu",
                 "fr_moe_down_combine", "fr_fused_moe", "fr_fused_experts", "fr_route_gate"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from fast_route_amd import _native
    if not os.path.exists(_native.LIB_PATH):
        pytest.fail("libfast_route_hip.so not built: run `python -m fast_route_amd.build`")
    handle = ctypes.CDLL(_native.LIB_PATH)
    for name in _declared():
        assert hasattr(handle, name), "missing export %s" % name
    # the ctypes table covers the header exactly
    assert sorted(_native.SIGNATURES) == _declared()


def test_host_only_calls_need_no_gpu():
    from fast_route_amd import _native
    lib = _native.lib()
    assert lib.fr_version() >= 100
    assert lib.fr_moe_align_workspace_bytes(128, 8) == 0
    assert lib.fr_moe_align_workspace_bytes(393216, 64) > 0
    assert lib.fr_moe_align_workspace_bytes(10, 5000) == -1
    p = _native.FrMoePlan()
    assert lib.fr_moe_get_plan(64, 4096, 14336, 8, 2, _native.FR_BF16, p) == 0
    assert p.block in (16, 32, 64, 128, 160, 256) and p.split_k >= 1
    assert p.sorted_len == 128 + 8 * (p.block - 1) and p.workspace_bytes > 0
    # argument errors come back as codes + message, never as aborts
    assert lib.fr_moe_get_plan(64, 4095, 14336, 8, 2, _native.FR_BF16, p) == -2
    assert b"multiples of 128" in lib.fr_last_error_string()
    with pytest.raises(AssertionError):
        _native.check(-2)
    assert lib.fr_gating_topk(None, _native.FR_F32, 4, 8, 8, 2, 1, None, None, None) == -1
    assert lib.fr_gating_topk(None, _native.FR_F32, 0, 8, 8, 2, 1, None, None, None) == 0


def test_plan_table():
    """The tile plan is host logic: routing block and K slices of the down projection per token count,
    as documented (Mixtral shape: 16-row blocks up to 8 pairs per expert, 32 below 26, 64 below 52 at
    H >= 4096, then 128 or - where the spread of the experts' loads around a multiple of 128 would cost
    every other expert one block more - 160; 2-byte operands take 256 rows (one wavefront per SIMD) from 350 pairs
    per expert on wherever their coarser blocks add less than 8 % of rows, 256 from 1200 pairs on otherwise; fp8 takes 160 rows only where
    a sixth of the blocks go and 256 from 900 on; the fine-grained shape with H = 2048 has no 64-row range and takes
    256 rows from 700 pairs per expert on)."""
    from fast_route_amd import _native
    lib = _native.lib()

    def plan(M, H, F, E, k, dt=_native.FR_BF16):
        p = _native.FrMoePlan()
        assert lib.fr_moe_get_plan(M, H, F, E, k, dt, p) == 0
        assert p.sorted_len == M * k + E * (p.block - 1)
        return p.block, p.split_k

    mix = lambda M, dt=_native.FR_BF16: plan(M, 4096, 14336, 8, 2, dt)
    assert [mix(M)[0] for M in (1, 32, 33, 103, 104, 207, 208, 469, 470, 670, 671, 768, 1024, 1280, 1400, 1536, 2048, 2304, 2560,
                               4096, 4800)] == \
        [16, 16, 32, 32, 64, 64, 128, 128, 160, 160, 128, 128, 160, 160, 128, 256, 256, 160, 256, 256, 256]
    import fast_route_amd as fr
    try:  # without the one-wavefront-per-SIMD kernel the 256-row tile takes over at 1200 pairs per expert
        with fr.tunables(no_quad=True):
            assert [mix(M)[0] for M in (1536, 2048, 4096, 4799, 4800)] == [160, 128, 160, 160, 256]
    finally:
        fr.reset_tunables()
    assert mix(1) == (16, 4) and mix(2) == (16, 2) and mix(3) == (16, 4) and mix(4) == (16, 4) and mix(16) == (16, 1)
    assert mix(128) == (64, 2)
    assert mix(4096)[1] == 1 and plan(16384, 4096, 14336, 8, 2)[0] == 256
    assert [mix(M, _native.FR_FP8_E4M3)[0] for M in (103, 104, 207, 208, 512, 768, 1024, 1200, 1280, 2048, 2304, 2560, 4096)] == \
        [32, 64, 64, 128, 160, 128, 160, 160, 256, 256, 256, 256, 256]
    fine = lambda M: plan(M, 2048, 1408, 64, 6)[0]
    assert [fine(M) for M in (85, 86, 341, 342, 1246, 1247, 7466, 7467, 43691)] == [16, 32, 32, 128, 128, 160, 160, 256, 256]
    # the scratch for splitting the last round exists exactly for 128- and 256-row blocks with a long K
    p = _native.FrMoePlan()
    lib.fr_moe_get_plan(4096, 4096, 14336, 8, 2, _native.FR_BF16, p)
    assert p.tail_bytes == 256 * 256 * 256 * 4
    lib.fr_moe_get_plan(16, 4096, 14336, 8, 2, _native.FR_BF16, p)
    assert p.tail_bytes == 0


def test_plan_invariants_on_random_shapes():
    """Whatever the shape, a plan is one the entry points can run: a routing block the kernels have, sorted_len as
    moe_align_block_size lays it out (`ops/fused_moe.py:133-175` of the reference: n + E * (block - 1) slots), at least
    one K slice and never more than the down projection has 128-byte K tiles, a workspace that holds the activated
    rows and the routing arrays, the same answer whatever the weight layout flags, and shape errors as codes."""
    import random
    from fast_route_amd import _native
    lib = _native.lib()
    rng = random.Random(20240229)
    p, q = _native.FrMoePlan(), _native.FrMoePlan()
    for case in range(600):
        dt = rng.choice([_native.FR_BF16, _native.FR_F16, _native.FR_FP8_E4M3])
        mult = 256 if dt == _native.FR_FP8_E4M3 else 128
        H, F = mult * rng.randint(1, 64), mult * rng.randint(1, 128)
        E = rng.choice([1, 2, 3, 8, 16, 60, 64, 128, 256, 1022, 1024])
        k = rng.randint(1, min(E, 8))
        M = rng.choice([0, 1, 2, 4, 5, 16, 100, 1000, 5000, 40000, 300000, rng.randint(1, 1 << 20)])
        where = "case %d: M=%d H=%d F=%d E=%d k=%d dtype=%d" % (case, M, H, F, E, k, dt)
        assert lib.fr_moe_get_plan(M, H, F, E, k, dt, p) == 0, where
        n, es = M * k, 1 if dt == _native.FR_FP8_E4M3 else 2
        assert p.block in (16, 32, 64, 128, 160, 256), where
        assert p.sorted_len == n + E * (p.block - 1), where
        assert 1 <= p.split_k <= max(1, F * es // 128), where
        assert 0 <= p.tail_bytes <= p.workspace_bytes, where
        assert p.workspace_bytes >= p.sorted_len * F * es + 4 * (p.sorted_len + n + E), where
        assert lib.fr_moe_get_plan(M, H, F, E, k, dt | _native.FR_W_TILED, q) == 0, where
        assert (q.block, q.split_k, q.workspace_bytes) == (p.block, p.split_k, p.workspace_bytes), where
        assert lib.fr_moe_get_plan(M, H + 64, F, E, k, dt, q) == -2, where
        assert lib.fr_moe_get_plan(M, H, F, E, E + 1, dt, q) == -2, where
    assert lib.fr_moe_get_plan(1 << 30, 4096, 14336, 8, 2, _native.FR_BF16, p) == -2
    assert lib.fr_moe_get_plan(16, 4096, 14336, 1025, 2, _native.FR_BF16, p) == -2


def test_ops_refuse_cpu_tensors():
    import torch
    from fast_route_amd.ops.fused_moe import moe_align_block_size
    with pytest.raises(AssertionError):
        moe_align_block_size(torch.zeros(4, 2, dtype=torch.int32), 16, 8)


def test_reference_import_paths_resolve():
    """The reference's module paths (fast_route.layers.*, fast_route.ops.*) import here."""
    from fast_route.layers.stable_route import fused_moe as a
    from fast_route.layers.vllm_route import fused_moe as b
    from fast_route.layers.profile_fused_route import fused_moe as c
    from fast_route.ops.stable_route import fused_route
    from fast_route.ops.fused_moe import invoke_fused_moe_kernel, moe_align_block_size
    import inspect
    assert list(inspect.signature(a).parameters) == ["hidden_states", "gate", "w1", "w2", "topk", "renormalize", "inplace"]
    assert list(inspect.signature(b).parameters) == ["hidden_states", "gate", "w1", "w2", "topk", "renormalize", "inplace"]
    assert list(inspect.signature(c).parameters)[:7] == ["hidden_states", "gate", "w1", "w2", "topk", "renormalize", "inplace"]
    assert list(inspect.signature(fused_route).parameters) == ["hidden_state", "gate", "topk", "topk_weights", "topk_ids", "renormalize"]
    assert list(inspect.signature(moe_align_block_size).parameters) == ["topk_ids", "block_size", "num_experts"]
    assert list(inspect.signature(invoke_fused_moe_kernel).parameters)[:4] == ["A", "B", "C", "topk_weights"]


def test_bench_refuses_more_than_one_gpu():
    """bench.py is single-GPU: any other --gpus value exits with a message that says so."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0
    assert "single-GPU" in r.stderr


def test_recorded_traffic_matches_profiles_file():
    """bench.py reports roofline.traffic from profiles/hbm_traffic.json for the workloads recorded there,
    as long as the grouped-GEMM kernel sources are the ones the record was measured with and the plan still
    picks the routing block (the tile) that was measured."""
    import importlib.util
    import json
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("bench_mod", os.path.join(root, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    rec = json.load(open(os.path.join(root, "profiles", "hbm_traffic.json")))
    key = "moe_layer_tflops_mixtral_bf16_M4096"
    assert rec[key]["traffic_bytes"] == rec[key]["fetch_bytes"] + rec[key]["write_bytes"]
    # the record counts only for the kernel sources it was measured with
    block = rec[key]["block"]
    want = rec[key]["traffic_bytes"] if rec.get("kernel_sources_sha") == mod.kernel_sources_sha() else None
    assert mod.recorded_traffic(key, block) == want
    assert mod.recorded_traffic(key, block + 1) is None
    assert mod.recorded_traffic("no_such_workload", block) is None


def test_tunables_override_the_plan_and_reset():
    """fr_moe_set_tunables is host logic: the plan follows the overrides, rejects values outside its ranges,
    and NULL restores the library's own choices."""
    import fast_route_amd as fr
    from fast_route_amd import _native
    lib = _native.lib()

    def plan(M):
        p = _native.FrMoePlan()
        assert lib.fr_moe_get_plan(M, 4096, 14336, 8, 2, _native.FR_BF16, p) == 0
        return p

    base = plan(4096)
    assert (base.block, base.split_k) == (256, 1) and base.tail_bytes > 0
    try:
        fr.set_tunables(block=128, split_k=3)
        p = plan(4096)
        assert (p.block, p.split_k) == (128, 3) and p.sorted_len == 8192 + 8 * 127
        assert fr.get_tunables() == {"block": 128, "split_k": 3, "group_m": 0, "no_tail_split": False, "epilogue_combine": False, "no_quad": False}
        with fr.tunables(no_tail_split=True):
            assert plan(4096).tail_bytes == 0 and plan(4096).block == 256  # the context replaces, then restores
        assert plan(4096).block == 128
        fr.set_tunables(split_k=64)  # as many slices as keep 8 K tiles each: 14336 / (8 * 64) = 28
        assert plan(4096).split_k == 28
        with pytest.raises(AssertionError):
            fr.set_tunables(block=48)
        with pytest.raises(AssertionError):
            fr.set_tunables(group_m=65)
    finally:
        fr.reset_tunables()
    p = plan(4096)
    assert (p.block, p.split_k, p.tail_bytes) == (base.block, base.split_k, base.tail_bytes)
    assert lib.fr_moe_prepare(_native.FR_F32) == -3
