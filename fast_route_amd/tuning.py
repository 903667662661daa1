"""Study knobs and set-up of the grouped GEMMs.

The reference's tile study edits per-GEMM config dictionaries by hand
(benchmarks/swizzle_moe/v1_moe_fused.py:311-344: block_m, group_m, split_k);
here the same three are process-wide overrides of the library's plan.
"""
from __future__ import annotations

import contextlib
import ctypes

from . import _native as N


def set_tunables(block: int = 0, split_k: int = 0, group_m: int = 0, no_tail_split: bool = False,
                 epilogue_combine: bool = False, no_quad: bool = False) -> None:
    """0 leaves a choice to the library.  block: routing block / token rows per tile
    (16, 32, 64, 128, 160, 256); split_k: K slices of the down projection; group_m: token blocks
    walked together over the feature tiles; no_tail_split: never split the last round of tiles;
    epilogue_combine: top-2 combine by atomic adds in the down GEMM's epilogue (measured slower than the combine kernel);
    no_quad: 256-row tiles take the eight-wavefront kernel instead of the one-wavefront-per-SIMD one (same results)."""
    t = N.FrMoeTunables(int(block), int(split_k), int(group_m), int(bool(no_tail_split)), int(bool(epilogue_combine)),
                        int(bool(no_quad)))
    N.check(N.lib().fr_moe_set_tunables(ctypes.byref(t)))


def reset_tunables() -> None:
    N.check(N.lib().fr_moe_set_tunables(None))


def get_tunables() -> dict:
    t = N.FrMoeTunables()
    N.check(N.lib().fr_moe_get_tunables(ctypes.byref(t)))
    return {"block": t.block, "split_k": t.split_k, "group_m": t.group_m, "no_tail_split": bool(t.no_tail_split),
            "epilogue_combine": bool(t.epilogue_combine), "no_quad": bool(t.no_quad)}


@contextlib.contextmanager
def tunables(**kw):
    """with tunables(block=128, split_k=2): ...   (restores the previous values on exit)"""
    before = get_tunables()
    set_tunables(**kw)
    try:
        yield
    finally:
        set_tunables(**before)


def prepare(dtype) -> None:
    """Per-device set-up of every grouped-GEMM kernel for torch dtype `dtype` (or "fp8") on the
    current device, e.g. before a first call under graph capture."""
    code = N.FR_FP8_E4M3 if dtype == "fp8" else N.dtype_code(dtype)
    N.check(N.lib().fr_moe_prepare(code))
