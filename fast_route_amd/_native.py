"""ctypes binding of libfast_route_hip.so (the C ABI in include/fast_route_hip.h)."""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_int, c_int32, c_int64, c_void_p

HERE = os.path.dirname(os.path.abspath(__file__))
# FR_NATIVE_LIB: another build of the library (a measurement build, see build.py); bench.py records which one ran
LIB_PATH = os.environ.get("FR_NATIVE_LIB") or os.path.join(HERE, "libfast_route_hip.so")

FR_F16, FR_BF16, FR_F32, FR_FP8_E4M3, FR_I32, FR_I64 = range(6)
FR_W1_TILED, FR_W2_TILED, FR_W_TILED = 0x100, 0x200, 0x300  # OR-ed into a dtype argument: w1 / w2 / both are in the layout of fr_moe_prepare_weights

_SHAPE_ERRORS = (-1, -2, -3, -4, -5)  # argument errors -> AssertionError like the reference's asserts


class FrMoePlan(ctypes.Structure):
    _fields_ = [("block", c_int32), ("split_k", c_int32), ("sorted_len", c_int64),
                ("workspace_bytes", c_int64), ("tail_bytes", c_int64)]


class FrMoeTunables(ctypes.Structure):
    _fields_ = [("block", c_int32), ("split_k", c_int32), ("group_m", c_int32), ("no_tail_split", c_int32),
                ("epilogue_combine", c_int32), ("no_quad", c_int32)]


# name -> (restype, argtypes); must list every symbol the header declares
SIGNATURES = {
    "fr_version": (c_int, []),
    "fr_last_error_string": (c_char_p, []),
    "fr_gating_topk": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "fr_route_gate": (c_int, [c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "fr_moe_align_workspace_bytes": (c_int64, [c_int64, c_int]),
    "fr_moe_align": (c_int, [c_void_p, c_int, c_int64, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "fr_moe_grouped_gemm": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                    c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "fr_moe_prepare": (c_int, [c_int]),
    "fr_moe_prepare_weights": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_void_p]),
    "fr_moe_set_tunables": (c_int, [ctypes.POINTER(FrMoeTunables)]),
    "fr_moe_get_tunables": (c_int, [ctypes.POINTER(FrMoeTunables)]),
    "fr_moe_get_plan": (c_int, [c_int64, c_int64, c_int64, c_int, c_int, c_int, ctypes.POINTER(FrMoePlan)]),
    "fr_moe_gateup_silu": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                   c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "fr_moe_down_combine": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                    c_int64, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "fr_fused_experts": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                 c_int, c_int, c_int, c_void_p, c_void_p, c_int64, c_void_p]),
    "fr_quant_e4m3_rows": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p]),
    "fr_moe_gateup_silu_fp8": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
                                       c_int64, c_int64, c_int, c_int, c_int, c_void_p, c_void_p]),
    "fr_moe_down_combine_fp8": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                        c_int64, c_int64, c_int64, c_int, c_int, c_int, c_int, c_int, c_void_p,
                                        c_void_p, c_void_p, c_void_p]),
    "fr_fused_moe_fp8": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64,
                                 c_int64, c_int64, c_int, c_int, c_int, c_void_p, c_void_p, c_int64, c_void_p]),
    "fr_fused_moe_noalloc": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int, c_int,
                                     c_int, c_int, c_void_p, c_void_p]),
    "fr_probe_mfma_stream": (c_int, [c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "fr_fused_moe": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int, c_int,
                             c_int, c_int, c_void_p, c_void_p, c_int64, c_void_p]),
}

_lib = None


def lib() -> ctypes.CDLL:
    """Loads the native library once.  Raises if it has not been built: there is
    no fallback path."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "fast_route_amd: %s is missing; build it with `python -m fast_route_amd.build`" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        _lib = handle
    return _lib


def check(rc: int) -> None:
    """Maps a negative return code to the exception the reference would raise."""
    if rc == 0:
        return
    msg = lib().fr_last_error_string().decode()
    if rc in _SHAPE_ERRORS:
        raise AssertionError(msg)
    raise RuntimeError("fast_route_amd native error %d: %s" % (rc, msg))


def dtype_code(dt) -> int:
    import torch
    table = {torch.float16: FR_F16, torch.bfloat16: FR_BF16, torch.float32: FR_F32,
             torch.int32: FR_I32, torch.int64: FR_I64}
    if dt not in table:
        raise AssertionError("unsupported dtype %s" % dt)
    return table[dt]


def stream_ptr(device) -> int:
    import torch
    return torch.cuda.current_stream(device).cuda_stream


def require_cuda(*tensors) -> None:
    for t in tensors:
        assert t.is_cuda, "fast_route_amd operators need tensors on an MI355X device (no CPU path)"
