"""MI355X-native fused Mixture-of-Experts layer behind fast-route's entry points.

Host code is PyTorch-ROCm (device memory and streams only); all compute is in
hand-written HIP kernels for gfx950, reached through the C ABI declared in
include/fast_route_hip.h.  There is no CPU or eager fallback: every operator
raises if the native library is missing.
"""
from . import _native  # noqa: F401
from .layers.fused_moe import fused_moe, fused_experts, prepare_weights  # noqa: F401
from .layers.fp8 import fused_moe_fp8, prepare_weights_fp8, quantize_rows_e4m3  # noqa: F401
from .ops.fused_moe import moe_align_block_size, invoke_fused_moe_kernel  # noqa: F401
from .ops.stable_route import fused_route, topk_softmax  # noqa: F401
from .tuning import get_tunables, prepare, reset_tunables, set_tunables, tunables  # noqa: F401

__all__ = [
    "fused_moe",
    "fused_experts",
    "prepare_weights",
    "fused_moe_fp8",
    "prepare_weights_fp8",
    "quantize_rows_e4m3",
    "moe_align_block_size",
    "invoke_fused_moe_kernel",
    "fused_route",
    "topk_softmax",
    "set_tunables",
    "get_tunables",
    "reset_tunables",
    "tunables",
    "prepare",
]
