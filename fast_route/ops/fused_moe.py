"""Same import path as the reference's fast_route/fast_route/ops/fused_moe.py."""
from fast_route_amd.ops.fused_moe import invoke_fused_moe_kernel, moe_align_block_size  # noqa: F401
