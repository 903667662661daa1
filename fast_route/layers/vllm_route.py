"""Same import path as the reference's fast_route/fast_route/layers/vllm_route.py."""
from fast_route_amd.layers.vllm_route import fused_moe  # noqa: F401
