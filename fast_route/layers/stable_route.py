"""Same import path as the reference's fast_route/fast_route/layers/stable_route.py."""
from fast_route_amd.layers.stable_route import fused_moe  # noqa: F401
