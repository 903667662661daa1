"""Same import path as the reference's fast_route/fast_route/layers/profile_fused_route.py."""
from fast_route_amd.layers.profile_fused_route import fused_moe  # noqa: F401
