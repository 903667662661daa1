"""Same import path as the reference's fast_route/fast_route/ops/stable_route.py."""
from fast_route_amd.ops.stable_route import fused_route  # noqa: F401
