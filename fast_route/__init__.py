"""Import-path compatibility: `fast_route.layers.*` and `fast_route.ops.*` resolve to
the MI355X implementation in `fast_route_amd` so existing callers of the
reference package keep working unchanged."""
