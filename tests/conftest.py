import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def native():
    """The loaded C-ABI library; GPU tests fail loudly when it is not built."""
    from fast_route_amd import _native
    return _native.lib()


@pytest.fixture
def rows256():
    """256-row routing blocks for the duration of a test: the plan keeps shapes with a short gate/up K on
    128-row blocks, and the tests of the 256-row tiles' last-round split build their routing for 256."""
    import fast_route_amd as fr
    with fr.tunables(block=256):
        yield
