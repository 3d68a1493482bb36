import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import fbw_oracle
    fbw_oracle.build()
    return fbw_oracle


@pytest.fixture(autouse=True)
def no_status_left_behind(request):
    """Device-side problems are reported by a later call by default; a test that provokes one must not
    hand it to the next test."""
    yield
    if request.node.get_closest_marker("gpu") is None:
        return
    from i6_native_ops_amd import cabi
    cabi.poll_status(wait=True)
    cabi.load().i6fbw_set_status_mode(2)
