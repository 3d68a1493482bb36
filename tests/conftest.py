import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_addoption(parser):
    parser.addoption("--runslow", action="store_true", default=False,
                     help="also run the tests marked slow (the packaging test compiles the whole library: minutes)")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu)")
    config.addinivalue_line("markers", "slow: takes minutes on the CPU; runs with --runslow or I6FBW_RUN_SLOW=1")


def pytest_collection_modifyitems(config, items):
    if config.getoption("--runslow") or os.environ.get("I6FBW_RUN_SLOW") == "1":
        return
    skip = pytest.mark.skip(reason="slow: run with --runslow or I6FBW_RUN_SLOW=1")
    for item in items:
        if "slow" in item.keywords:
            item.add_marker(skip)


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
