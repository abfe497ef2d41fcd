import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle_mod():
    import oracle
    oracle.lib()
    return oracle


@pytest.fixture(autouse=True)
def guarded_tensor_allocations(request):
    """Every distconv-style tensor a GPU test allocates lies between two guard zones of a known
    byte pattern, and the zones are checked when the test ends: a kernel that stores in front of
    or behind a tensor's allocation fails the test that ran it, whatever that test compares."""
    if request.node.get_closest_marker("gpu") is None:
        yield
        return
    import helpers
    with helpers.guarded_allocations() as allocated:
        yield allocated
    helpers.check_guards(allocated)
