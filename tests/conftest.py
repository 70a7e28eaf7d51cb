import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def ctx():
    """One HIP context for the whole GPU session."""
    import libgpuarray_amd as ga
    if ga.count_devices() == 0:
        pytest.skip("no HIP device")
    c = ga.init("hip0")
    ga.set_default_context(c)
    return c


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as O
    return O
