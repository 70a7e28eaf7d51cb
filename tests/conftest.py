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


@pytest.fixture
def knobs(ctx):
    """Sets tuning knobs for one test: knobs(REDUX_FUSED=0) puts
    GPUARRAY_REDUX_FUSED=0 into the environment and has the context read its
    tuning table again (a context reads the environment once, when it is made);
    None removes a knob.  Everything is put back, and read back, afterwards."""
    saved = {}

    def set_knobs(**values):
        for short, value in values.items():
            name = "GPUARRAY_" + short
            saved.setdefault(name, os.environ.get(name))
            if value is None:
                os.environ.pop(name, None)
            else:
                os.environ[name] = str(value)
        ctx.reload_tuning()

    yield set_knobs
    for name, old in saved.items():
        if old is None:
            os.environ.pop(name, None)
        else:
            os.environ[name] = old
    ctx.reload_tuning()
