import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


# The compiler behind hipRTC keeps a cache of the code objects it has made,
# keyed by source text and options (AMD_COMGR_CACHE_DIR; by default under the
# user's home, which need not be writable on a test machine, and the cache is
# then off).  Every kernel of the GPU suite costs 0.25 to 0.6 s to compile, a
# few thousand compilations in all, many of them of the same text (a new
# context or an evicted module compiles again): with the cache in a directory
# of the tree the suite takes about 4.5 minutes instead of 10, and less when
# the directory still holds an earlier run's entries (it is not tracked: like
# the built library it travels with the tree).  It only saves time: a kernel
# whose text has changed is simply compiled.  Set before the library (and with
# it hipRTC) is loaded.
_COMGR_CACHE = os.path.join(os.path.dirname(os.path.abspath(__file__)), ".comgr_cache")
if "AMD_COMGR_CACHE_DIR" not in os.environ:
    try:
        os.makedirs(_COMGR_CACHE, exist_ok=True)
        os.environ["AMD_COMGR_CACHE_DIR"] = _COMGR_CACHE
        # never evict: carried entries are older than the compiler's default age limit
        os.environ.setdefault("AMD_COMGR_CACHE_POLICY", "prune_interval=8760h:prune_after=87600h")
    except OSError:
        pass


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
