"""lru_cache and prod of the tools module (reference pygpu/tools.py:171-222): no device needed."""
import os
import sys

import pytest

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


def tools():
    try:
        from libgpuarray_amd import tools as t
    except OSError as e:      # the C library is not built
        pytest.skip(str(e))
    return t


def test_prod():
    t = tools()
    assert t.prod([]) == 1 and t.prod((2, 3, 7)) == 42 and t.prod(iter([5])) == 5


def test_lru_cache_counts_and_evicts():
    t = tools()
    calls = []

    @t.lru_cache(maxsize=20)
    def f(a, b=0):
        calls.append((a, b))
        return a * 10 + b

    assert f(1) == 10 and f(1) == 10 and f(2, 3) == 23
    assert (f.hits, f.misses) == (1, 2) and calls == [(1, 0), (2, 3)]
    assert f.get(1) == 10 and f.hits == 2
    with pytest.raises(KeyError):
        f.get(99)
    # 21 distinct keys held -> the two least recently used go (20 // 10)
    for k in range(100, 119):
        f(k)
    assert f.misses == 21
    n = len(calls)
    # (2, 3) and then (1,) were the two least recently used: both are computed again
    f(2, 3)
    f(1)
    assert len(calls) == n + 2
    f.clear()
    assert (f.hits, f.misses) == (0, 0)
    assert f(1) == 10 and f.misses == 1
    assert f.maxsize == 20 and f.__name__ == "f"
