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


def test_c_argument_lists_and_dtype_names():
    """parse_c_args / parse_c_arg_backend / massage_op / the spelling registry
    (reference pygpu/dtypes.py:36-147, pygpu/reduction.py:13-30)."""
    t = tools()
    import numpy as np
    from libgpuarray_amd import dtypes, reduction
    got = reduction.parse_c_args("float *a, const ga_half *b, unsigned int n, GLOBAL_MEM double x[4]")
    assert got == (t.ArrayArg("float32", "a"), t.ArrayArg("float16", "b"), t.ScalarArg("uint32", "n"),
                   t.ArrayArg("float64", "x"))
    with pytest.raises(ValueError):
        reduction.parse_c_args("quux *a")
    with pytest.raises(ValueError):
        dtypes.parse_c_arg_backend("float *", t.ScalarArg, t.ArrayArg)
    assert reduction.massage_op("a[i]*b[i] + c") == "a[0]*b[0] + c"
    assert [reduction._ceil_log2(x) for x in (0, 1, 2, 3, 4, 5, 1024, 1025)] == [0, 0, 1, 2, 2, 3, 10, 11]
    assert dtypes.NAME_TO_DTYPE["unsigned char"] == np.dtype("uint8")
    assert dtypes.dtype_to_ctype("int16") == "ga_short"
    with pytest.raises(ValueError):
        dtypes.dtype_to_ctype(None)
    with pytest.raises(RuntimeError):
        dtypes.register_dtype(np.int32, ["float"])        # the spelling belongs to float32
    dtypes.register_dtype(np.int32, ["int32_t"])
    assert reduction.parse_c_args("int32_t *v")[0].dtype == np.dtype("int32")
