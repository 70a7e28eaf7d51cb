"""check_args on device arrays: the vectors of the reference's own test
(pygpu/tests/test_tools.py:6-118: shapes, slicing, offsets in, collapsed dims /
strides / offsets out), plus the rule checked against brute force: walking the
collapsed description visits the same byte addresses in the same order as
walking the arrays themselves."""
import itertools

import numpy as np
import pytest

from libgpuarray_amd.tools import check_args, as_argument, ArrayArg, ScalarArg
from support import gen_gpuarray

pytestmark = pytest.mark.gpu


def pair(ctx, shape, **kw):
    return gen_gpuarray(shape, "float32", ctx=ctx, **kw)[1]


# (first array: shape, knobs), (second array or None), check_args knobs, expected result
VECTORS = [
    (((50,), {}), ((50,), {}), {}, (50, 1, (50,), ((4,), (4,)), (0, 0))),
    (((50, 1, 20), {}), ((50, 1, 20), {}), {},
     (1000, 3, (50, 1, 20), ((80, 80, 4), (80, 80, 4)), (0, 0))),
    (((50, 1, 20), {}), ((50, 1, 20), {}), dict(collapse=False),
     (1000, 3, (50, 1, 20), ((80, 80, 4), (80, 80, 4)), (0, 0))),
    (((50, 1, 20), {}), ((50, 1, 20), {}), dict(collapse=True),
     (1000, 1, (1000,), ((4,), (4,)), (0, 0))),
    (((50, 1, 20), dict(sliced=2, offseted_inner=True)), ((50, 1, 20), {}), dict(collapse=True),
     (1000, 2, (50, 20), ((168, 4), (80, 4)), (4, 0))),
    (((50, 2, 10), dict(sliced=2, offseted_outer=True)), ((50, 2, 10), {}), dict(collapse=True),
     (1000, 2, (50, 20), ((160, 4), (80, 4)), (80, 0))),
    (((1,), {}), None, dict(collapse=False), (1, 1, (1,), ((4,),), (0,))),
    (((1, 1), {}), None, dict(collapse=True), (1, 1, (1,), ((4,),), (0,))),
    (((1,), {}), ((50,), {}), dict(broadcast=True), (50, 1, (50,), ((0,), (4,)), (0, 0))),
    (((50, 1, 20), dict(sliced=2, offseted_inner=True)), ((50, 1, 20), {}),
     dict(collapse=True, broadcast=True), (1000, 2, (50, 20), ((168, 4), (80, 4)), (4, 0))),
    (((10, 20, 30), {}), ((1, 1, 1), {}), dict(broadcast=True),
     (6000, 3, (10, 20, 30), ((2400, 120, 4), (0, 0, 0)), (0, 0))),
]


@pytest.mark.parametrize("case", range(len(VECTORS)))
def test_reference_vectors(ctx, case):
    a, b, kw, want = VECTORS[case]
    arrays = [pair(ctx, a[0], **a[1])]
    if b is not None:
        arrays.append(pair(ctx, b[0], **b[1]))
    assert check_args(tuple(arrays), **kw) == want


def addresses(dims, strides, offset):
    return [offset + sum(i * s for i, s in zip(idx, strides))
            for idx in itertools.product(*[range(d) for d in dims])]


@pytest.mark.parametrize("seed", range(12))
def test_collapse_keeps_the_walk(ctx, seed):
    rng = np.random.default_rng(seed)
    nd = int(rng.integers(1, 5))
    shape = tuple(int(v) for v in rng.integers(1, 5, nd))
    a = pair(ctx, shape, sliced=int(rng.choice([1, 2, -1])), offseted_inner=bool(rng.integers(2)))
    b = pair(ctx, shape, order="f" if rng.integers(2) else "c")
    bshape = tuple(1 if rng.integers(3) == 0 else d for d in shape)
    c = pair(ctx, bshape)
    n, cnd, dims, strs, offs = check_args((a, 2.5, b, c), collapse=True, broadcast=True)
    assert n == int(np.prod(shape)) and cnd == len(dims) and int(np.prod(dims)) == n
    assert strs[1] is None and offs[1] is None
    full = np.broadcast_shapes(shape, bshape)
    for k, arr in ((0, a), (2, b), (3, c)):
        st = tuple(0 if d == 1 and f != 1 else s for d, f, s in zip(arr.shape, full, arr.strides))
        assert addresses(dims, strs[k], offs[k]) == addresses(full, st, arr.offset)


def test_errors_and_descriptors(ctx):
    a, b = pair(ctx, (4, 5)), pair(ctx, (4, 1))
    with pytest.raises(ValueError):
        check_args((a, b))                      # shapes differ, no broadcasting asked
    with pytest.raises(ValueError):
        check_args((a, pair(ctx, (20,))))       # ranks differ
    with pytest.raises(ValueError):
        check_args((a, pair(ctx, (4, 3))), broadcast=True)
    with pytest.raises(TypeError):
        check_args((1.0, 2))
    assert check_args((a, b), broadcast=True)[3] == ((20, 4), (4, 0))
    assert check_args((a,), collapse=None)[1:3] == (1, (20,))
    x, s = as_argument(a, "x"), as_argument(np.float64(2), "s")
    assert isinstance(x, ArrayArg) and x.isarray() and x.expr() == "x[i]"
    assert x.decltype() == "GLOBAL_MEM ga_float *" and x.ctype() == "ga_float"
    assert isinstance(s, ScalarArg) and not s.isarray() and s.expr() == "s"
    assert s.decltype() == "ga_double" and s.spec() == np.dtype("float64")
    assert x == ArrayArg("float32", "x") and x != ScalarArg("float32", "x")
    assert hash(x) == hash(ArrayArg(np.float32, "x"))
