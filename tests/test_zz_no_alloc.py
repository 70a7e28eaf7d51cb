"""GpuReduction_call_noalloc: the variant of GpuReduction_call that keeps the
partial results of a split reduction in a device array that is part of the
library (no allocation on the way).  Its results are held to those of
GpuReduction_call on the same inputs: bit for bit for integer sums and for
max/argmax (value and first index), within 1e-5 relative for float32 sums (the
two entry points may combine the partials in a different order), and both to
NumPy.  Every case makes two calls in a row on the shared array, the second on
a smaller input, so that anything the second call read beyond its own partials
would be the first call's."""
import zlib

import numpy as np
import pytest

import libgpuarray_amd as ga
from libgpuarray_amd import _lib
from support import check_float_sum

pytestmark = pytest.mark.gpu


CASES = [
    # name, op, dtype, big shape, small shape, axes, result dtype, index result
    ("full float32 sum", "sum", "float32", (1 << 24,), ((1 << 22) + 3,), (0,), "float32", False),
    ("full int32 sum", "sum", "int32", (1 << 24,), ((1 << 21) + 5,), (0,), "int64", False),
    ("full maxandargmax", "maxandargmax", "float32", (1 << 23,), ((1 << 20) + 7,), (0,), "float32", True),
    ("few long rows", "sum", "float32", (6, 1 << 21), (3, (1 << 19) + 1), (1,), "float32", False),
    ("columns, split", "sum", "int32", (1 << 14, 512), (5000, 384), (0,), "int32", False),
    ("columns, split, arg", "maxandargmax", "float32", (1 << 14, 256), (4097, 200), (0,), "float32", True),
    ("not split", "sum", "float32", (8192, 1024), (100, 33), (1,), "float32", False),
    # leading dims over short kept rows, in one launch (the array walked as one run
    # of chunks, the groups' partial rows in the static array) ...
    ("short kept rows", "sum", "float32", (1 << 20, 10), (1 << 19, 6), (0,), "float32", False),
    ("short kept rows, int", "sum", "int32", (1 << 18, 3, 5), (1 << 18, 3, 3), (0,), "int64", False),
    # ... and longer ones through folded rows: every m rows taken as one long row, then
    # the m copies of each output combined; all intermediate results in the static array
    ("folded rows", "sum", "float32", (1 << 14, 250), (5000, 250), (0,), "float32", False),
    # leading and a short trailing run of dims around kept ones: the leading dims first,
    # their partial results in the static array, then the trailing run of those
    ("leading dims first", "sum", "float32", (64, 512, 49), (32, 700, 49), (0, 2), "float32", False),
    ("leading dims first, int", "sum", "int32", (16, 4, 300, 7, 7), (64, 2, 100, 4, 4), (0, 1, 3, 4), "int64", False),
]


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_noalloc_matches_call_on_two_calls_in_a_row(ctx, case):
    name, opname, dtype, big, small, axes, d0_dtype, has_index = case
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    op = ga.GpuReduction(ctx, opname, dtype)
    hosts = []
    for shape in (big, small):
        if dtype == "int32":
            h = rng.integers(-1000, 1001, shape, dtype=np.int32)
        else:
            h = rng.standard_normal(shape, dtype=np.float32)
            if has_index:   # ties: the first of equal maxima must win
                h = np.round(h * 4) / 4
            else:           # a mean away from zero: no sum here is a cancellation
                h += np.float32(0.5)
        hosts.append(h)
    srcs = [ga.array(h, context=ctx) for h in hosts]
    shapes = [tuple(d for k, d in enumerate(h.shape) if k not in axes) for h in hosts]

    def outputs():
        return ([ga.empty(s, d0_dtype, context=ctx) for s in shapes],
                [ga.empty(s, "int64", context=ctx) if has_index else None for s in shapes])

    # the existing entry point (this also builds the kernels of both layouts)
    ref_v, ref_i = outputs()
    for k in range(2):
        op(srcs[k], list(axes), d0=ref_v[k], d1=ref_i[k])
    # the new one: two calls in a row, the second on the smaller input
    got_v, got_i = outputs()
    for k in range(2):
        op(srcs[k], list(axes), d0=got_v[k], d1=got_i[k], noalloc=True)
    ctx.sync()

    for k in range(2):
        g, r = np.asarray(got_v[k]), np.asarray(ref_v[k])
        h = hosts[k]
        if opname == "sum" and dtype == "float32":
            truth = h.sum(axis=axes, dtype=np.float64)
            scale = np.abs(h).sum(axis=axes, dtype=np.float64)
            # each entry point to the float64 sum: 1e-5 relative (see
            # check_float_sum for results that are cancellations)
            _, fallback = check_float_sum(g, truth, scale, cancel=1e-2,
                                          what="%s, call %d, new entry point" % (name, k))
            check_float_sum(r, truth, scale, cancel=1e-2, what="%s, call %d, existing entry point" % (name, k))
            assert fallback <= 0.05, (name, k, fallback)     # held to 1e-5 relative, not to the fallback
        elif opname == "sum":
            assert np.array_equal(g, r), (name, k)
            assert np.array_equal(g, h.sum(axis=axes, dtype=np.dtype(d0_dtype))), (name, k)
        else:
            assert np.array_equal(g, r), (name, k)
            gi, ri = np.asarray(got_i[k]), np.asarray(ref_i[k])
            assert np.array_equal(gi, ri), (name, k)
            ax = axes[0]
            assert np.array_equal(g, h.max(axis=ax)) and np.array_equal(gi, h.argmax(axis=ax)), (name, k)


def test_noalloc_refuses_what_it_would_have_to_allocate_for(ctx, knobs):
    # kernels not built yet: building loads a code object, which allocates
    op = ga.GpuReduction(ctx, "prod", "float64")
    x = ga.zeros((1000, 37), "float64", context=ctx)
    out = ga.empty((1000,), "float64", context=ctx)
    with pytest.raises(_lib.UnsupportedException, match="not built"):
        op(x, [1], d0=out, noalloc=True)
    op(x, [1], d0=out)                      # builds them
    op(x, [1], d0=out, noalloc=True)        # now served
    assert np.array_equal(np.asarray(out), np.zeros(1000))

    # More partials than the static array holds.  With the default tuning no
    # split leaves more than about 3 MiB of them; asking for 256 groups per
    # compute unit cuts these 65536 columns into 8 pieces each: 6 MiB.
    op = ga.GpuReduction(ctx, "sum", "float32")
    big = ga.zeros((512, 65536), "float32", context=ctx)
    res = ga.empty((65536,), "float32", context=ctx)
    knobs(REDUX_GROUPS_PER_CU=256)
    op(big, [0], d0=res)
    with pytest.raises(_lib.GpuArrayException, match="static scratch array holds") as e:
        op(big, [0], d0=res, noalloc=True)
    assert e.value.code == _lib.GA_XLARGE_ERROR
    knobs(REDUX_GROUPS_PER_CU=None)
    op(big, [0], d0=res)
    op(big, [0], d0=res, noalloc=True)      # the default split fits
    assert not np.asarray(res).any()
    # operators with an expression have their own entry point
    from libgpuarray_amd import reduction as R
    dot = R.MapReduction(ctx, "sum", "float32", "p*q", [R.ArrayArg("float32", "p"), R.ArrayArg("float32", "q")])
    err = _lib.lib.GpuReduction_call_noalloc(dot.gr, res._ref, None, big._ref, 1, (_lib.C.c_int * 1)(0), 0)
    assert err == _lib.GA_INVALID_ERROR
