"""An elementwise expression feeding a reduction in one kernel
(GpuReduction_new_map / GpuReduction_call_map, ReductionKernel(map_expr=...)):
the reference's own cases (pygpu/tests/test_reduction.py:12-84), bit-exact
comparisons with the CPU checker on data where every operation is exact, and
tolerance comparisons elsewhere (1e-5 relative for float32 sums)."""
import itertools

import numpy as np
import pytest

import libgpuarray_amd as ga
from libgpuarray_amd import _lib, gpuarray
from libgpuarray_amd import reduction as R
from libgpuarray_amd.reduction import ReductionKernel, MapReduction, ArrayArg, ScalarArg, as_argument
from support import to_gpu_view, gen_gpuarray

pytestmark = pytest.mark.gpu

DTYPES_NO_COMPLEX_BIG = ["float32", "float64", "int32", "int64", "uint32", "uint64"]


# ---- pygpu/tests/test_reduction.py:12-56: "a + b" over every axis subset ---------------------

@pytest.mark.parametrize("dtype", DTYPES_NO_COMPLEX_BIG)
def test_red_array_basic(ctx, dtype):
    for shape, redux in [((10,), [True]),
                         ((20, 30), [True, True]), ((20, 30), [True, False]), ((20, 30), [False, True]),
                         ((8, 5, 10), [True, True, True]), ((8, 5, 10), [True, True, False]),
                         ((8, 5, 10), [True, False, True]), ((8, 5, 10), [False, True, True]),
                         ((8, 5, 10), [True, False, False]), ((8, 5, 10), [False, True, False]),
                         ((8, 5, 10), [False, False, True])]:
        c, g = gen_gpuarray(shape, dtype, ctx=ctx)
        axes = tuple(i for i, r in enumerate(redux) if r)
        out_c = c.sum(axis=axes, dtype=dtype)
        out_g = ReductionKernel(ctx, dtype, "0", "a + b", redux)(g)
        assert out_c.shape == out_g.shape and out_g.dtype == np.dtype(dtype)
        assert np.allclose(out_c, np.asarray(out_g), rtol=2e-5)


@pytest.mark.parametrize("redux", [[True, False, False], [True, False, True], [False, True, True],
                                   [False, True, False]])
def test_red_big_array(ctx, redux):                       # test_reduction.py:48-53
    c, g = gen_gpuarray((2000, 30, 100), "float32", ctx=ctx)
    axes = tuple(i for i, r in enumerate(redux) if r)
    out_g = ReductionKernel(ctx, "float32", "0", "a + b", redux)(g)
    assert np.allclose(c.sum(axis=axes, dtype=np.float64), np.asarray(out_g), rtol=2e-5)


def test_red_broadcast(ctx):                               # test_reduction.py:57-84
    dtype = float
    redux = [False, True, False]
    nx, gx = gen_gpuarray((5, 10, 15), dtype, ctx=ctx)
    ny, gy = gen_gpuarray((1, 10, 15), dtype, ctx=ctx)
    nz = (nx * ny).sum(axis=1)
    args = [as_argument(gx, "a"), as_argument(gy, "b")]
    gz = ReductionKernel(ctx, dtype, "0", "a+b", redux, map_expr="a[i]*b[i]", arguments=args)(
        gx, gy, broadcast=True)
    assert np.allclose(nz, np.asarray(gz))
    with pytest.raises(ValueError):
        ReductionKernel(ctx, dtype, "0", "a+b", redux, map_expr="a[i]*b[i]", arguments=args)(gx, gy)


def test_constructor_rules(ctx):                           # pygpu/reduction.py:137-177
    with pytest.raises(ValueError, match="no axes"):
        ReductionKernel(ctx, "float32", "0", "a+b", [False, False])
    two = [ArrayArg("float32", "x"), ArrayArg("float32", "y")]
    with pytest.raises(ValueError, match="more than one"):
        ReductionKernel(ctx, "float32", "0", "a+b", [True], arguments=two)
    with pytest.raises(ValueError, match="at least one vector"):
        ReductionKernel(ctx, "float32", "0", "a+b", [True], map_expr="s", arguments=[ScalarArg("float32", "s")])
    k = ReductionKernel(ctx, "float32", "0", "a+b", [True], map_expr="x[i]*y[i]",
                        arguments="float *x, const float *y")
    assert [type(a) for a in k.arguments] == [ArrayArg, ArrayArg]
    g = gpuarray.array(np.arange(6, dtype=np.float32), context=ctx)
    assert float(np.asarray(k(g, g))) == 55.0
    with pytest.raises(TypeError):
        k(g, g, out=gpuarray.empty((), "float64", context=ctx))
    with pytest.raises(TypeError):
        k(g, g, out=gpuarray.empty((1,), "float32", context=ctx))
    with pytest.raises(TypeError):
        k(g, g, bogus=1)


# ---- bit-exact against the CPU checker -----------------------------------------------------

def _layouts(rng, dt):
    """(x, y) host views over one common shape, integer-valued so that sums of
    products are exact in float32 and float64."""
    def ints(shape):
        return rng.integers(-8, 9, size=shape).astype(dt)
    yield ints((5, 10, 15)), ints((1, 10, 15))
    yield ints((64, 300)), ints((64, 300))
    yield ints((64, 300)), ints((1, 300))
    yield ints((64, 300)), ints((64, 1))
    yield ints((300, 64)).T, ints((64, 300))
    yield ints((40, 9, 28))[::2, ::-1, 1::3], ints((28, 9, 40)).T[::2, :, 1::3]
    yield ints((7, 4096)), ints((7, 4096))
    yield ints((3, 5000))[:, 1:], ints((3, 5000))[:, :-1]     # second operand aligned, first not
    yield ints((2, 3, 4, 5, 6)), ints((2, 1, 4, 1, 6))


@pytest.mark.parametrize("dt", [np.float32, np.float64], ids=["f32", "f64"])
def test_dot_like_sums_match_the_checker(ctx, oracle, dt):
    rng = np.random.default_rng(31)
    for x, y in _layouts(rng, dt):
        nd = x.ndim
        gx, _ = to_gpu_view(x, ctx)
        gy, _ = to_gpu_view(y, ctx)
        for r in range(1, nd + 1):
            for axes in itertools.combinations(range(nd), r):
                if nd > 3 and r not in (1, nd):
                    continue
                redux = [i in axes for i in range(nd)]
                k = ReductionKernel(ctx, dt, "0", "a+b", redux, map_expr="p[i]*q[i]",
                                    arguments=[ArrayArg(dt, "p"), ArrayArg(dt, "q")])
                got = np.asarray(k(gx, gy, broadcast=True))
                want = oracle.reduk_map2(oracle.MAP_MUL, oracle.RED_ADD, x, y, 0.0, list(axes), ls=64)
                assert got.shape == want.shape
                assert np.array_equal(got, want), (x.shape, x.strides, y.strides, axes)


def test_scalar_argument_and_max_reduction(ctx, oracle):
    rng = np.random.default_rng(32)
    x = rng.standard_normal((33, 257)).astype(np.float32)
    y = rng.standard_normal((33, 257)).astype(np.float32)
    gx, gy = gpuarray.array(x, context=ctx), gpuarray.array(y, context=ctx)
    args = [ArrayArg("float32", "u"), ArrayArg("float32", "v"), ScalarArg("float32", "s")]
    # max is exact whatever the order: bit-exact on arbitrary data
    k = ReductionKernel(ctx, "float32", "-INFINITY", "max(a, b)", [False, True],
                        map_expr="fabsf(u[i] - v[i])", arguments=args)
    got = np.asarray(k(gx, gy, 0.0))
    want = oracle.reduk_map2(oracle.MAP_ABSDIFF, oracle.RED_MAX, x, y, 0.0, [1])
    assert np.array_equal(got, want)
    xi = rng.integers(-8, 9, size=(33, 257)).astype(np.float32)
    yi = rng.integers(-8, 9, size=(33, 257)).astype(np.float32)
    k2 = ReductionKernel(ctx, "float32", "0", "a+b", [True, False], map_expr="s*u[i] + v[i]",
                         arguments=args)
    got = np.asarray(k2(gpuarray.array(xi, context=ctx), gpuarray.array(yi, context=ctx), 3.0))
    want = oracle.reduk_map2(oracle.MAP_SAXPY, oracle.RED_ADD, xi, yi, 3.0, [0])
    assert np.array_equal(got, want)


def test_built_in_operations_over_an_expression(ctx):
    """max and argmax of |a-b|, any(a > b), integer dot product with a wide
    accumulator: exact whatever the order, so NumPy is the answer."""
    rng = np.random.default_rng(33)
    a = rng.standard_normal((300, 1000)).astype(np.float32)
    b = rng.standard_normal((300, 1000)).astype(np.float32)
    b[7] = a[7]                                            # a row of ties: index 0 wins
    ga_, gb = gpuarray.array(a, context=ctx), gpuarray.array(b, context=ctx)
    args = [ArrayArg("float32", "a"), ArrayArg("float32", "b")]
    op = MapReduction(ctx, "maxandargmax", "float32", "fabsf(a - b)", args)
    d0 = gpuarray.empty((300,), "float32", context=ctx)
    d1 = gpuarray.empty((300,), "int64", context=ctx)
    op([ga_, gb], [1], d0=d0, d1=d1)
    diff = np.abs(a - b)
    assert np.array_equal(np.asarray(d0), diff.max(axis=1))
    assert np.array_equal(np.asarray(d1), diff.argmax(axis=1))
    # the other axis, lanes along the free dim
    d0 = gpuarray.empty((1000,), "float32", context=ctx)
    d1 = gpuarray.empty((1000,), "int64", context=ctx)
    op([ga_, gb], [0], d0=d0, d1=d1)
    assert np.array_equal(np.asarray(d0), diff.max(axis=0))
    assert np.array_equal(np.asarray(d1), diff.argmax(axis=0))

    anyop = MapReduction(ctx, "any", "float32", "a > b + 3.5f", args)
    d = gpuarray.empty((300,), "bool", context=ctx)
    anyop([ga_, gb], [1], d0=d)
    assert np.array_equal(np.asarray(d), (a > b + np.float32(3.5)).any(axis=1))

    p = rng.integers(-128, 128, size=(50, 4096), dtype=np.int8)
    q = rng.integers(-128, 128, size=(50, 4096), dtype=np.int8)
    dot = MapReduction(ctx, "sum", "int32", "(ga_int)p * (ga_int)q",
                       [ArrayArg("int8", "p"), ArrayArg("int8", "q")])
    d = gpuarray.empty((50,), "int32", context=ctx)
    dot([gpuarray.array(p, context=ctx), gpuarray.array(q, context=ctx)], [1], d0=d)
    assert np.array_equal(np.asarray(d), (p.astype(np.int32) * q.astype(np.int32)).sum(axis=1, dtype=np.int32))


def test_mixed_types_half_and_float(ctx):
    rng = np.random.default_rng(34)
    h = rng.integers(-4, 5, size=(128, 768)).astype(np.float16)
    f = rng.integers(-4, 5, size=(128, 768)).astype(np.float32)
    op = MapReduction(ctx, "sum", "float32", "h * f", [ArrayArg("float16", "h"), ArrayArg("float32", "f")])
    d = gpuarray.empty((128,), "float32", context=ctx)
    op([gpuarray.array(h, context=ctx), gpuarray.array(f, context=ctx)], [1], d0=d)
    assert np.array_equal(np.asarray(d), (h.astype(np.float32) * f).sum(axis=1))
    # half result: accumulated in float, stored as half
    oph = MapReduction(ctx, "sum", "float16", "h * f", [ArrayArg("float16", "h"), ArrayArg("float32", "f")])
    dh = gpuarray.empty((768,), "float16", context=ctx)
    oph([gpuarray.array(h, context=ctx), gpuarray.array(f, context=ctx)], [0], d0=dh)
    assert np.array_equal(np.asarray(dh), (h.astype(np.float32) * f).sum(axis=0).astype(np.float16))


def test_argument_errors(ctx):
    L = _lib.lib
    import ctypes as C
    descr = (_lib.ElemwiseArg * 2)()
    descr[0].name, descr[0].typecode, descr[0].flags = b"a", _lib.GA_FLOAT, _lib.GE_READ
    descr[1].name, descr[1].typecode, descr[1].flags = b"b", _lib.GA_FLOAT, _lib.GE_WRITE
    gr = C.c_void_p()

    def new(op, red, neu, acc, expr, n):
        return L.GpuReduction_new_map(C.byref(gr), ctx.ctx, op, red, neu, acc, b"", expr, n,
                                      C.cast(descr, C.c_void_p), 0)

    assert new(_lib.GA_REDUCE_SUM, None, None, _lib.GA_FLOAT, b"a*b", 2) == _lib.GA_VALUE_ERROR
    descr[1].flags = _lib.GE_READ
    descr[1].name = b"a"
    assert new(_lib.GA_REDUCE_SUM, None, None, _lib.GA_FLOAT, b"a*a", 2) == _lib.GA_VALUE_ERROR
    descr[1].name = b"b"
    assert new(_lib.GA_REDUCE_CUSTOM, None, None, _lib.GA_FLOAT, b"a*b", 2) == _lib.GA_INVALID_ERROR
    assert new(_lib.GA_REDUCE_SUM, None, None, _lib.GA_FLOAT, b"", 2) == _lib.GA_INVALID_ERROR
    assert new(_lib.GA_REDUCE_XOR, None, None, _lib.GA_FLOAT, b"a*b", 2) == _lib.GA_UNSUPPORTED_ERROR
    assert new(99, None, None, _lib.GA_FLOAT, b"a*b", 2) == _lib.GA_INVALID_ERROR
    assert not gr.value

    args = [ArrayArg("float32", "a"), ArrayArg("float32", "b")]
    op = MapReduction(ctx, "sum", "float32", "a*b", args)
    x = gpuarray.array(np.ones((4, 6), np.float32), context=ctx)
    y3 = gpuarray.array(np.ones((4, 6, 1), np.float32), context=ctx)
    y5 = gpuarray.array(np.ones((4, 5), np.float32), context=ctx)
    y1 = gpuarray.array(np.ones((1, 6), np.float32), context=ctx)
    d = gpuarray.empty((4,), "float32", context=ctx)
    with pytest.raises(ValueError):
        op([x, y3], [1], d0=d)
    with pytest.raises(ValueError):
        op([x, y5], [1], d0=d, broadcast=True)
    with pytest.raises(ValueError):
        op([x, y1], [1], d0=d)                          # no broadcasting asked for
    op([x, y1], [1], d0=d, broadcast=True)
    assert np.asarray(d).tolist() == [6.0] * 4
    with pytest.raises(ValueError):                     # result type is the accumulator's
        op([x, x], [1], d0=gpuarray.empty((4,), "float64", context=ctx))
    with pytest.raises(ValueError):
        op([x, gpuarray.array(np.ones((4, 6)), context=ctx)], [1], d0=d)
    # a multi-argument operator cannot go through the one-source entry point
    ax = (C.c_int * 1)(1)
    assert L.GpuReduction_call(op.gr, d._ptr(), None, x._ptr(), 1, ax, 0) == _lib.GA_INVALID_ERROR
    # a broken expression surfaces the compiler's message at first use
    bad = MapReduction(ctx, "sum", "float32", "a * nonsense", args)
    with pytest.raises(_lib.GpuArrayException):
        bad([x, x], [1], d0=d)


def test_reduce1_reference_signature(ctx):                # pygpu/reduction.py:294-319
    c, g = gen_gpuarray((6, 7), "float32", ctx=ctx)
    assert np.allclose(np.asarray(R.reduce1(g, "+", "0", "float32", axis=1)), c.sum(axis=1), rtol=1e-5)
    assert np.allclose(np.asarray(R.reduce1(g, "*", "1", "float64", axis=0)),
                       c.prod(axis=0, dtype=np.float64), rtol=1e-6)
    got = R.reduce1(g, None, "-INFINITY", "float32", axis=None, oper="max(a, b)")
    assert float(np.asarray(got)) == c.max()
    with pytest.raises(ValueError):
        R.reduce1(g, "+", "0", "float32", axis=2)


def test_large_dot_product_is_exact(ctx):
    """2^26 elements per operand, one pass: integer-valued floats whose
    products sum exactly in float64; and the float32 result within 1e-5."""
    rng = np.random.default_rng(35)
    n = 1 << 26
    a = rng.integers(-3, 4, size=n).astype(np.float32)
    b = rng.integers(-3, 4, size=n).astype(np.float32)
    ga_, gb = gpuarray.array(a, context=ctx), gpuarray.array(b, context=ctx)
    want = int((a.astype(np.int64) * b.astype(np.int64)).sum())
    k64 = MapReduction(ctx, "sum", "float64", "(ga_double)a * (ga_double)b",
                       [ArrayArg("float32", "a"), ArrayArg("float32", "b")])
    d = gpuarray.empty((), "float64", context=ctx)
    k64([ga_, gb], [0], d0=d)
    assert float(np.asarray(d)) == float(want)
    k32 = ReductionKernel(ctx, "float32", "0", "a+b", [True], map_expr="x[i]*y[i]",
                          arguments=[ArrayArg("float32", "x"), ArrayArg("float32", "y")])
    got = float(np.asarray(k32(ga_, gb)))
    assert abs(got - want) <= 1e-5 * max(abs(want), float(np.abs(a * b).sum()) * 1e-2)
    # sum of squares equals the count of each magnitude: closed form
    sq = ReductionKernel(ctx, "float64", "0", "a+b", [True], map_expr="x[i]*x[i]",
                         arguments=[ArrayArg("float32", "x")])
    assert float(np.asarray(sq(ga_))) == float((a.astype(np.int64) ** 2).sum())
