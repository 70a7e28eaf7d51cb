"""ndgpuarray operators, in-place operators, comparisons, divmod, broadcasting
and the rule that an output is never broadcast: the reference's Python tests
(pygpu/tests/test_elemwise.py:17-372, pygpu/tests/test_reduction.py:86-130)
with NumPy as the expected value for shape, dtype and content."""
import operator

import numpy as np
import pytest

import libgpuarray_amd as ga
from libgpuarray_amd import gpuarray, ndgpuarray as elemary
from libgpuarray_amd.dtypes import dtype_to_ctype, get_common_dtype
from libgpuarray_amd.elemwise import as_argument, ielemwise2, GpuElemwise, arg
from support import gen_gpuarray

pytestmark = pytest.mark.gpu

dtypes_test = ["float32", "int8", "uint64"]
operators1 = [operator.neg, operator.pos, operator.abs]
operators2 = [operator.add, operator.sub, operator.floordiv, operator.mod, operator.mul,
              operator.truediv, operator.eq, operator.ne, operator.lt, operator.le, operator.gt,
              operator.ge]
ioperators2 = [operator.iadd, operator.isub, operator.ifloordiv, operator.imod, operator.imul,
               operator.itruediv]
elems = [2, 0.3, np.asarray(3, dtype="int8"), np.asarray(7, dtype="uint32"),
         np.asarray(2.45, dtype="float32")]


def check_meta_content(x, y):
    assert x.shape == y.shape and x.dtype == y.dtype
    assert np.allclose(np.asarray(x), y)


def numpy_op(op, a, b):
    """NumPy's answer, or None where NumPy itself refuses the operand types."""
    try:
        with np.errstate(all="ignore"):
            return op(a, b)
    except TypeError:
        return None


@pytest.mark.parametrize("dtype", dtypes_test + ["float16"])
@pytest.mark.parametrize("op", operators1, ids=lambda o: o.__name__)
def test_elemwise1_ops_array(ctx, op, dtype):
    if dtype == "uint64" and op is operator.neg:
        pytest.skip("negating unsigned values wraps; NumPy warns")
    c, g = gen_gpuarray((50,), dtype, ctx=ctx, cls=elemary)
    out_c, out_g = op(c), op(g)
    assert type(out_g) is elemary
    check_meta_content(out_g, out_c)


@pytest.mark.parametrize("dtype2", dtypes_test)
@pytest.mark.parametrize("dtype1", dtypes_test)
@pytest.mark.parametrize("op", operators2, ids=lambda o: o.__name__)
def test_elemwise2_ops_array(ctx, op, dtype1, dtype2):
    ac, ag = gen_gpuarray((50,), dtype1, ctx=ctx, cls=elemary)
    bc, bg = gen_gpuarray((50,), dtype2, nozeros=True, ctx=ctx, cls=elemary, rng=np.random.default_rng(1))
    out_c = numpy_op(op, ac, bc)
    out_g = op(ag, bg)
    check_meta_content(out_g, out_c)


@pytest.mark.parametrize("dtype2", dtypes_test)
@pytest.mark.parametrize("dtype1", dtypes_test)
@pytest.mark.parametrize("op", ioperators2, ids=lambda o: o.__name__)
def test_ielemwise2_ops_array(ctx, op, dtype1, dtype2):
    incr = 10 if (op is operator.isub and dtype1[0] == "u") else 0
    ac, ag = gen_gpuarray((50,), dtype1, incr=incr, ctx=ctx, cls=elemary)
    bc, bg = gen_gpuarray((50,), dtype2, nozeros=True, ctx=ctx, cls=elemary, rng=np.random.default_rng(1))
    out_c = numpy_op(op, ac, bc)
    if out_c is None:
        return          # NumPy refuses the cast; the device keeps the older, laxer rule
    out_g = op(ag, bg)
    assert out_g is ag
    assert np.allclose(out_c, np.asarray(out_g), atol=1e-6)


def test_elemwise_f16(ctx):
    c, g = gen_gpuarray((50,), "float16", ctx=ctx, cls=elemary)
    d, h = gen_gpuarray((50,), "float16", ctx=ctx, cls=elemary, rng=np.random.default_rng(2))
    check_meta_content(-g, -c)
    check_meta_content(g + h, c + d)
    g += h
    c += d
    assert np.allclose(c, np.asarray(g), atol=1e-2)


@pytest.mark.parametrize("elem", elems, ids=lambda e: "%s_%s" % (type(e).__name__, getattr(e, "dtype", "")))
@pytest.mark.parametrize("dtype", dtypes_test)
@pytest.mark.parametrize("op", operators2, ids=lambda o: o.__name__)
def test_elemwise2_ops_mixed(ctx, op, dtype, elem):
    c, g = gen_gpuarray((50,), dtype, ctx=ctx, cls=elemary)
    out_c = numpy_op(op, c, elem)
    if out_c is not None:
        check_meta_content(op(g, elem), out_c)
    c, g = gen_gpuarray((50,), dtype, nozeros=True, ctx=ctx, cls=elemary)
    out_c = numpy_op(op, elem, c)
    if out_c is not None:
        check_meta_content(op(elem, g), out_c)


@pytest.mark.parametrize("elem", elems, ids=lambda e: "%s_%s" % (type(e).__name__, getattr(e, "dtype", "")))
@pytest.mark.parametrize("dtype", dtypes_test)
@pytest.mark.parametrize("op", ioperators2, ids=lambda o: o.__name__)
def test_ielemwise2_ops_mixed(ctx, op, dtype, elem):
    incr = 10 if (op is operator.isub and dtype[0] == "u") else 0
    c, g = gen_gpuarray((50,), dtype, incr=incr, ctx=ctx, cls=elemary)
    out_c = numpy_op(op, c, elem)
    if out_c is None:
        return
    out_g = op(g, elem)
    assert out_g is g
    check_meta_content(out_g, out_c)


@pytest.mark.parametrize("dtype2", dtypes_test)
@pytest.mark.parametrize("dtype1", dtypes_test)
def test_divmod_array(ctx, dtype1, dtype2):
    ac, ag = gen_gpuarray((50,), dtype1, ctx=ctx, cls=elemary)
    bc, bg = gen_gpuarray((50,), dtype2, nozeros=True, ctx=ctx, cls=elemary, rng=np.random.default_rng(1))
    out_c, out_g = divmod(ac, bc), divmod(ag, bg)
    check_meta_content(out_g[0], out_c[0])
    check_meta_content(out_g[1], out_c[1])


@pytest.mark.parametrize("elem", elems, ids=lambda e: "%s_%s" % (type(e).__name__, getattr(e, "dtype", "")))
@pytest.mark.parametrize("dtype", dtypes_test)
def test_divmod_mixed(ctx, dtype, elem):
    c, g = gen_gpuarray((50,), dtype, nozeros=True, ctx=ctx, cls=elemary)
    for x, y, gx, gy in ((c, elem, g, elem), (elem, c, elem, g)):
        out_c = numpy_op(divmod, x, y)
        if out_c is None:
            continue
        out_g = divmod(gx, gy)
        check_meta_content(out_g[0], out_c[0])
        check_meta_content(out_g[1], out_c[1])


def test_elemwise_bool(ctx):                              # test_elemwise.py:298-310
    with pytest.raises(ValueError):
        bool(gpuarray.empty((2,), context=ctx))
    assert not bool(gpuarray.zeros((1,), context=ctx))
    assert not bool(gpuarray.zeros((), context=ctx))


@pytest.mark.parametrize("shapea,shapeb", [((3, 5), (3, 5)), ((1, 5), (3, 5)), ((3, 5), (3, 1)),
                                           ((1, 5), (3, 1)), ((3, 1), (3, 5)), ((1, 1), (1, 1)),
                                           ((3, 4, 5), (4, 5)), ((4, 5), (3, 4, 5)), ((), ())])
def test_broadcast(ctx, shapea, shapeb):                  # test_elemwise.py:313-333
    ac, ag = gen_gpuarray(shapea, "float32", ctx=ctx, cls=elemary)
    bc, bg = gen_gpuarray(shapeb, "float32", ctx=ctx, cls=elemary, rng=np.random.default_rng(1))
    check_meta_content(ag + bg, ac + bc)


@pytest.mark.parametrize("shapea,shapeb", [((1, 4), (6, 4)), ((2, 1, 8, 7), (2, 2, 8, 7))])
def test_output_is_never_broadcast(ctx, shapea, shapeb):  # test_elemwise.py:66-118
    def run_ielemwise2(sa, sb, broadcast):
        na, g_a = gen_gpuarray(sa, ctx=ctx, cls=elemary)
        nb, g_b = gen_gpuarray(sb, ctx=ctx, cls=elemary, rng=np.random.default_rng(1))
        ielemwise2(g_a, "+", g_b, broadcast=broadcast)
        na = na + nb
        assert np.allclose(na, np.asarray(g_a), atol=1e-6)

    def check_elemwise2(sa, sb, output_shape, broadcast):
        na, g_a = gen_gpuarray(sa, ctx=ctx, cls=elemary)
        nb, g_b = gen_gpuarray(sb, ctx=ctx, cls=elemary, rng=np.random.default_rng(1))
        odtype = get_common_dtype(g_a, g_b, True)
        res = gpuarray.empty(output_shape, dtype=odtype, context=ctx, cls=elemary)
        args = [as_argument(res, "res", write=True), as_argument(g_a, "a", read=True),
                as_argument(g_b, "b", read=True)]
        oper = "res = (%(out_t)s)a %(op)s (%(out_t)s)b" % {"op": "+", "out_t": dtype_to_ctype(odtype)}
        GpuElemwise(ctx, oper, args, convert_f16=True)(res, g_a, g_b, broadcast=broadcast)
        assert np.allclose(na + nb, np.asarray(res), atol=1e-6)

    with pytest.raises(ValueError):
        run_ielemwise2(shapea, shapeb, False)
    with pytest.raises(ValueError):
        run_ielemwise2(shapea, shapeb, True)
    with pytest.raises(ValueError):
        check_elemwise2(shapeb, shapeb, shapea, False)
    with pytest.raises(ValueError):
        check_elemwise2(shapeb, shapeb, shapea, True)
    run_ielemwise2(shapeb, shapea, True)
    check_elemwise2(shapea, shapea, shapeb, True)
    check_elemwise2(shapea, shapeb, shapeb, True)
    check_elemwise2(shapeb, shapea, shapeb, True)


@pytest.mark.parametrize("dtype", ["float32", "float64"])
def test_infinity_preamble(ctx, dtype):                   # test_elemwise.py:336-372
    ac, ag = gen_gpuarray((2,), dtype, ctx=ctx, cls=elemary)
    out_g = ag._empty_like_me()
    flt = "ga_float" if dtype == "float32" else "ga_double"
    preamble = ("WITHIN_KERNEL %s infinity() {return INFINITY;}\n"
                "WITHIN_KERNEL %s neg_infinity() {return -INFINITY;}\n" % (flt, flt))
    out_arg = arg("out", out_g.dtype, scalar=False, read=False, write=True)
    GpuElemwise(ctx, "out = infinity()", [out_arg], preamble=preamble)(out_g)
    assert np.array_equal(np.full(2, np.inf, dtype), np.asarray(out_g))
    GpuElemwise(ctx, "out = neg_infinity()", [out_arg], preamble=preamble)(out_g)
    assert np.array_equal(np.full(2, -np.inf, dtype), np.asarray(out_g))


DTYPES_NO_COMPLEX = ["float32", "float64", "int8", "int16", "uint8", "uint16", "int32", "int64",
                     "uint32", "uint64"]


@pytest.mark.parametrize("axis", [None, 0, 1])
def test_reduction_ops(ctx, axis):                        # test_reduction.py:86-110
    cases = [(op, "bool") for op in ("all", "any")] + \
            [(op, dt) for op in ("prod", "sum", "min", "max") for dt in DTYPES_NO_COMPLEX]
    for op, dtype in cases:
        c, g = gen_gpuarray((2, 3), dtype=dtype, ctx=ctx, cls=elemary)
        rc = getattr(c, op)(axis=axis)
        rg = getattr(g, op)(axis=axis)
        check_meta_content(rg, rc)
        outc = np.empty(rc.shape, dtype=rc.dtype)
        outg = gpuarray.empty(rg.shape, dtype=rg.dtype, context=ctx)
        getattr(c, op)(axis=axis, out=outc)
        getattr(g, op)(axis=axis, out=outg)
        check_meta_content(outg, outc)


def test_reduction_wrong_type(ctx):                       # test_reduction.py:113-130
    c, g = gen_gpuarray((2, 3), dtype="float32", ctx=ctx, cls=elemary)
    with pytest.raises(TypeError):
        g.sum(out=gpuarray.empty((2, 3), dtype="int32", context=ctx))
    with pytest.raises(TypeError):
        g.sum(out=gpuarray.empty((3, 2), dtype="float32", context=ctx))
