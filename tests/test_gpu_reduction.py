"""Reductions on the device, through the C ABI, against
  - the reference's own four maxandargmax tests (tests/check_reduction.c) on
    its PCG32 data, bit for bit, with the CPU checker as the expected value,
  - the checker / NumPy on seeded random layouts, every op and dtype,
  - the Python layer's rules for sum/prod/all/any (pygpu/tests/test_reduction.py).
Integer, boolean and index results must be identical; float sums are held to
1e-5 of the float64 sum (relative to the sum of magnitudes when the result
itself is tiny), fp16 inputs to 1e-2."""
import ctypes as C

import numpy as np
import pytest

import libgpuarray_amd as ga
from libgpuarray_amd import _lib, gpuarray, reduction as R
from support import to_gpu_view, gen_gpuarray, check_float_sum

pytestmark = pytest.mark.gpu
lib = _lib.lib


def np_maxandargmax(x, redux, op="max"):
    free = [i for i in range(x.ndim) if i not in redux]
    y = x.transpose(free + list(redux)).reshape([x.shape[i] for i in free] + [-1])
    return (y.max(-1), y.argmax(-1)) if op == "max" else (y.min(-1), y.argmin(-1))


def assert_sum_close(got, x64sum, abs64sum, rtol=1e-5, cancel=1e-2):
    """1e-5 of the float64 sum wherever the sum is not a cancellation; 8
    float32 epsilons of the sum of magnitudes below that, where a relative
    bound on a result near zero means nothing.  The layout tests, whose sums
    have as few as three elements, call a result a cancellation when it is
    below 1e-2 of the sum of magnitudes: one rounding of one partial sum of
    that size is already 1e-5 of such a result in float32, whatever the order.
    The benchmark's long sums are held to 1e-3 (cancel=1e-3).  Returns (largest
    relative error among the results held to rtol, fraction of results that
    took the fallback)."""
    return check_float_sum(got, x64sum, abs64sum, rtol=rtol, cancel=cancel)


# ---- the reference's four tests ------------------------------------------------------

@pytest.mark.parametrize("shape,redux", [
    ((32, 50, 79), [0, 2]),                       # test_reduction
    ((32, 50, 79), [2, 0]),                       # test_idxtranspose
    ((1171, 373, 2, 1, 2, 1, 2, 1), [2, 4, 7, 5]),  # test_veryhighrank
    ((32, 50, 79), [0, 1, 2]),                    # test_alldimsreduced
])
def test_reference_maxandargmax_tests(shape, redux, ctx, oracle):
    x = oracle.pcg_fill_f32(int(np.prod(shape)), seed=1).reshape(shape)
    g = gpuarray.array(x, context=ctx)
    oshape = tuple(d for i, d in enumerate(shape) if i not in redux)
    gmax = gpuarray.empty(oshape, "float32", context=ctx)
    garg = gpuarray.empty(oshape, "uint64", context=ctx)    # the tests allocate GA_ULONG
    gmax.memset(0xff)
    garg.memset(0xff)
    arr = (C.c_uint * len(redux))(*redux)
    assert lib.GpuArray_maxandargmax(gmax._ptr(), garg._ptr(), g._ptr(), len(redux), arr) == 0
    wm, wa = oracle.maxandargmax(x, redux)
    assert np.array_equal(np.asarray(gmax), wm)
    assert np.array_equal(np.asarray(garg).astype(np.int64), wa)
    nm, na = np_maxandargmax(x, redux)
    assert np.array_equal(wm, nm) and np.array_equal(wa, na)


def test_maxandargmax_argument_errors(ctx):         # src/gpuarray_reduction.c:198-261
    g = gpuarray.zeros((4, 5), "float32", context=ctx)
    m = gpuarray.empty((4,), "float32", context=ctx)
    a = gpuarray.empty((4,), "uint64", context=ctx)
    def call(n, axes, src=g, dm=m, da=a):
        arr = (C.c_uint * max(len(axes), 1))(*axes)
        return lib.GpuArray_maxandargmax(dm._ptr() if dm is not None else None,
                                         da._ptr() if da is not None else None,
                                         src._ptr() if src is not None else None, n, arr)
    assert call(1, [1]) == 0
    assert call(0, []) == _lib.GA_INVALID_ERROR
    assert call(3, [0, 1, 1]) == _lib.GA_INVALID_ERROR
    assert call(2, [1, 1]) == _lib.GA_INVALID_ERROR
    assert call(1, [2]) == _lib.GA_INVALID_ERROR
    assert call(1, [1], dm=None) == _lib.GA_INVALID_ERROR
    assert call(1, [1], src=None) == _lib.GA_INVALID_ERROR
    z = gpuarray.zeros((), "float32", context=ctx)
    assert call(1, [0], src=z) == _lib.GA_INVALID_ERROR
    # destination shape is checked here (the reference does not, and would
    # write out of bounds)
    wrong = gpuarray.empty((5,), "float32", context=ctx)
    assert call(1, [1], dm=wrong) == _lib.GA_VALUE_ERROR


def test_ties_nan_and_signed_zero(ctx, oracle):
    x = np.zeros((6, 300), np.float32)
    x[0, [250, 17, 123]] = 4.0                    # ties -> first index
    x[1, :] = 2.0                                 # constant row -> 0
    x[2, :] = np.arange(300)                      # increasing -> last
    x[3, 5] = np.nan; x[3, 9] = 1.0               # NaN not first: ignored
    x[4, 0] = np.nan; x[4, 9] = 1.0               # NaN first: stays
    x[5, :] = -0.0; x[5, 100] = 0.0               # equal zeros: first one scanned
    g = gpuarray.array(x, context=ctx)
    v, i = R.maxandargmax(g, axis=1)
    wm, wa = oracle.maxandargmax(x, [1])
    got_v, got_i = np.asarray(v), np.asarray(i)
    assert np.array_equal(got_i, wa) and got_i.tolist() == [17, 0, 299, 9, 0, 0]
    assert np.array_equal(got_v.view(np.uint32), wm.view(np.uint32))     # bits, incl. NaN and -0
    # plain max gives the same values as maxandargmax
    assert np.array_equal(np.asarray(R.max(g, axis=1)).view(np.uint32), wm.view(np.uint32))
    # ties across a split full reduction and across wavefronts
    big = np.zeros(1 << 20, np.float32)
    big[[900000, 70000, 1 << 19]] = 1.0
    v, i = R.maxandargmax(gpuarray.array(big, context=ctx))
    assert np.asarray(v) == 1.0 and np.asarray(i) == 70000
    v, i = R.minandargmin(gpuarray.array(-big, context=ctx))
    assert np.asarray(v) == -1.0 and np.asarray(i) == 70000


@pytest.mark.parametrize("seed", range(5))
def test_random_layouts_arg_reductions_vs_checker(seed, ctx, oracle):
    rng = np.random.default_rng(200 + seed)
    for _ in range(10):
        nd = int(rng.integers(1, 5))
        shape = [int(x) for x in rng.integers(1, [70, 12, 7, 4][:nd])]
        rng.shuffle(shape)
        dt = rng.choice(["float32", "float64", "int32", "float16"])
        base = (rng.integers(-20, 20, [2 * d + 1 for d in shape])).astype(dt)  # many ties
        idx = tuple(slice(int(rng.integers(0, 2)), None, 2) for _ in shape)
        v = base[idx][tuple(slice(0, d) for d in shape)]
        v = v.transpose(rng.permutation(nd))
        nr = int(rng.integers(1, nd + 1))
        redux = [int(a) for a in rng.permutation(nd)[:nr]]
        g, _ = to_gpu_view(v, ctx)
        gv, gi = R._arg_reduce(g, "maxandargmax", redux, True)
        wm, wa = oracle.maxandargmax(v, redux)
        assert np.array_equal(np.asarray(gi), wa), (v.shape, v.strides, redux, dt)
        assert np.array_equal(np.asarray(gv), wm)


def test_destination_strides_are_honoured(ctx, oracle):
    rng = np.random.default_rng(31)
    x = rng.normal(size=(9, 40, 11)).astype(np.float32)
    g = gpuarray.array(x, context=ctx)
    # results go into every other column of a Fortran-ordered block
    bigm = gpuarray.zeros((9, 22), "float32", "F", context=ctx)
    biga = gpuarray.zeros((9, 22), "int64", "F", context=ctx)
    dm, da = bigm[:, ::2], biga[:, ::2]
    op = ga.GpuReduction(ctx, "maxandargmax", "float32")
    op(g, [1], d0=dm, d1=da)
    wm, wa = oracle.maxandargmax(x, [1])
    assert np.array_equal(np.asarray(bigm)[:, ::2], wm) and np.all(np.asarray(bigm)[:, 1::2] == 0)
    assert np.array_equal(np.asarray(biga)[:, ::2], wa)


# ---- sum / prod / all / any: the Python layer's rules ---------------------------------

DTYPES = ["bool", "int8", "uint8", "int16", "uint16", "int32", "uint32", "int64", "uint64",
          "float32", "float64"]


@pytest.mark.parametrize("shape,redux", [
    ((10,), [True]), ((20, 30), [True, True]), ((20, 30), [True, False]), ((20, 30), [False, True]),
    ((8, 5, 10), [True, True, True]), ((8, 5, 10), [True, True, False]),
    ((8, 5, 10), [True, False, True]), ((8, 5, 10), [False, True, True]),
    ((8, 5, 10), [True, False, False]), ((8, 5, 10), [False, True, False]),
    ((8, 5, 10), [False, False, True]),
])
def test_red_array_basic(shape, redux, ctx, oracle):   # pygpu/tests/test_reduction.py:12-53
    rng = np.random.default_rng(1)
    axes = tuple(i for i, r in enumerate(redux) if r)
    for dt in ["int8", "uint8", "int16", "uint16", "int32", "uint32", "float32", "float64"]:
        c, g = gen_gpuarray(shape, dt, ctx=ctx, rng=rng)
        out = R.reduce1(g, "+", "0", dt, axis=axes)          # same dtype in and out, as the test
        want = c.sum(axis=axes, dtype=dt)
        assert out.shape == want.shape and out.dtype == np.dtype(dt)
        if np.dtype(dt).kind in "iu":
            assert np.array_equal(np.asarray(out), want)
        else:
            assert np.allclose(np.asarray(out), want, rtol=2e-5)
            chk = oracle.reduk("sum", c, list(axes), dt, ls=64)
            assert np.allclose(np.asarray(out), chk, rtol=2e-5)


@pytest.mark.parametrize("redux", [[True, False, False], [True, False, True],
                                   [False, True, True], [False, True, False]])
def test_red_big_array(redux, ctx):                    # pygpu/tests/test_reduction.py:41-46
    rng = np.random.default_rng(2)
    axes = tuple(i for i, r in enumerate(redux) if r)
    c, g = gen_gpuarray((2000, 30, 100), "float32", ctx=ctx, rng=rng)
    out = np.asarray(R.sum(g, axis=axes))
    want = c.astype(np.float64).sum(axis=axes)
    assert np.allclose(out, want, rtol=2e-5)
    assert_sum_close(out, want, np.abs(c.astype(np.float64)).sum(axis=axes))


@pytest.mark.parametrize("axis", [None, 0, 1, -1, (0, 1)])
def test_reduction_ops_meta_and_content(axis, ctx):    # pygpu/tests/test_reduction.py:86-110
    rng = np.random.default_rng(3)
    for op in ("all", "any"):
        c, g = gen_gpuarray((2, 3), "bool", ctx=ctx, rng=rng, high=1.6)
        rc, rg = getattr(c, op)(axis=axis), getattr(R, op)(g, axis=axis)
        assert rg.shape == np.shape(rc) and rg.dtype == np.dtype("bool")
        assert np.array_equal(np.asarray(rg), rc)
    for op in ("prod", "sum", "min", "max"):
        for dt in DTYPES:
            c, g = gen_gpuarray((2, 3), dt, ctx=ctx, rng=rng, high=5)
            rc, rg = getattr(c, op)(axis=axis), getattr(R, op)(g, axis=axis)
            assert rg.shape == np.shape(rc), (op, dt)
            assert rg.dtype == np.asarray(rc).dtype, (op, dt, rg.dtype, np.asarray(rc).dtype)
            if np.dtype(dt).kind == "f":
                assert np.allclose(np.asarray(rg), rc, rtol=1e-6)
            else:
                assert np.array_equal(np.asarray(rg), rc), (op, dt)
            # and again into a caller-provided output
            outg = gpuarray.empty(rg.shape, rg.dtype, context=ctx)
            getattr(R, op)(g, axis=axis, out=outg)
            assert np.array_equal(np.asarray(outg), np.asarray(rg))


def test_reduction_wrong_out_and_axis(ctx):            # pygpu/tests/test_reduction.py:113-128
    c, g = gen_gpuarray((2, 3), "float32", ctx=ctx)
    with pytest.raises(TypeError):
        R.sum(g, out=gpuarray.empty((2, 3), "int32", context=ctx))
    with pytest.raises(TypeError):
        R.sum(g, axis=0, out=gpuarray.empty((2,), "float32", context=ctx))
    with pytest.raises(ValueError):
        R.sum(g, axis=2)
    with pytest.raises(ValueError):
        R.sum(g, axis=-3)
    # the C entry point checks shapes itself
    op = ga.GpuReduction(ctx, "sum", "float32")
    with pytest.raises(ValueError):
        op(g, [0], d0=gpuarray.empty((2,), "float32", context=ctx))
    with pytest.raises(ga.GpuArrayException):
        op(g, [0, 0], d0=gpuarray.empty((), "float32", context=ctx))
    with pytest.raises(ga.GpuArrayException):
        op(g, [], d0=gpuarray.empty((2, 3), "float32", context=ctx))
    with pytest.raises(ga.GpuArrayException):   # source dtype differs from the operator's
        op(g.astype("float64"), [0], d0=gpuarray.empty((3,), "float64", context=ctx))


def test_reduction_0d_and_empty(ctx):                  # pygpu/tests/test_reduction.py:131-142
    for val in (True, False):
        g = gpuarray.array(np.array(val), context=ctx)
        assert bool(np.asarray(R.any(g))) == val and bool(np.asarray(R.all(g))) == val
    # reducing an empty axis gives the neutral element; nothing to write when
    # the result itself is empty
    e = gpuarray.zeros((4, 0), "float32", context=ctx)
    assert np.array_equal(np.asarray(R.sum(e, axis=1)), np.zeros(4, np.float32))
    assert np.array_equal(np.asarray(R.prod(e, axis=1)), np.ones(4, np.float32))
    assert np.array_equal(np.asarray(R.all(e, axis=1)), np.ones(4, bool))
    assert np.array_equal(np.asarray(R.any(e, axis=1)), np.zeros(4, bool))
    assert R.sum(e, axis=0).shape == (0,)
    with pytest.raises(ValueError):
        R.max(e, axis=1)


def test_float16_is_accepted_with_float32_accumulation(ctx):
    # the reference refuses float16 here (pygpu/tests/test_reduction.py:145-148);
    # this engine widens to float32.  NumPy is the only expected value.
    rng = np.random.default_rng(5)
    x = rng.uniform(-4, 4, (37, 513)).astype(np.float16)
    g = gpuarray.array(x, context=ctx)
    want = x.astype(np.float64).sum(axis=1)
    got32 = np.asarray(R.sum(g, axis=1, dtype="float32"))
    assert np.allclose(got32, want, rtol=1e-2) and np.allclose(got32, want, rtol=1e-5, atol=1e-4)
    got16 = np.asarray(R.sum(g, axis=1))                # float16 result, float32 accumulator
    assert got16.dtype == np.float16
    assert np.array_equal(got16, got32.astype(np.float16))


# ---- every op, strided layouts, both kernel families, split and unsplit ---------------

def np_reduce(op, x, axes, out_dtype=None):
    axes = tuple(axes)
    if op == "sum":
        return x.sum(axis=axes, dtype=out_dtype)
    if op == "prod":
        return x.prod(axis=axes, dtype=out_dtype)
    if op == "prodnz":
        return np.where(x == 0, 1, x).prod(axis=axes, dtype=out_dtype)
    if op == "and":
        return np.bitwise_and.reduce(x, axis=axes)
    if op == "or":
        return np.bitwise_or.reduce(x, axis=axes)
    if op == "xor":
        return np.bitwise_xor.reduce(x, axis=axes)
    if op == "all":
        return x.all(axis=axes)
    if op == "any":
        return x.any(axis=axes)
    raise KeyError(op)


LAYOUTS = [
    # (base shape, view maker, axes): chosen to hit row/col kernels, vector and
    # scalar loads, multi-dim reduced and free sets, and split rows
    ((64, 1000), lambda b: b, [1]),
    ((64, 1000), lambda b: b, [0]),
    ((300, 257), lambda b: b[:, 1:], [1]),
    ((300, 257), lambda b: b.T, [1]),
    ((3, 70000), lambda b: b, [1]),                 # few long rows: split + second pass
    ((70000, 3), lambda b: b, [0]),                 # few long columns: split + second pass
    ((70000, 3), lambda b: b, [1]),                 # many tiny rows
    ((16, 64, 256), lambda b: b[:, :, ::2], [0, 2]),
    ((16, 64, 256), lambda b: b[:, :, ::2], [1]),
    ((16, 64, 256), lambda b: b[:, :, ::2], [2]),
    ((16, 64, 256), lambda b: b[::-1, :, ::-3], [2, 0]),
    ((5, 6, 7, 8), lambda b: b.transpose(3, 1, 0, 2), [0, 2]),
    ((5, 6, 7, 8), lambda b: b, [0, 1, 2, 3]),
    ((1 << 21,), lambda b: b, [0]),
]


@pytest.mark.parametrize("layout", range(len(LAYOUTS)))
def test_all_value_ops_on_layouts(layout, ctx):
    shape, view, axes = LAYOUTS[layout]
    rng = np.random.default_rng(300 + layout)
    others = ["uint8", "int64", "float64", "int16", "uint32", "int8"]
    for dt in ("int32", "float32", others[layout % len(others)]):
        if np.dtype(dt).kind == "f":
            base = rng.normal(0, 1, shape).astype(dt)
        else:
            base = rng.integers(-3 if np.dtype(dt).kind == "i" else 0, 4, shape).astype(dt)
        v = view(base)
        g, _ = to_gpu_view(v, ctx)
        ops = ["sum", "prod", "prodnz", "all", "any"]
        if np.dtype(dt).kind in "iu":
            ops += ["and", "or", "xor"]
        for op in ops:
            if op in ("sum", "prod", "prodnz"):
                odt = R._upcast(dt)
            elif op in ("all", "any"):
                odt = np.dtype("bool")
            else:
                odt = np.dtype(dt)
            want = np_reduce(op, v, axes, odt if op in ("sum", "prod", "prodnz") else None)
            out = R._reduce_named(g, op, odt, axis=tuple(axes))
            got = np.asarray(out)
            assert got.shape == want.shape, (op, dt)
            if np.dtype(dt).kind == "f" and op in ("sum",):
                x64 = v.astype(np.float64)
                assert_sum_close(got, x64.sum(axis=tuple(axes)), np.abs(x64).sum(axis=tuple(axes)))
            elif np.dtype(dt).kind == "f" and op in ("prod", "prodnz"):
                with np.errstate(all="ignore"):
                    w64 = np_reduce(op, v.astype(np.float64), axes)
                ok = np.isclose(got, w64, rtol=1e-3) | ~np.isfinite(w64) | (np.abs(w64) < 1e-30)
                assert np.all(ok), (op, dt)
            else:
                assert np.array_equal(got, want), (op, dt, layout)
        for op in ("max", "min"):
            want = v.max(axis=tuple(axes)) if op == "max" else v.min(axis=tuple(axes))
            assert np.array_equal(np.asarray(getattr(R, op)(g, axis=tuple(axes))), want), (op, dt)
        wm, wa = np_maxandargmax(v, axes, "min")
        gv, gi = R._arg_reduce(g, "minandargmin", axes, True)
        assert np.array_equal(np.asarray(gv), wm) and np.array_equal(np.asarray(gi), wa), dt
        gi = R._arg_reduce(g, "argmax", axes, False)
        assert np.array_equal(np.asarray(gi), np_maxandargmax(v, axes)[1]), dt


@pytest.mark.parametrize("axes", [(0, 2), (1,), (2,), (0, 1, 2)])
def test_float16_on_stepped_views(ctx, axes):
    """float16 through the stride-2 view of the layouts above (the reference
    refuses float16 sums, pygpu/reduction.py:156-160: NumPy on float64 is the
    only expected value; min/max and their indices are exact)."""
    rng = np.random.default_rng(77)
    base = rng.uniform(-4, 4, (16, 64, 256)).astype(np.float16)
    base[3, 5, 10] = base[3, 5, 200] = np.float16(4.5)          # a tie on a stepped row
    for view in (lambda b: b[:, :, ::2], lambda b: b[::-1, :, ::-3]):
        v = view(base)
        g, _ = to_gpu_view(v, ctx)
        x64 = v.astype(np.float64)
        want, mag = x64.sum(axis=axes), np.abs(x64).sum(axis=axes)
        got32 = np.asarray(R.sum(g, axis=axes, dtype="float32"))
        assert got32.dtype == np.float32
        assert np.allclose(got32, want, rtol=1e-2)               # the stated bound for fp16 inputs
        assert_sum_close(got32, want, mag, cancel=1e-2)          # what fp32 accumulation achieves
        got16 = np.asarray(R.sum(g, axis=axes))
        assert got16.dtype == np.float16 and np.array_equal(got16, got32.astype(np.float16))
        assert np.array_equal(np.asarray(R.max(g, axis=axes)), v.max(axis=axes))
        assert np.array_equal(np.asarray(R.min(g, axis=axes)), v.min(axis=axes))
        for name in ("max", "min"):
            wm, wa = np_maxandargmax(v, list(axes), name)
            gv, gi = R._arg_reduce(g, name + "andarg" + name, list(axes), True)
            assert np.array_equal(np.asarray(gv), wm) and np.array_equal(np.asarray(gi), wa), name
        assert np.array_equal(np.asarray(R.any(g, axis=axes)), v.any(axis=axes))
        assert np.array_equal(np.asarray(R.all(g, axis=axes)), v.all(axis=axes))


@pytest.mark.parametrize("dtype", ["float32", "int32", "uint8", "float16", "float64", "int16"])
def test_short_kept_rows_in_one_launch(ctx, dtype):
    """redux_pcols: kept rows of 1 to 1000 elements (row bytes below 256, or
    not a multiple of 16), totals that end inside a 16-byte chunk, several
    leading and several kept dims, a result with its own strides, a half
    result; sum, product, any / all, integer min / max and the bitwise ones,
    against NumPy (values small enough for every sum to be exact)."""
    rng = np.random.default_rng(1234)
    es = np.dtype(dtype).itemsize
    kept_lengths = [1, 2, 3, 5, 7, 10, 12, 17, 33, 63, 100, 250, 255, 1000]
    launches = []
    for F in kept_lengths:
        rowb = F * es
        if rowb % 16 == 0 and rowb >= 256:
            continue
        R0 = ((6 << 20) // rowb) | 1            # an odd row count: the total ends inside a chunk for most F
        for shape, axes in (((R0, F), (0,)), ((3, R0 // 3 + 1, F), (0, 1))):
            if F == 12:
                shape, axes = (shape[0],) * 1 + shape[1:-1] + (3, 4), axes        # two kept dims
            lo, hi = (0, 3) if np.dtype(dtype).kind == "u" else (-2, 3)
            host = rng.integers(lo, hi, size=shape).astype(dtype)
            g = gpuarray.array(host, context=ctx)
            ctx.kernel_timing(True)
            if np.dtype(dtype).kind == "f":
                got = np.asarray(R.sum(g, axis=axes, dtype="float32"))
                n = len(ctx.kernel_times())
                assert np.array_equal(got, host.sum(axis=axes, dtype=np.float64).astype(np.float32)), (shape, "sum")
            else:
                got = np.asarray(R.sum(g, axis=axes, dtype="int64"))
                n = len(ctx.kernel_times())
                assert np.array_equal(got, host.sum(axis=axes, dtype=np.int64)), (shape, "sum")
            ctx.kernel_timing(False)
            launches.append((F, n))
            for name, npf in (("all", np.all), ("any", np.any)):
                got = np.asarray(R._reduce_named(g, name, np.dtype("bool"), axis=axes))
                assert np.array_equal(got, npf(host, axis=axes)), (shape, name)
            if np.dtype(dtype).kind in "iu":
                for name, npf in (("max", np.max), ("min", np.min)):
                    assert np.array_equal(np.asarray(getattr(R, name)(g, axis=axes)), npf(host, axis=axes)), (shape, name)
                got = np.asarray(R._reduce_named(g, "xor", np.dtype(dtype), axis=axes))
                assert np.array_equal(got, np.bitwise_xor.reduce(host, axis=axes if len(axes) == 1 else None)
                                      if len(axes) == 1 else
                                      np.bitwise_xor.reduce(np.bitwise_xor.reduce(host, axis=0), axis=0)), (shape, "xor")
    # kept rows of 2 to 63 elements of a type whose accumulators fit the lane went out as one launch
    if dtype in ("float32", "float64", "int32", "float16"):
        assert all(n == 1 for F, n in launches if 2 <= F <= 63), launches
    # a result with strides of its own, a half result, a product of +-1
    host = rng.integers(-2, 3, size=(1 << 20, 10)).astype(dtype)
    g = gpuarray.array(host, context=ctx)
    wide = gpuarray.zeros((10, 3), "int64" if np.dtype(dtype).kind in "iu" else "float32", context=ctx)
    ga.GpuReduction(ctx, "sum", dtype)(g, [0], d0=wide[:, 1])
    assert np.array_equal(np.asarray(wide)[:, 1], host.sum(axis=0, dtype=np.float64).astype(np.asarray(wide).dtype))
    assert not np.asarray(wide)[:, 0].any() and not np.asarray(wide)[:, 2].any()
    if dtype == "float16":
        got = np.asarray(R.sum(g, axis=0))
        assert got.dtype == np.float16
        assert np.array_equal(got, host.sum(axis=0, dtype=np.float64).astype(np.float32).astype(np.float16))
    signs = rng.choice(np.array([1, -1]).astype(dtype) if np.dtype(dtype).kind != "u" else np.array([1, 1], dtype), size=(1 << 20, 6))
    got = np.asarray(R._reduce_named(gpuarray.array(signs, context=ctx), "prod", np.dtype(dtype), axis=(0,)))
    assert np.array_equal(got, np.prod(signs.astype(np.float64), axis=0).astype(dtype))


def test_integer_invariants(ctx):
    # exact in any order: permuting the data or reducing axis by axis gives
    # the same integers
    rng = np.random.default_rng(41)
    x = rng.integers(-1000, 1001, (40, 50, 60), dtype=np.int32)
    g = gpuarray.array(x, context=ctx)
    both = np.asarray(R.sum(g, axis=(0, 2)))
    step = np.asarray(R.sum(R.sum(g, axis=2), axis=0))
    assert np.array_equal(both, step) and np.array_equal(both, x.sum(axis=(0, 2)))
    perm = rng.permutation(x.reshape(-1))
    assert np.asarray(R.sum(gpuarray.array(perm, context=ctx))) == x.sum()
    # wrap-around modulo 2^32 when the result type is the input type
    big = np.full(100000, 2 ** 30, np.int32)
    got = np.asarray(R.reduce1(gpuarray.array(big, context=ctx), "+", "0", "int32"))
    assert got == np.int32(np.int64(100000 * 2 ** 30).astype(np.int32))


def test_sum_is_reproducible_run_to_run(ctx):
    rng = np.random.default_rng(42)
    g = gpuarray.array(rng.normal(0, 1, 1 << 22).astype(np.float32), context=ctx)
    first = np.asarray(R.sum(g)).tobytes()
    for _ in range(5):
        assert np.asarray(R.sum(g)).tobytes() == first


# ---- the benchmark's shapes at full size -----------------------------------------------------

def _record(name, **figures):
    """Achieved errors of the benchmark's float sums: printed, and appended to
    float_sum_errors.jsonl in the directory GPUARRAY_TEST_RECORD_DIR names, if
    it names one."""
    import json
    import os
    out = os.environ.get("GPUARRAY_TEST_RECORD_DIR")
    if out:
        try:
            os.makedirs(out, exist_ok=True)
            with open(os.path.join(out, "float_sum_errors.jsonl"), "a") as f:
                f.write(json.dumps(dict(name=name, **figures)) + "\n")
        except OSError:
            pass
    print(name, figures)


def test_config3a_sum_axis1_8192(ctx, oracle):
    x = np.random.default_rng(2).standard_normal((8192, 8192), dtype=np.float32)
    g = gpuarray.array(x, context=ctx)
    got = np.asarray(R.sum(g, axis=1))
    # float64 sums without a float64 copy of the array
    want, mag = x.sum(axis=1, dtype=np.float64), np.abs(x).sum(axis=1, dtype=np.float64)
    worst, fallback = assert_sum_close(got, want, mag, cancel=1e-3)
    # Rows of 8192 N(0,1) values: |sum| ~ 90, sum of magnitudes ~ 6536, so
    # about 6 % of the rows are cancellations below 1e-3 of it; every other
    # row is held to 1e-5 relative.
    assert fallback <= 0.08, fallback
    _record("C3a sum axis 1 of 8192x8192", max_relative_error=worst, rows_on_fallback=fallback)
    # the reference's own order (one group per row, pygpu/reduction.py:85-132)
    # on the first rows, at its tolerance
    chk = oracle.reduk("sum", x[:64], [1], "float32", ls=256)
    assert np.allclose(got[:64], chk, rtol=2e-5, atol=1e-3)
    # and the other axis (column kernel)
    got0 = np.asarray(R.sum(g, axis=0))
    worst0, fallback0 = assert_sum_close(got0, x.sum(axis=0, dtype=np.float64),
                                         np.abs(x).sum(axis=0, dtype=np.float64), cancel=1e-3)
    assert fallback0 <= 0.08, fallback0
    _record("sum axis 0 of 8192x8192", max_relative_error=worst0, rows_on_fallback=fallback0)


def test_config3b_full_sum_2p28(ctx):
    n = 1 << 28
    x = np.random.default_rng(3).standard_normal(n, dtype=np.float32)
    g = gpuarray.array(x, context=ctx)
    got = float(np.asarray(R.sum(g)))
    want = float(x.sum(dtype=np.float64))
    assert abs(got - want) <= 1e-5 * abs(want), (got, want)
    _record("C3b full sum of 2^28", relative_error=abs(got - want) / abs(want), sum=want)
    # size-independent properties: the halves add up, and a shifted copy adds n*shift
    h = float(np.asarray(R.sum(g[:n // 2]))) + float(np.asarray(R.sum(g[n // 2:])))
    assert abs(h - want) <= 1e-5 * abs(want)
    ones = gpuarray.empty((n,), "float32", context=ctx)
    ga.GpuElemwise(ctx, "o = 1.0f", [ga.arg("o", "float32", write=True)])(ones)
    assert float(np.asarray(R.sum(ones))) == float(n)          # exact: all partials are integers
    v, i = R.maxandargmax(g)
    assert float(np.asarray(v)) == float(x.max()) and int(np.asarray(i)) == int(x.argmax())


def test_config4_maxandargmax_logits(ctx, oracle):
    """BASELINE configuration 4 at its stated shape: maxandargmax over the last
    axis of (65536, 1000) normal(0, 2) floats, 5 % of the rows with their
    maximum copied into one to three other columns.  Through the C entry point
    (reference tests/check_reduction.c:85-160 checks it against a CPU loop)."""
    rng = np.random.default_rng(4)
    x = rng.normal(0, 2, (65536, 1000)).astype(np.float32)
    rows = rng.choice(65536, 3277, replace=False)              # 5 % of the rows get duplicated maxima
    for r in rows:
        cols = rng.choice(1000, int(rng.integers(1, 4)), replace=False)
        x[r, cols] = x[r].max()
    g = gpuarray.array(x, context=ctx)
    gmax = gpuarray.empty((65536,), "float32", context=ctx)
    garg = gpuarray.empty((65536,), "uint64", context=ctx)
    arr = (C.c_uint * 1)(1)
    assert lib.GpuArray_maxandargmax(gmax._ptr(), garg._ptr(), g._ptr(), 1, arr) == 0
    got_m, got_a = np.asarray(gmax), np.asarray(garg).astype(np.int64)
    assert np.array_equal(got_m, x.max(axis=1))
    assert np.array_equal(got_a, x.argmax(axis=1))             # NumPy: first index on ties
    # the rows really hold ties, and the first of them is what came back
    tied = (x[rows] == x[rows].max(axis=1, keepdims=True)).sum(axis=1)
    assert (tied >= 2).sum() >= 3200     # (a drawn column can be the maximum's own)
    wm, wa = oracle.maxandargmax(x[rows[:512]], [1])           # the reference's scan on tied rows
    assert np.array_equal(got_m[rows[:512]], wm) and np.array_equal(got_a[rows[:512]], wa)
    # the Python-level entry point takes the same kernels
    v, i = R.maxandargmax(g, axis=1)
    assert np.array_equal(np.asarray(v), got_m) and np.array_equal(np.asarray(i), got_a)


def test_config5_mixed_dtypes_strided(ctx, oracle):
    """BASELINE configuration 5 at its stated shape: a (256, 512, 1024) array
    taken with a step of 2 along the last axis; fp16 summed over axes (0, 2)
    into fp32, int32 summed over axis 1, uint8 any / all over axis 2
    (reference pattern: pygpu/tests/test_reduction.py:86-110)."""
    shape = (256, 512, 1024)
    rng = np.random.default_rng(5)
    h = rng.uniform(-4, 4, shape).astype(np.float16)
    gh = gpuarray.array(h, context=ctx)[:, :, ::2]
    assert gh.shape == (256, 512, 512) and gh.strides == (1048576, 2048, 4)
    got = np.asarray(R.sum(gh, axis=(0, 2), dtype="float32"))
    want = h[:, :, ::2].astype(np.float64).sum(axis=(0, 2))
    assert got.dtype == np.float32 and np.allclose(got, want, rtol=1e-2)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-2)
    del gh, h

    rng = np.random.default_rng(6)
    i32 = rng.integers(-1000, 1001, shape, dtype=np.int32)
    gi = gpuarray.array(i32, context=ctx)[:, :, ::2]
    got = np.asarray(R.sum(gi, axis=1))
    assert got.dtype == np.int64 and np.array_equal(got, i32[:, :, ::2].sum(axis=1))
    got32 = np.asarray(R.sum(gi, axis=1, dtype="int32"))
    assert np.array_equal(got32, i32[:, :, ::2].sum(axis=1, dtype=np.int32))
    chk = oracle.reduk("sum", i32[:4, :, ::2], [1], "int64", ls=64)
    assert np.array_equal(got[:4], chk)
    del gi, i32

    rng = np.random.default_rng(7)
    u8 = (rng.random(shape) < 1e-4).astype(np.uint8)
    gu = gpuarray.array(u8, context=ctx)[:, :, ::2]
    any_, all_ = np.asarray(R.any(gu, axis=2)), np.asarray(R.all(gu, axis=2))
    assert any_.dtype == np.bool_ and np.array_equal(any_, u8[:, :, ::2].any(axis=2))
    assert np.array_equal(all_, u8[:, :, ::2].all(axis=2)) and not all_.any()
    assert 0 < any_.sum() < any_.size                          # the test data exercises both answers
    chk_any = oracle.reduk("any", u8[:2, :, ::2], [2], "bool", ls=64)
    assert np.array_equal(any_[:2], chk_any.astype(bool))
    ones = gpuarray.array(np.ones((8, 16, 64), np.uint8), context=ctx)[:, :, ::2]
    assert np.asarray(R.all(ones, axis=2)).all()


# ---- reduced dims with outer ones side by side, several outputs per lane ----------

def _check_ops(ctx, host, axes):
    """sum (exact for ints, 1e-5 for floats), maxandargmax and minandargmin
    (bit-exact, first index on ties) of `host` over `axes`."""
    g, _ = to_gpu_view(host, ctx)
    axes = tuple(axes)
    if host.dtype.kind in "iu":
        got = np.asarray(R.sum(g, axis=axes, dtype="int64"))
        assert np.array_equal(got, host.sum(axis=axes, dtype=np.int64))
    else:
        got = np.asarray(R.sum(g, axis=axes))
        want = host.sum(axis=axes, dtype=np.float64)
        scale = np.abs(host).sum(axis=axes, dtype=np.float64)
        assert_sum_close(got, want, scale)
    # flattened index over the reduced axes in ascending order = NumPy's on the moved array
    moved = np.moveaxis(host, axes, range(host.ndim - len(axes), host.ndim))
    flat = moved.reshape(moved.shape[:host.ndim - len(axes)] + (-1,))
    for name, fn, afn in (("maxandargmax", np.max, np.argmax), ("minandargmin", np.min, np.argmin)):
        val, idx = getattr(R, name)(g, axis=axes)
        assert np.array_equal(np.asarray(val), fn(flat, axis=-1)), name
        assert np.array_equal(np.asarray(idx), afn(flat, axis=-1)), name


@pytest.mark.parametrize("dtype", ["float32", "int32", "uint8", "float64"])
def test_short_rows_share_a_wavefront(ctx, dtype):
    rng = np.random.default_rng(50)
    for shape in ((1000, 1), (1000, 2), (1000, 3), (1003, 4), (517, 8), (777, 33), (513, 100),
                  (129, 250), (65, 511), (70000, 5)):
        host = rng.integers(0, 50, size=shape).astype(dtype)          # many ties
        _check_ops(ctx, host, [1])
    # rows that are not contiguous in the free direction, and a stepped inner dim
    base = rng.integers(0, 50, size=(301, 40)).astype(dtype)
    _check_ops(ctx, base[::3, :12], [1])
    _check_ops(ctx, base[::-1, ::2], [1])


@pytest.mark.parametrize("dtype", ["float32", "int32", "uint8", "float16", "float64", "int16"])
def test_short_contiguous_rows_staged_in_lds(ctx, dtype, knobs):
    """Many short rows lying one after the other take the kernel that stages a
    group's rows in LDS (here from 1000 rows on, so that the case stays
    small): every row length up to the limit, starts off the 16-byte boundary,
    a last group that is not full, ties, and NaN / signed zero placement."""
    knobs(REDUX_SROWS_MIN_ROWS=1)
    rng = np.random.default_rng(54)
    item = np.dtype(dtype).itemsize
    # up to 256 bytes per row, 384 where the row length is no multiple of 16 bytes
    lengths = [n for n in (2, 3, 5, 6, 7, 8, 12, 16, 17, 31, 32, 33, 47, 48, 63, 64, 91, 100, 128, 181,
                           255, 256, 333, 383)
               if 16 < n * item <= (384 if (n * item) % 16 else 256)]
    for n in lengths:
        rows = int(rng.integers(300, 1500))
        flat = rng.integers(0, 12, size=rows * n + 7).astype(dtype)      # many ties
        for off in (0, 1, 3):
            host = flat[off:off + rows * n].reshape(rows, n)
            if dtype == "float16":
                g, _ = to_gpu_view(host, ctx)
                val, idx = R.maxandargmax(g, axis=1)
                assert np.array_equal(np.asarray(val), host.max(axis=1))
                assert np.array_equal(np.asarray(idx), host.argmax(axis=1))
                got = np.asarray(R.sum(g, axis=1, dtype="float32"))
                assert np.array_equal(got, host.astype(np.float32).sum(axis=1))   # small integers: exact
            else:
                _check_ops(ctx, host, [1])
    if dtype in ("float32", "float64"):
        host = rng.standard_normal((2000, 33)).astype(dtype)
        host[5, 0] = np.nan            # element 0: the result is NaN at index 0
        host[6, 7] = np.nan            # elsewhere: ignored
        host[7, :] = 0.0
        host[7, 4] = -0.0              # equal to the zeros before it: index 0 stays
        host[8, :] = -0.0
        host[8, 9] = 0.0
        g, _ = to_gpu_view(host, ctx)
        val, idx = R.maxandargmax(g, axis=1)
        val, idx = np.asarray(val), np.asarray(idx)
        assert np.isnan(val[5]) and idx[5] == 0
        assert val[6] == np.nanmax(host[6]) and idx[6] == np.nanargmax(host[6])
        assert idx[7] == 0 and not np.signbit(val[7])
        assert idx[8] == 0 and np.signbit(val[8])
        keep = np.ones(2000, bool)
        keep[[5, 6]] = False
        assert np.array_equal(val[keep], host[keep].max(axis=1))
        assert np.array_equal(idx[keep], host[keep].argmax(axis=1))
    if dtype == "uint8":
        host = (rng.random((5000, 40)) < 0.02).astype(dtype)
        g, _ = to_gpu_view(host, ctx)
        assert np.array_equal(np.asarray(R.any(g, axis=1)), host.any(axis=1))
        assert np.array_equal(np.asarray(R.all(g, axis=1)), host.all(axis=1))
        ones = np.ones((5000, 40), dtype)
        ones[17, 39] = 0
        g, _ = to_gpu_view(ones, ctx)
        assert np.array_equal(np.asarray(R.all(g, axis=1)), ones.all(axis=1))


@pytest.mark.parametrize("dtype", ["float32", "int32", "uint8", "float16", "float64", "int16", "int64"])
def test_tiny_contiguous_rows_walked_in_registers(ctx, dtype, knobs):
    """Rows of at most 32 bytes lying one after the other, the first on a
    16-byte boundary, take the kernel that keeps a lane's rows in registers
    (here from one row on and for every row length it can take, so that the
    cases stay small): row lengths with one, two and more chunks per lane, a
    last lane whose run of rows is cut short, a view that starts inside its
    buffer (on a boundary, and off one: that one falls back), every
    operation, ties, NaN and signed zero placement."""
    knobs(REDUX_TROWS_MIN_ROWS=1, REDUX_TROWS_DIRECT=2)
    rng = np.random.default_rng(57)
    item = np.dtype(dtype).itemsize
    lengths = [n for n in (2, 3, 4, 5, 6, 7, 8, 12, 14, 16, 32) if n * item <= 32]
    per16 = 16 // item
    for n in lengths:
        rows = int(rng.integers(257, 900))
        flat = rng.integers(0, 12, size=rows * n + 2 * per16 + 3).astype(dtype)      # many ties
        for off in (0, per16, 1) if n in (3, 4) else (0, per16):
            host = flat[off:off + rows * n].reshape(rows, n)
            g, _ = to_gpu_view(host, ctx)
            if dtype == "float16":
                val, idx = R.maxandargmax(g, axis=1)
                assert np.array_equal(np.asarray(val), host.max(axis=1)), (n, off)
                assert np.array_equal(np.asarray(idx), host.argmax(axis=1)), (n, off)
                got = np.asarray(R.sum(g, axis=1, dtype="float32"))
                assert np.array_equal(got, host.astype(np.float32).sum(axis=1)), (n, off)   # small integers: exact
                continue
            _check_ops(ctx, host, [1])
            if n not in (3, 4):      # every row length is a kernel of its own: the other operations on two of them
                continue
            ops = ["prod", "prodnz", "all", "any"] + (["and", "or", "xor"] if np.dtype(dtype).kind in "iu" else [])
            small = host % 3 if np.dtype(dtype).kind in "iu" else host
            gs, _ = to_gpu_view(small, ctx)
            for op in ops:
                odt = R._upcast(dtype) if op in ("prod", "prodnz") else np.dtype("bool") if op in ("all", "any") else np.dtype(dtype)
                want = np_reduce(op, small, [1], odt if op in ("prod", "prodnz") else None)
                got = np.asarray(R._reduce_named(gs, op, odt, axis=(1,)))
                if np.dtype(dtype).kind == "f" and op in ("prod", "prodnz"):
                    assert np.allclose(got, np_reduce(op, small.astype(np.float64), [1]), rtol=1e-4), (op, n, off)
                else:
                    assert np.array_equal(got, want), (op, n, off)
            assert np.array_equal(np.asarray(R.min(g, axis=(1,))), host.min(axis=1))
            assert np.array_equal(np.asarray(R._arg_reduce(g, "argmin", [1], False)), host.argmin(axis=1))
            # results that do not lie side by side, or start off the boundary of a lane's store
            for dst in (gpuarray.zeros((2 * rows,), dtype, context=ctx)[::2],
                        gpuarray.zeros((rows + 1,), dtype, context=ctx)[1:]):
                R._reduce_named(g, "max", np.dtype(dtype), axis=(1,), out=dst)
                assert np.array_equal(np.asarray(dst), host.max(axis=1)), (n, off)
    if np.dtype(dtype).kind == "f":
        n = 32 // item - 1
        host = rng.integers(-20, 20, size=(3001, n)).astype(dtype)
        nan_first = rng.choice(3001, 40, replace=False)
        host[nan_first[:20], 0] = np.nan                          # stays
        host[nan_first[20:], rng.integers(1, n, 20)] = np.nan     # ignored
        host[nan_first[3], :] = np.nan
        host[7, :] = 0.0
        host[7, 2] = -0.0              # equal to the zeros before it: index 0 stays
        host[8, :] = -0.0
        host[8, 1] = 0.0
        g, _ = to_gpu_view(host, ctx)
        for name, nanfn, argfn in (("maxandargmax", np.nanmax, np.nanargmax), ("minandargmin", np.nanmin, np.nanargmin)):
            val, idx = getattr(R, name)(g, axis=1)
            val, idx = np.asarray(val), np.asarray(idx)
            for r in range(3001):
                if np.isnan(host[r, 0]):
                    assert np.isnan(val[r]) and idx[r] == 0, (name, r)
                else:
                    assert val[r] == nanfn(host[r]) and idx[r] == argfn(host[r]), (name, r)
            assert idx[7] == 0 and not np.signbit(val[7])
            assert idx[8] == 0 and np.signbit(val[8])


@pytest.mark.parametrize("dtype", ["float32", "float64", "float16"])
@pytest.mark.parametrize("staged", [0, 1])
def test_nan_in_first_position_of_short_rows(ctx, dtype, staged, knobs):
    """The NaN rule of the sequential scan (a NaN stays only when it is the
    first element) in the kernels that take it from their own registers: rows
    sharing a wavefront in every lane geometry, rows shifted to a load
    boundary, one row per wavefront, rows staged in LDS."""
    knobs(REDUX_SROWS=staged, REDUX_SROWS_MIN_ROWS=1)
    rng = np.random.default_rng(55)
    for n in (2, 3, 4, 8, 15, 16, 33, 64, 100, 129, 250, 513, 1000, 1001):
        rows = 131
        host = rng.integers(-20, 20, size=(rows, n)).astype(dtype)
        first = rng.choice(rows, 20, replace=False)
        host[first[:10], 0] = np.nan                     # stays
        host[first[10:], rng.integers(1, n, 10)] = np.nan   # ignored
        host[first[3], :] = np.nan                       # all NaN
        flat = np.concatenate([np.zeros(1, dtype), host.ravel()])
        for view in (host, flat[1:].reshape(rows, n)):   # aligned, and one element off
            g, _ = to_gpu_view(view, ctx)
            for name, nanfn, argfn in (("maxandargmax", np.nanmax, np.nanargmax),
                                       ("minandargmin", np.nanmin, np.nanargmin)):
                val, idx = getattr(R, name)(g, axis=1)
                val, idx = np.asarray(val), np.asarray(idx)
                for r in range(rows):
                    if np.isnan(view[r, 0]):
                        assert np.isnan(val[r]) and idx[r] == 0, (name, n, r)
                    else:
                        assert val[r] == nanfn(view[r]) and idx[r] == argfn(view[r]), (name, n, r)


def _strict_scan(row, better):
    """The reference's scan (src/gpuarray_reduction.c:545-607): the first
    element, then every later one that compares strictly better."""
    bv, bi = row[0], 0
    for i in range(1, len(row)):
        if better(row[i], bv):
            bv, bi = row[i], i
    return bv, bi


@pytest.mark.parametrize("dtype", ["float32", "float64", "float16"])
@pytest.mark.parametrize("staged", [0, 1])
def test_nans_among_values_equal_to_the_neutral_element(ctx, dtype, staged, knobs):
    """Rows of NaN, -inf and +inf only (few finite values): a NaN loses every
    compare, a value equal to the scan's starting value never replaces it, so
    the answer is the row's first element unless a later one beats it, and
    the first of the equals among those.  Over rows (every short-row kernel)
    and over columns."""
    knobs(REDUX_SROWS=staged, REDUX_SROWS_MIN_ROWS=1, REDUX_TROWS_MIN_ROWS=1)
    rng = np.random.default_rng(66)
    pool = np.array([np.nan, np.nan, -np.inf, -np.inf, np.inf, 1.0], dtype)
    for n in (2, 3, 4, 6, 8, 15, 16, 24, 32, 33, 64, 100, 250, 1001):
        rows = 97
        for lo_only in (True, False):
            host = pool[rng.integers(0, 4 if lo_only else 6, size=(rows, n))]
            host[:8, 0] = np.nan
            host[8:16, 0] = -np.inf
            for axis, view in ((1, host), (0, np.ascontiguousarray(host.T))):
                g, _ = to_gpu_view(view, ctx)
                seq = host
                for name, better in (("maxandargmax", lambda a, b: a > b), ("minandargmin", lambda a, b: a < b)):
                    data = seq if name == "maxandargmax" else -seq
                    gd = g if name == "maxandargmax" else to_gpu_view(-view, ctx)[0]
                    val, idx = getattr(R, name)(gd, axis=axis)
                    val, idx = np.asarray(val), np.asarray(idx)
                    for r in range(rows):
                        wv, wi = _strict_scan(data[r], better)
                        assert idx[r] == wi and (val[r] == wv or (np.isnan(wv) and np.isnan(val[r]))), \
                            (name, n, axis, r, lo_only, data[r][:8])


@pytest.mark.parametrize("dtype", ["uint8", "int8", "bool"])
def test_one_byte_elements_four_per_operation(ctx, dtype):
    """sum / any / all over one-byte elements (combined a 32-bit word at a
    time): extreme values, every alignment of start and end, stepped views,
    long rows split over groups, rows sharing a wavefront."""
    rng = np.random.default_rng(56)

    def make(shape):
        if dtype == "bool":
            return rng.random(shape) < 0.5
        info = np.iinfo(dtype)
        h = rng.integers(info.min, info.max + 1, size=shape).astype(dtype)
        h.reshape(-1)[::7] = info.max
        h.reshape(-1)[3::11] = info.min
        return h

    def check(view, axes):
        g, _ = to_gpu_view(view, ctx)
        axes = tuple(axes)
        want = view.sum(axis=axes, dtype=np.int64)
        assert np.array_equal(np.asarray(R.sum(g, axis=axes, dtype="int64")), want)
        if dtype != "int8":
            assert np.array_equal(np.asarray(R.sum(g, axis=axes, dtype="uint32")), want.astype(np.uint32))
        assert np.array_equal(np.asarray(R.any(g, axis=axes)), view.any(axis=axes))
        assert np.array_equal(np.asarray(R.all(g, axis=axes)), view.all(axis=axes))

    for shape in ((64, 8192), (300, 1000), (1000, 33), (513, 100), (7, 70001), (2000, 16), (3, 1 << 20)):
        check(make(shape), [1])
    flat = make((1 << 22) + 37)
    for off, n in ((0, 1 << 22), (1, (1 << 22) + 3), (5, 1 << 21), (16, (1 << 22) - 15), (3, 100003)):
        check(flat[off:off + n], [0])
    base = make((256, 4096))
    check(base[:, ::2], [1])
    check(base[:, 1::4], [1])
    check(base[:, 3:4001], [1])
    check(base[::3, 5::2], [1])
    # where any / all flip on a single element in every byte position of a word
    for pos in range(0, 40):
        z = np.zeros((4, 4099), dtype)
        z[1, pos] = 1
        z[2, 4098 - pos] = 1
        o = np.ones((4, 4099), dtype)
        o[1, pos] = 0
        o[3, 4098 - pos] = 0
        for h in (z, o, z[:, 1:], o[:, 2:4097]):
            g, _ = to_gpu_view(h, ctx)
            assert np.array_equal(np.asarray(R.any(g, axis=1)), h.any(axis=1)), pos
            assert np.array_equal(np.asarray(R.all(g, axis=1)), h.all(axis=1)), pos


@pytest.mark.parametrize("dtype", ["float32", "int32", "float64", "uint8", "int16"])
def test_short_inner_dim_with_outer_reduced_dims(ctx, dtype):
    rng = np.random.default_rng(51)
    for shape, axes in (((32, 16, 7, 7), (0, 2, 3)), ((16, 24, 16, 20), (1, 3)), ((9, 5, 3), (0, 2)),
                        ((40, 3, 50, 4), (0, 3)), ((6, 7, 1030, 2), (0, 1, 3)), ((300, 2, 16), (0, 2))):
        host = rng.integers(0, 30, size=shape).astype(dtype)
        _check_ops(ctx, host, axes)
    # enough outer coordinates for the range to be split into partials
    host = rng.integers(0, 30, size=(4096, 3, 12)).astype(dtype)
    _check_ops(ctx, host, (0, 2))


@pytest.mark.parametrize("dtype", ["float32", "int32", "uint8", "int8", "int16", "float64", "float16"])
def test_several_outputs_per_lane(ctx, dtype):
    rng = np.random.default_rng(52)
    # (the 8192-wide cases have enough outputs for split-major partials; the narrow ones
    # take 8 or 16 lane rows)
    shapes = ((300, 1000), (8, 4096), (1000, 256), (37, 20), (513, 772), (4, 64, 260), (2000, 8192),
              (5, 300, 4096), (3000, 64), (7, 1500, 32), (1201, 16), (900, 8), (4000, 100))
    for shape in shapes:
        host = rng.integers(0, 40, size=shape).astype(dtype)
        if dtype == "float16":
            g, _ = to_gpu_view(host, ctx)
            val, idx = R.maxandargmax(g, axis=0)
            assert np.array_equal(np.asarray(val), host.max(axis=0))
            assert np.array_equal(np.asarray(idx), host.argmax(axis=0))
            continue
        _check_ops(ctx, host, [0])
    # misaligned bases and strides fall back to narrower loads
    base = rng.integers(0, 40, size=(300, 1001)).astype(dtype if dtype != "float16" else "float32")
    _check_ops(ctx, base[:, 1:], [0])
    _check_ops(ctx, base[:, :1000], [0])
    _check_ops(ctx, base[::2, 2:998:2], [0])


@pytest.mark.parametrize("dtype", ["float32", "int32", "uint8", "float16", "float64"])
def test_ragged_and_misaligned_rows_take_vector_loads(ctx, dtype):
    """Rows whose length is not a multiple of the load, or that start at an
    address that is only element-aligned: every element still counts once."""
    rng = np.random.default_rng(53)
    for shape in ((300, 1023), (7, 4097), (64, 33), (1, 100003), (5, 4), (129, 17), (3, 70001)):
        host = rng.integers(0, 40, size=shape).astype(dtype)
        if dtype == "float16":
            g, _ = to_gpu_view(host, ctx)
            val, idx = R.maxandargmax(g, axis=1)
            assert np.array_equal(np.asarray(val), host.max(axis=1))
            assert np.array_equal(np.asarray(idx), host.argmax(axis=1))
            got = np.asarray(R.sum(g, axis=1, dtype="float32"))
            assert np.array_equal(got, host.astype(np.float32).sum(axis=1))     # small integers: exact
            continue
        _check_ops(ctx, host, [1])
    base = rng.integers(0, 40, size=(50, 2051)).astype(dtype if dtype != "float16" else "float32")
    _check_ops(ctx, base[:, 1:], [1])           # aligned length, misaligned start
    _check_ops(ctx, base[:, 3:2050], [1])
    _check_ops(ctx, base[::-1, 2:], [1])
    flat = rng.integers(0, 40, size=(1 << 22) + 5).astype(dtype if dtype != "float16" else "float32")
    _check_ops(ctx, flat[1:], [0])              # split over many groups, ragged end
    _check_ops(ctx, flat[3:-1], [0])


@pytest.mark.parametrize("dtype", ["float32", "float64", "float16", "int8", "uint8", "int16", "int32", "int64"])
def test_column_scans_keep_the_first_of_equals(ctx, dtype):
    """Arg-min/max (and floating min/max) with lanes along the free dim: a lane
    scans its share of the reduced range in rising order with a strict compare
    when the index rises along the scan, else with the index compare.  Columns
    that hold only the scan's starting value (type minimum / maximum, -inf /
    +inf), ties within a lane and between lanes and splits, NaN after the
    first position, signed zeros; reduced ranges of one dim, of two dims in
    index order, and of two dims whose memory order is not the index order."""
    rng = np.random.default_rng(77)
    dt = np.dtype(dtype)
    lo, hi = ((-np.inf, np.inf) if dt.kind == "f" else (np.iinfo(dt).min, np.iinfo(dt).max))
    for shape, axes in (((700, 96), (0,)), ((5000, 256), (0,)), ((9, 130, 64), (0, 1)),
                        ((40, 2, 33, 128), (0, 2)), ((64, 8192), (0,)), ((2100, 8), (0,))):
        host = rng.integers(0, 3, size=shape).astype(dt)                  # ties everywhere
        cols = host.reshape(-1, shape[-1])
        cols[:, 0] = lo                                                   # only the starting value of a max scan
        cols[:, 1] = hi                                                   # ... of a min scan
        cols[:, 2] = lo; cols[cols.shape[0] // 2:, 2] = hi
        cols[:, 3] = hi; cols[cols.shape[0] // 3, 3] = lo
        if dt.kind == "f":
            cols[5, 4] = np.nan                                           # not first: passed over
            cols[0, 5] = np.nan                                           # first: stays
            cols[:, 6] = -0.0; cols[cols.shape[0] - 2, 6] = 0.0           # equal zeros
            cols[:, 7] = 0.0; cols[3, 7] = -0.0
        views = [host]
        if len(axes) == 2:
            # the same values with the two reduced dims swapped in memory: the scan no
            # longer meets the elements in index order
            order = list(range(host.ndim))
            order[axes[0]], order[axes[1]] = order[axes[1]], order[axes[0]]
            views.append(np.ascontiguousarray(host.transpose(order)).transpose(order))
        for v in views:
            g, _ = to_gpu_view(v, ctx)
            moved = np.moveaxis(v, axes, range(v.ndim - len(axes), v.ndim))
            flat = moved.reshape(moved.shape[:v.ndim - len(axes)] + (-1,))
            for name, better in (("maxandargmax", np.greater), ("minandargmin", np.less)):
                # sequential scan with a strict compare, as the reference's kernel does it
                want_v = flat[..., 0].copy()
                want_i = np.zeros(flat.shape[:-1], np.int64)
                for j in range(1, flat.shape[-1]):
                    b = better(flat[..., j], want_v)
                    want_v = np.where(b, flat[..., j], want_v)
                    want_i = np.where(b, j, want_i)
                val, idx = getattr(R, name)(g, axis=axes)
                assert np.array_equal(np.asarray(idx), want_i), (name, shape, axes, v.strides)
                got = np.asarray(val)
                bits = "u%d" % dt.itemsize
                assert np.array_equal(got.view(bits), want_v.astype(dt).view(bits)), (name, shape, axes)
                if dt.kind == "f":
                    plain = np.asarray(getattr(R, name[:3])(g, axis=axes))
                    assert np.array_equal(plain.view(bits), want_v.astype(dt).view(bits)), (name[:3], shape)


def test_split_reductions_finish_in_one_launch(ctx, knobs):
    """A reduction whose outputs are cut into pieces: the piece that finishes
    last combines the partials in the same launch (a counter per output, or per
    tile of outputs of the column kernel, that the launch leaves at zero).
    Many such calls in a row on changing shapes, against NumPy, against the
    two-launch path, and twice for bit-identical float results."""
    rng = np.random.default_rng(91)
    cases = []
    for n in (1 << 16, (1 << 18) + 3, 1 << 20, (1 << 22) - 5):
        cases.append(((n,), (0,)))
    cases += [((4, 1 << 20), (1,)), ((16, 1 << 18), (1,)), ((3, 5, 1 << 16), (1, 2)),     # rows in pieces
              ((4096, 256), (0,)), ((100000, 64), (0,)), ((70, 3000, 40), (1,)),          # columns in pieces
              ((20000, 1000), (0,)), ((1 << 19, 8), (0,))]
    # long pieces: beyond one group per compute unit the single launch is taken again
    long_pieces = [((1 << 26,), (0,)), ((64, 1 << 20), (1,)), ((2048, 32768), (0,))]
    for rep in range(2):
        for dtype in ("float32", "int32", "float64"):
            for shape, axes in cases + (long_pieces if rep == 0 and dtype != "float64" else []):
                host = rng.integers(-30, 30, size=shape).astype(dtype)
                g, _ = to_gpu_view(host, ctx)
                if host.dtype.kind == "i":
                    got = np.asarray(R.sum(g, axis=axes, dtype="int64"))
                    assert np.array_equal(got, host.sum(axis=axes, dtype=np.int64)), (shape, axes)
                else:
                    got = np.asarray(R.sum(g, axis=axes))
                    want = host.sum(axis=axes, dtype=np.float64)
                    scale = np.abs(host).sum(axis=axes, dtype=np.float64)
                    assert np.all(np.abs(got - want) <= 1e-5 * np.maximum(scale, 1e-30)), (shape, axes)
                    again = np.asarray(R.sum(g, axis=axes))
                    assert np.array_equal(got.view("u%d" % got.dtype.itemsize),
                                          again.view("u%d" % got.dtype.itemsize)), (shape, axes)
                moved = np.moveaxis(host, axes, range(host.ndim - len(axes), host.ndim))
                flat = moved.reshape(moved.shape[:host.ndim - len(axes)] + (-1,))
                val, idx = R.maxandargmax(g, axis=axes)
                assert np.array_equal(np.asarray(val), flat.max(axis=-1)), (shape, axes)
                assert np.array_equal(np.asarray(idx), flat.argmax(axis=-1)), (shape, axes)
    # the same slots of the partials carry other values in every call: a piece that
    # read a leftover of the call before would show
    for shape, axes in (((1 << 20,), (0,)), ((8, 1 << 18), (1,)), ((4096, 256), (0,))):
        g = gpuarray.zeros(shape, "int32", context=ctx)
        count = int(np.prod([shape[a] for a in axes]))
        for k in range(1, 120):
            g[...] = np.int32(k if k % 3 else -k)
            got = np.asarray(R.sum(g, axis=axes, dtype="int64"))
            assert np.all(got == count * (k if k % 3 else -k)), (shape, k)
    # the two-launch path gives the same integers and indices
    host = rng.integers(-30, 30, size=(100000, 64)).astype("int32")
    flat = rng.integers(-30, 30, size=(1 << 20) + 1).astype("float32")
    g, _ = to_gpu_view(host, ctx)
    gf, _ = to_gpu_view(flat, ctx)
    one = (np.asarray(R.sum(g, axis=0, dtype="int64")), np.asarray(R.maxandargmax(gf)[1]))
    knobs(REDUX_FUSED=0)
    two = (np.asarray(R.sum(g, axis=0, dtype="int64")), np.asarray(R.maxandargmax(gf)[1]))
    knobs(REDUX_FUSED=None)
    assert np.array_equal(one[0], two[0]) and np.array_equal(one[0], host.sum(axis=0, dtype=np.int64))
    assert one[1] == two[1] == flat.argmax()
    # NaN in the first position of a cut row stays; later NaNs are passed over
    x = rng.normal(size=1 << 20).astype("float32")
    x[0] = np.nan
    x[5000] = np.nan
    gx, _ = to_gpu_view(x, ctx)
    v, i = R.maxandargmax(gx)
    assert np.isnan(np.asarray(v)) and int(np.asarray(i)) == 0
    x[0] = -1.0
    gx, _ = to_gpu_view(x, ctx)
    v, i = R.maxandargmax(gx)
    assert np.asarray(v) == np.nanmax(x) and int(np.asarray(i)) == int(np.nanargmax(x))


@pytest.mark.parametrize("loose", [1, 0])
@pytest.mark.parametrize("dtype", ["float32", "int32", "uint32"])
def test_column_reductions_of_four_byte_elements_on_any_layout(ctx, knobs, dtype, loose):
    """Reductions over leading or middle axes whose kept rows start at any
    element and have any length (REDUX_COL_LOOSE: a lane still takes four
    adjacent outputs, with loads that assume four-byte boundaries only; the
    lane at the end of a row takes what exists of its four one by one).
    Kept rows of 4 to 1001 elements inside wider buffers, every phase of the
    first element, one and several pieces of the reduced range (with the
    finish in the same launch and in a second one), folded rows switched off
    so that dense arrays come here too; results against NumPy, exact."""
    knobs(REDUX_COL_LOOSE=loose, REDUX_COL_LOOSE_MIN_BYTES=1, REDUX_FOLD=0, REDUX_PCOLS=0)
    rng = np.random.default_rng(870 + loose)
    draw = lambda shape: rng.integers(0 if dtype == "uint32" else -20, 21, size=shape).astype(dtype)
    ops = [("sum", lambda g, ax: R.sum(g, axis=ax),
            lambda v, ax: v.sum(axis=ax, dtype=np.float64 if dtype == "float32" else np.int64))]
    if dtype != "float32":
        ops += [("max", lambda g, ax: R.max(g, axis=ax), lambda v, ax: v.max(axis=ax)),
                ("min", lambda g, ax: R.min(g, axis=ax), lambda v, ax: v.min(axis=ax))]
    if dtype == "uint32":
        ops += [("xor", lambda g, ax: R._reduce_named(g, "xor", g.dtype, axis=ax),
                 lambda v, ax: np.bitwise_xor.reduce(v, axis=ax))]
    for rows, n, lead, pad in ((33, 4, 1, 0), (700, 5, 0, 0), (70, 7, 3, 2), (1500, 131, 2, 1), (64, 1001, 0, 0),
                               (5000, 66, 1, 1), (9, 1001, 3, 0), (40000, 9, 0, 2), (2100, 259, 1, 0)):
        root = draw((rows, lead + n + pad))
        view = root[:, lead:lead + n]
        g, _ = to_gpu_view(view, ctx)
        for name, call, want in ops:
            assert np.array_equal(np.asarray(call(g, 0)), want(view, 0)), (name, rows, n, lead, pad)
    # a middle axis, and the two outer axes of three
    root = draw((6, 300, 70 + 3))
    view = root[:, :, 2:72 - 1]
    g, _ = to_gpu_view(view, ctx)
    for name, call, want in ops:
        assert np.array_equal(np.asarray(call(g, 1)), want(view, 1)), name
    assert np.array_equal(np.asarray(R.sum(g, axis=(0, 1))), ops[0][2](view, (0, 1)))


@pytest.mark.parametrize("even", [1, 0])
def test_column_pieces_counted_to_fill_the_compute_units_evenly(ctx, knobs, even):
    """The column kernel cuts the reduced range into the number of pieces that
    leaves every compute unit with the same number of groups where one exists
    near its target (REDUX_COL_BALANCE), and gives float sums a third group
    per unit where the inner kept dim leaves lanes idle (REDUX_COL_IDLE).
    Tiles of outputs that do not divide the unit count (3, 5, 12, 192 of them),
    kept rows of 160 and 72 elements, leading and middle axes; sums, integer
    and float extrema with positions, against NumPy, exact, whichever count
    of pieces the plan takes."""
    knobs(REDUX_COL_BALANCE=even, REDUX_COL_IDLE=even, REDUX_FOLD=0, REDUX_PCOLS=0)
    rng = np.random.default_rng(4300 + even)
    for shape, ax in (((6000, 768), 0), ((5000, 640), 0), ((9000, 160), 0), ((2500, 3000), 0), ((1100, 1280), 0),
                      ((64, 600, 320), 1), ((64, 700, 160), 1), ((32, 1500, 72), 1), ((3, 4000, 257), 1)):
        host = rng.integers(-20, 21, size=shape).astype(np.float32)
        g = gpuarray.array(host, context=ctx)
        assert np.array_equal(np.asarray(R.sum(g, axis=ax)), host.sum(axis=ax, dtype=np.float64).astype(np.float32)), shape
        v, i = R.maxandargmax(g, axis=ax)
        assert np.array_equal(np.asarray(v), host.max(axis=ax)) and np.array_equal(np.asarray(i), host.argmax(axis=ax)), shape
        gi = gpuarray.array(host.astype(np.int32), context=ctx)
        assert np.array_equal(np.asarray(R.sum(gi, axis=ax, dtype="int64")), host.astype(np.int64).sum(axis=ax)), shape
        assert np.array_equal(np.asarray(R.min(gi, axis=ax)), host.astype(np.int32).min(axis=ax)), shape


@pytest.mark.parametrize("order", [0, 1, 2])
def test_column_kernel_groups_numbered_to_keep_neighbours_on_one_die(ctx, knobs, order):
    """The column kernel may number its groups so that the neighbours along the
    inner kept dim run one after another on the same die (REDUX_XCD: 0 never,
    1 when kept rows start off the 128-byte lines, 2 always).  The numbering
    must reach every tile of outputs and every piece of the reduced range
    exactly once: leading, middle and several axes, group counts that are and
    are not multiples of 8 (also fewer than 8), one and several pieces per
    output with the finish inside the launch, sums, extrema with positions and
    any / all, against NumPy, exact."""
    knobs(REDUX_XCD=order, REDUX_FOLD=0, REDUX_PCOLS=0)
    rng = np.random.default_rng(4100 + order)
    for shape, ax in (((700, 1000), 0), ((64, 130, 250), 1), ((3, 20000, 37), 1), ((9, 40, 1001), (0, 1)),
                      ((40000, 9), 0), ((5, 7, 300, 129), (0, 2)), ((2, 100000, 4), 1), ((333, 8191), 0),
                      ((17, 1200, 513), 1), ((4100, 2050), 0)):
        host = rng.integers(-20, 21, size=shape).astype(np.float32)
        g = gpuarray.array(host, context=ctx)
        assert np.array_equal(np.asarray(R.sum(g, axis=ax)), host.sum(axis=ax, dtype=np.float64).astype(np.float32)), shape
        assert np.array_equal(np.asarray(R.min(g, axis=ax)), host.min(axis=ax)), shape
        gi = gpuarray.array(host.astype(np.int32), context=ctx)
        assert np.array_equal(np.asarray(R.sum(gi, axis=ax, dtype="int64")), host.astype(np.int64).sum(axis=ax)), shape
        if isinstance(ax, int):
            v, i = R.maxandargmax(g, axis=ax)
            assert np.array_equal(np.asarray(v), host.max(axis=ax)) and np.array_equal(np.asarray(i), host.argmax(axis=ax)), shape
        gb = gpuarray.array((host > -20).astype(np.bool_), context=ctx)
        assert np.array_equal(np.asarray(R.all(gb, axis=ax)), (host > -20).all(axis=ax)), shape
    # kept rows that start off the 128-byte lines inside a wider buffer
    root = rng.integers(-20, 21, size=(1200, 777)).astype(np.float32)
    view = root[:, 5:774]
    g, _ = to_gpu_view(view, ctx)
    assert np.array_equal(np.asarray(R.sum(g, axis=0)), view.sum(axis=0, dtype=np.float64).astype(np.float32))
    assert np.array_equal(np.asarray(R.max(g, axis=0)), view.max(axis=0))


@pytest.mark.parametrize("rows,cols", [(300, 70001), (130, 150000), (520, 66000), (41, 300000), (10, 700001), (48, 140003), (3, 2000000)])
def test_rows_cut_to_even_out_the_compute_units(ctx, knobs, rows, cols):
    """A few hundred long rows, one group each, would leave some compute units
    with one group more than the others: such rows are cut into pieces, and
    rows that are in pieces anyway into the nearest number of pieces that
    fills the units evenly (REDUX_BALANCE).  Whole and cut rows must agree bit for bit on data whose
    sums are exact, and with NumPy; the cut is there when the plan allows it
    (more than one launch, or a finish inside the first)."""
    rng = np.random.default_rng(rows)
    host = rng.integers(-30, 31, size=(rows, cols)).astype(np.float32)
    host[rng.integers(0, rows, 40), rng.integers(1, cols, 40)] = np.nan
    g = gpuarray.array(host, context=ctx)
    clean = np.nan_to_num(host)
    gi = gpuarray.array(clean.astype(np.int32), context=ctx)
    gc = gpuarray.array(clean, context=ctx)
    got = {}
    for balance in (0, 1):
        knobs(REDUX_BALANCE=balance)
        v, i = R.maxandargmax(g, axis=1)
        got[balance] = (np.asarray(R.sum(gc, axis=1)), np.asarray(R.sum(gi, axis=1, dtype="int64")),
                        np.asarray(v), np.asarray(i), np.asarray(R.min(gc, axis=1)))
    for a, b in zip(got[0], got[1]):
        assert np.array_equal(a, b)
    assert np.array_equal(got[1][0], clean.sum(axis=1, dtype=np.float64).astype(np.float32))
    assert np.array_equal(got[1][1], clean.astype(np.int64).sum(axis=1))
    assert np.array_equal(got[1][2], np.nanmax(host, axis=1)) and np.array_equal(got[1][3], np.nanargmax(host, axis=1))
    assert np.array_equal(got[1][4], clean.min(axis=1))


@pytest.mark.parametrize("seed", range(6))
def test_single_launch_finish_equals_two_launches_bit_for_bit(ctx, knobs, seed):
    """Every family of split reduction that can end in its own launch (row and
    column kernels, 4- and 8-byte accumulators, integer, float, with and
    without an index) against the same call finished by a second launch
    (REDUX_FUSED=0), bit for bit, over sixty drawn shapes per seed; the first
    mismatch stops the test.  The single launch orders its partials with
    device-scope atomics and a counter; the two launches with nothing but
    stream order.  Float data are small integers, so that every sum is exact
    and the two forms, which group the partials differently, must agree in
    every bit (specification of the result: reference pygpu/reduction.py:85-132);
    values change from call to call, so a partial left over from an earlier
    call, or one read before it arrived, shows."""
    rng = np.random.default_rng(9100 + seed)
    ops = [("sum", "float32", "float32"), ("sum", "float64", "float64"), ("sum", "int32", "int64"),
           ("sum", "int32", "int32"), ("sum", "int16", "int64"), ("max", "float32", None),
           ("min", "float64", None), ("max", "int32", None), ("maxandargmax", "float32", None),
           ("minandargmin", "float64", None), ("maxandargmax", "int32", None), ("argmax", "float32", None),
           ("prod", "int32", "int64"), ("any", "uint8", None), ("all", "int32", None), ("xor", "uint32", None)]

    def draw_shape():
        kind = int(rng.integers(0, 6))
        if kind == 0:      # one long row
            return (int(rng.integers(1 << 15, 1 << 22)),), (0,)
        if kind == 1:      # a few long rows
            return (int(rng.integers(2, 40)), int(rng.integers(1 << 14, 1 << 18))), (1,)
        if kind == 2:      # long columns, few to many outputs
            return (int(rng.integers(1 << 11, 1 << 15)), int(rng.choice([8, 64, 100, 256, 1000, 4096]))), (0,)
        if kind == 3:      # reduced dims around a kept one
            return (int(rng.integers(8, 200)), int(rng.integers(2, 30)), int(rng.integers(256, 8192))), (0, 2)
        if kind == 4:      # a middle axis over long columns
            return (int(rng.integers(2, 8)), int(rng.integers(1 << 10, 1 << 13)), int(rng.choice([32, 128, 512]))), (1,)
        return (int(rng.integers(1 << 16, 1 << 20)), int(rng.choice([1, 2, 3, 8]))), (0,)

    def run_all(cases):
        out, launches = [], []
        for g, name, odt, axes in cases:
            ctx.kernel_timing(True)
            if name in ("maxandargmax", "minandargmin"):
                r = R._arg_reduce(g, name, list(axes), True)
            elif name == "argmax":
                r = (R._arg_reduce(g, name, list(axes), False),)
            else:
                r = (R._reduce_named(g, name, np.dtype(odt) if odt else
                                     (np.dtype("bool") if name in ("any", "all") else g.dtype), axis=axes),)
            launches.append(len(ctx.kernel_times()))
            ctx.kernel_timing(False)
            out.append([np.asarray(x) for x in r])
        return out, launches

    single_launch_taken = 0
    for batch in range(4):
        cases, hosts = [], []
        for _ in range(15):
            name, dt, odt = ops[int(rng.integers(0, len(ops)))]
            shape, axes = draw_shape()
            if name == "prod":
                host = rng.choice(np.array([1, 1, 1, -1], dt), size=shape)     # +-2^k: exact in int64
                host.reshape(-1)[rng.integers(0, host.size, 20)] = 2
            elif name in ("any", "all"):
                host = (rng.random(shape) < (0.0005 if name == "any" else 0.9995)).astype(dt)
            elif np.dtype(dt).kind == "u":
                host = rng.integers(0, 1 << 16, size=shape).astype(dt)
            else:
                host = rng.integers(-40, 41, size=shape).astype(dt)
            g, _ = to_gpu_view(host, ctx)
            cases.append((g, name, odt, axes))
            hosts.append(host)
        one, n_one = run_all(cases)
        knobs(REDUX_FUSED=0)
        two, n_two = run_all(cases)
        knobs(REDUX_FUSED=None)
        for k, (a, b) in enumerate(zip(one, two)):
            what = (seed, batch, k, cases[k][1], hosts[k].dtype.name, hosts[k].shape, cases[k][3],
                    n_one[k], n_two[k])
            assert len(a) == len(b)
            for x, y in zip(a, b):
                assert x.dtype == y.dtype and x.shape == y.shape, what
                assert x.tobytes() == y.tobytes(), what
            single_launch_taken += n_one[k] < n_two[k]
        # and against NumPy for the plain sums (exact data)
        for k, (g, name, odt, axes) in enumerate(cases):
            if name == "sum":
                assert np.array_equal(one[k][0], hosts[k].sum(axis=axes, dtype=odt)), (seed, batch, k)
    # the draw must really exercise the single launch
    assert single_launch_taken >= 15, single_launch_taken


@pytest.mark.parametrize("dtype", ["uint8", "int8", "bool"])
def test_any_all_over_columns_of_bytes(ctx, dtype):
    """any / all with lanes along the free dim over one-byte elements: the
    words of a lane's load are combined whole and taken apart at the end.
    Values 0x01, 0x7f, 0x80, 0xff and 0 next to one another in a word (a test
    of one byte must not leak into its neighbours), 4, 8 and 16 columns per
    lane, split and unsplit ranges, a single element that flips a column."""
    rng = np.random.default_rng(57)
    vals = np.array([0, 1, 0x7f, 0x80, 0xff, 0, 0, 2], np.uint8)
    for shape in ((300, 1024), (4096, 256), (37, 64), (5000, 4096), (9, 130, 128), (1000, 20)):
        raw = vals[rng.integers(0, len(vals), size=shape)]
        host = (raw != 0) if dtype == "bool" else raw.view(dtype) if dtype == "int8" else raw
        cols = host.reshape(-1, shape[-1])
        cols[:, 0] = 0                       # any: false
        cols[:, 1] = 1 if dtype != "int8" else -128   # all: true
        cols[:, 2] = 0; cols[cols.shape[0] // 2, 2] = 1     # one element makes any true
        cols[:, 3] = 1; cols[cols.shape[0] - 1, 3] = 0      # one element makes all false
        cols[:, 5] = 0                                       # a zero column between non-zero ones
        cols[:, 4] = 1; cols[:, 6] = 1
        axes = tuple(range(host.ndim - 1))
        for view in (host, host[..., 4:], host[1::2]):
            g, _ = to_gpu_view(view, ctx)
            assert np.array_equal(np.asarray(R.any(g, axis=axes)), view.any(axis=axes)), (shape, view.shape)
            assert np.array_equal(np.asarray(R.all(g, axis=axes)), view.all(axis=axes)), (shape, view.shape)
            if view.ndim == 3:
                assert np.array_equal(np.asarray(R.any(g, axis=(1,))), view.any(axis=1))
                assert np.array_equal(np.asarray(R.all(g, axis=(0,))), view.all(axis=0))


@pytest.mark.parametrize("dtype", ["float64", "int64", "float32", "int16", "uint8"])
def test_stepped_inner_dim_of_every_width(ctx, dtype):
    """Reduced rows that take every 2nd, 3rd or 4th element (8-byte elements
    four apart leave no load that holds two of them)."""
    rng = np.random.default_rng(93)
    for shape in ((16, 4), (300, 4000), (5, 70001), (2000, 64)):
        base = rng.integers(0, 50, size=shape).astype(dtype)
        for step in (2, 3, 4):
            for view in (base[:, ::step], base[:, 1::step], base[:, :1], base[::step, ::step]):
                _check_ops(ctx, view, [1])
                _check_ops(ctx, view, [0, 1])


def test_stepped_eight_byte_rows_are_planned(ctx):
    """The planner's arithmetic alone (no look at the values): an 8-byte
    element type whose reduced dim steps by four elements."""
    base = np.zeros((16, 4), np.float64)
    g, _ = to_gpu_view(base[:, :1], ctx)
    for axes in ((0, 1), (0,), (1,)):
        assert np.asarray(R.sum(g, axis=axes)).shape == base[:, :1].sum(axis=axes).shape
        v, i = R.maxandargmax(g, axis=axes)
        assert np.asarray(i).dtype == np.int64
    g, _ = to_gpu_view(np.zeros((64, 4096), np.int64)[:, ::4], ctx)
    assert np.asarray(R.sum(g, axis=1)).shape == (64,)


@pytest.mark.parametrize("fold", [1, 2, 0])
def test_a_run_of_middle_axes_over_short_kept_rows_is_folded_per_slab(ctx, knobs, fold):
    """The same folding under leading dims that are kept: (O, R, F) over the
    middle run of axes is O slabs, each folded like a dense array (REDUX_FOLD:
    1 slabs too, 2 leading axes only, 0 never).  One and two kept dims in
    front, one and two reduced axes (in either order), kept rows of 1 to 250
    elements, row counts with and without a divisor, a strided destination;
    integer results exact, against NumPy."""
    knobs(REDUX_FOLD=fold, REDUX_FOLD_SLAB_MIN_BYTES=1)
    rng = np.random.default_rng(72)
    cases = (((64, 1000, 250), (1,), "float32"), ((8, 65536, 33), (1,), "int32"), ((16, 64, 64, 62), (1, 2), "int32"),
             ((16, 64, 64, 62), (2, 1), "float32"), ((3, 5, 4096, 30), (2,), "uint8"), ((40, 4099, 10), (1,), "int32"),
             ((128, 16384, 1), (1,), "float32"), ((6, 262144, 3), (1,), "float16"))
    for shape, axes, dt in cases:
        host = rng.integers(-3 if np.dtype(dt).kind in "if" else 0, 4, size=shape).astype(dt)
        g = gpuarray.array(host, context=ctx)
        odt = "int64" if np.dtype(dt).kind in "iu" else "float32"
        got = np.asarray(R.sum(g, axis=axes, dtype=odt))
        assert np.array_equal(got, host.sum(axis=axes, dtype=np.int64).astype(odt)), (shape, axes, dt)
        got = np.asarray(R._reduce_named(g, "any", np.dtype("bool"), axis=axes))
        assert np.array_equal(got, host.any(axis=axes)), (shape, axes, dt)
        if np.dtype(dt).kind in "iu":
            assert np.array_equal(np.asarray(R.max(g, axis=axes)), host.max(axis=axes)), (shape, axes, dt)
        else:
            val, idx = R.maxandargmax(g, axis=axes[:1])      # keeps the order of the scan: not folded
            assert np.array_equal(np.asarray(val), host.max(axis=axes[0]))
            assert np.array_equal(np.asarray(idx), host.argmax(axis=axes[0]))
    host = rng.integers(-3, 4, size=(64, 1000, 250)).astype(np.float32)
    g = gpuarray.array(host, context=ctx)
    wide = gpuarray.zeros((64, 250, 3), "float32", context=ctx)
    ga.GpuReduction(ctx, "sum", "float32")(g, [1], d0=wide[:, :, 1])
    assert np.array_equal(np.asarray(wide)[:, :, 1], host.sum(axis=1))
    assert not np.asarray(wide)[:, :, [0, 2]].any()


@pytest.mark.parametrize("slabs", [1, 0])
def test_a_middle_run_of_axes_under_many_small_slabs(ctx, knobs, slabs):
    """(O, R, F) reduced over its middle run with many slabs of a few KiB to a
    few hundred and short kept rows: one group walks a whole slab as one run
    of 16-byte chunks and writes the slab's F outputs itself (REDUX_PSLABS; 0:
    the column kernel).  Kept rows of 3 to 100 elements, 4- and 8-byte and
    half elements, slabs whose chunk count is and is not a multiple of the
    active lanes, two reduced dims, a strided destination; every operation
    that may be regrouped, against NumPy."""
    knobs(REDUX_PSLABS=slabs, REDUX_FOLD_MIN_BYTES=1)
    rng = np.random.default_rng(5300 + slabs)
    cases = (((600, 512, 12), (1,)), ((1000, 256, 30), (1,)), ((520, 100, 33), (1,)), ((512, 7, 64, 20), (1, 2)),
             ((700, 64, 100), (1,)), ((2048, 344, 3), (1,)), ((513, 1024, 5), (1,)), ((16, 40, 300, 4, 6), (2,)))
    every = ("float32", "int32", "float16", "float64")
    for ci, (shape, axes) in enumerate(cases):
        for dt in (every if ci < 2 else every[ci % 2::2]):
            host = rng.integers(-3, 4, size=shape).astype(dt)
            g = gpuarray.array(host, context=ctx)
            kept = tuple(d for i, d in enumerate(shape) if i not in axes)
            odt = "int64" if dt == "int32" else ("float32" if dt == "float16" else dt)
            got = np.asarray(R.sum(g, axis=axes, dtype=odt))
            assert got.shape == kept
            assert np.array_equal(got, host.sum(axis=axes, dtype=np.int64).astype(got.dtype)), (shape, dt, "sum")
            for name, npf in (("all", np.all), ("any", np.any)):
                got = np.asarray(R._reduce_named(g, name, np.dtype("bool"), axis=axes))
                assert np.array_equal(got, npf(host, axis=axes)), (shape, dt, name)
            if dt == "int32":
                for name, npf in (("max", np.max), ("min", np.min)):
                    assert np.array_equal(np.asarray(getattr(R, name)(g, axis=axes)), npf(host, axis=axes)), (shape, dt, name)
                got = np.asarray(R._reduce_named(g, "xor", np.dtype(dt), axis=axes))
                assert np.array_equal(got, np.bitwise_xor.reduce(host, axis=axes)), (shape, dt, "xor")
            else:
                v, i = R.maxandargmax(g, axis=axes[:1]) if len(axes) == 1 else (None, None)
                if v is not None:   # keeps the order of the scan: the planned path, still right
                    assert np.array_equal(np.asarray(v), host.max(axis=axes[0]))
                    assert np.array_equal(np.asarray(i), host.argmax(axis=axes[0]))
    # float sums to tolerance, a strided destination
    host = rng.standard_normal((800, 300, 20)).astype(np.float32) + np.float32(0.5)
    g = gpuarray.array(host, context=ctx)
    wide = gpuarray.zeros((800, 20, 3), "float32", context=ctx)
    ga.GpuReduction(ctx, "sum", "float32")(g, [1], d0=wide[:, :, 1])
    x64 = host.astype(np.float64)
    assert_sum_close(np.asarray(wide)[:, :, 1], x64.sum(axis=1), np.abs(x64).sum(axis=1))
    assert not np.asarray(wide)[:, :, [0, 2]].any()


@pytest.mark.parametrize("two_calls", [1, 0])
def test_leading_and_short_trailing_axes_around_kept_ones(ctx, knobs, two_calls):
    """Per-channel reductions over (batch, channel, a small height x width):
    leading and trailing dims reduced around kept ones.  With a trailing run of
    at most REDUX_OUTER_FIRST bytes the leading dims are reduced first, at full
    load width, and the short trailing run of the partial results second (0:
    one call).  Every operation that may be regrouped, integer and floating
    types, three to five dims, a strided destination, results against NumPy;
    arg-reductions and floating extrema keep the single call and stay right."""
    knobs(REDUX_OUTER_FIRST=4096 if two_calls else 0, REDUX_FOLD_MIN_BYTES=1)
    rng = np.random.default_rng(5100 + two_calls)
    cases = (((64, 400, 49), (0, 2)), ((16, 3000, 33), (0, 2)), ((8, 4, 500, 7, 7), (0, 1, 3, 4)), ((128, 100, 4, 4), (0, 2, 3)),
             ((6, 5, 70, 3, 16), (0, 1, 4)), ((2, 100000, 12), (0, 2)), ((32, 64, 256), (0, 2)), ((32, 64, 257), (0, 2)))
    every = ("float32", "int32", "int8", "float16", "uint8", "float64")
    for ci, (shape, axes) in enumerate(cases):
        for dt in (every[:2] if ci else every):
            host = rng.integers(-3 if np.dtype(dt).kind in "if" else 0, 4, size=shape).astype(dt)
            g = gpuarray.array(host, context=ctx)
            kept = tuple(d for i, d in enumerate(shape) if i not in axes)
            got = np.asarray(R.sum(g, axis=axes, dtype="int64" if np.dtype(dt).kind in "iu" else
                                   ("float64" if dt == "float64" else "float32")))
            assert got.shape == kept
            assert np.array_equal(got, host.sum(axis=axes, dtype=np.int64).astype(got.dtype)), (shape, dt, "sum")
            for name, npf in (("all", np.all), ("any", np.any)):
                got = np.asarray(R._reduce_named(g, name, np.dtype("bool"), axis=axes))
                assert np.array_equal(got, npf(host, axis=axes)), (shape, dt, name)
            if np.dtype(dt).kind in "iu":
                for name, npf in (("max", np.max), ("min", np.min)):
                    assert np.array_equal(np.asarray(getattr(R, name)(g, axis=axes)), npf(host, axis=axes)), (shape, dt, name)
                got = np.asarray(R._reduce_named(g, "xor", np.dtype(dt), axis=axes))
                assert np.array_equal(got, np.bitwise_xor.reduce(host, axis=axes)), (shape, dt, "xor")
            else:
                # floating extrema follow the order of the scan: one call, still right
                assert np.array_equal(np.asarray(R.max(g, axis=axes)), host.max(axis=axes)), (shape, dt, "max")
    # products of +-1, float sums to tolerance, a strided destination
    host = rng.choice(np.array([1.0, -1.0], dtype=np.float32), size=(64, 300, 20))
    g = gpuarray.array(host, context=ctx)
    got = np.asarray(R._reduce_named(g, "prod", np.dtype("float32"), axis=(0, 2)))
    assert np.array_equal(got, np.prod(host.astype(np.float64), axis=(0, 2)).astype(np.float32))
    host = rng.standard_normal((64, 500, 49)).astype(np.float32) + np.float32(0.5)
    g = gpuarray.array(host, context=ctx)
    wide = gpuarray.zeros((500, 3), "float32", context=ctx)
    ga.GpuReduction(ctx, "sum", "float32")(g, [0, 2], d0=wide[:, 1])
    x64 = host.astype(np.float64)
    assert_sum_close(np.asarray(wide)[:, 1], x64.sum(axis=(0, 2)), np.abs(x64).sum(axis=(0, 2)))
    assert not np.asarray(wide)[:, [0, 2]].any()
    # reduxList in any order
    out = gpuarray.empty((500,), "float32", context=ctx)
    ga.GpuReduction(ctx, "sum", "float32")(g, [2, 0], d0=out)
    assert_sum_close(np.asarray(out), x64.sum(axis=(0, 2)), np.abs(x64).sum(axis=(0, 2)))


@pytest.mark.parametrize("route", ["one launch", "folded", "neither"])
def test_leading_dims_with_short_kept_rows_are_folded(ctx, knobs, route):
    """Reducing the leading dims of a dense array whose kept rows are short or
    off a 16-byte boundary: in one launch that walks the array as one run of
    chunks (redux_pcols) where the row length allows it, else through folded
    rows (every m rows taken as one, then the m copies of each output
    combined): every operation that may be regrouped, integer and floating
    types, one and two leading dims, row counts with and without a usable
    divisor, a strided destination; against NumPy, by each of the two routes
    and with both switched off."""
    fold = "0" if route == "neither" else "1"
    knobs(REDUX_FOLD=fold, REDUX_PCOLS=1 if route == "one launch" else 0)
    rng = np.random.default_rng(71)
    cases = (((1 << 20, 10), (0,)), ((1 << 21, 3), (0,)), ((16384, 1001), (0,)),
             ((1024, 1024, 4), (0, 1)), ((1048573, 5), (0,)), ((3 * (1 << 18), 6, 2), (0,)),
             ((1 << 22, 1), (0,)))
    every = ("float32", "int32", "int8", "float16", "uint8")
    for ci, (shape, axes) in enumerate(cases if fold == "1" else cases[:1]):
        # three types on the first shape, one per shape after that
        for dt in (every[:4:2] + every[3:4] if ci == 0 and fold == "1" else (every[ci % 5],)):
            if np.prod(shape) * np.dtype(dt).itemsize < (4 << 20):
                continue
            host = rng.integers(-3 if np.dtype(dt).kind in "if" else 0, 4, size=shape).astype(dt)
            g = gpuarray.array(host, context=ctx)
            kept = tuple(d for i, d in enumerate(shape) if i not in axes)
            got = np.asarray(R.sum(g, axis=axes, dtype="int64" if np.dtype(dt).kind in "iu" else "float32"))
            assert got.shape == kept
            assert np.array_equal(got, host.sum(axis=axes, dtype=np.int64).astype(got.dtype)), (shape, dt, "sum")
            for name, npf in (("all", np.all), ("any", np.any)):
                got = np.asarray(R._reduce_named(g, name, np.dtype("bool"), axis=axes))
                assert np.array_equal(got, npf(host, axis=axes)), (shape, dt, name)
            if np.dtype(dt).kind in "iu":
                for name, npf in (("max", np.max), ("min", np.min)):
                    assert np.array_equal(np.asarray(getattr(R, name)(g, axis=axes)), npf(host, axis=axes)), (shape, dt, name)
                for name, npf in (("and", np.bitwise_and), ("or", np.bitwise_or), ("xor", np.bitwise_xor)):
                    got = np.asarray(R._reduce_named(g, name, np.dtype(dt), axis=axes))
                    assert np.array_equal(got, npf.reduce(host, axis=axes)), (shape, dt, name)
            else:
                # arg-reductions and floating min / max keep the order of the scan: not folded, still right
                val, idx = R.maxandargmax(g, axis=axes)
                moved = host.reshape(-1, int(np.prod(kept)))
                assert np.array_equal(np.asarray(val).ravel(), moved.max(axis=0))
                assert np.array_equal(np.asarray(idx).ravel(), moved.argmax(axis=0))
    # kept rows of whole 16-byte pieces between 256 and 512 bytes (one launch too: the
    # column kernel's second tile of 256 bytes would be mostly idle), and 256 bytes exactly
    for shape, dt in (((1 << 16, 72), "float32"), ((1 << 15, 36), "float64"), ((1 << 16, 68), "int32"),
                      ((40000, 124), "float32"), ((1 << 16, 64), "float32")):
        host = rng.integers(-3, 4, size=shape).astype(dt)
        g = gpuarray.array(host, context=ctx)
        got = np.asarray(R.sum(g, axis=0, dtype="int64" if dt == "int32" else dt))
        assert np.array_equal(got, host.sum(axis=0, dtype=np.int64 if dt == "int32" else np.float64).astype(got.dtype)), (shape, dt)
        if dt == "int32":
            assert np.array_equal(np.asarray(R.max(g, axis=0)), host.max(axis=0)), (shape, dt)
    # products (of +-1, so that nothing overflows), float sums to tolerance, a strided destination
    host = rng.choice(np.array([1.0, -1.0], dtype=np.float32), size=(1 << 20, 6))
    g = gpuarray.array(host, context=ctx)
    got = np.asarray(R._reduce_named(g, "prod", np.dtype("float32"), axis=(0,)))
    assert np.array_equal(got, np.prod(host.astype(np.float64), axis=0).astype(np.float32))
    host = rng.standard_normal((1 << 20, 10)).astype(np.float32) + np.float32(0.5)
    g = gpuarray.array(host, context=ctx)
    wide = gpuarray.zeros((10, 3), "float32", context=ctx)
    o = ga.GpuReduction(ctx, "sum", "float32")
    o(g, [0], d0=wide[:, 1])
    x64 = host.astype(np.float64)
    assert_sum_close(np.asarray(wide)[:, 1], x64.sum(axis=0), np.abs(x64).sum(axis=0))
    assert not np.asarray(wide)[:, [0, 2]].any()
