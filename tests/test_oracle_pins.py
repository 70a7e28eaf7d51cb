"""Pins the CPU checker (oracle/) before anything is compared against it:
  - the literal scenarios of the reference's elementwise tests
    (tests/check_elemwise.c:39-880) and argument-check tests
    (pygpu/tests/test_tools.py:6-118),
  - maxandargmax against an independent NumPy formulation on the reference's
    own PCG32 data (tests/check_reduction.c) and against closed forms,
  - the Python reduction template against NumPy, float64 sums and closed forms.
Runs without a GPU."""
import json
import os

import numpy as np
import pytest

KATS = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kats.json")))
BCAST, NOCOLLAPSE, PAD = 0x100, 0x200, 0x400
F16 = np.array(KATS["f16_table_0_to_9"]["half_bits"], dtype=np.uint16).view(np.float16)


def farr(vals, shape, order="C", dtype=np.uint32):
    """An array whose MEMORY holds vals in order, with the given shape/order
    (the reference tests write a flat buffer into C- or F-ordered arrays)."""
    return np.array(vals, dtype=dtype).reshape(shape, order=order)


# ---- tests/check_elemwise.c literal scenarios --------------------------------

def test_f16_table_is_the_integers():
    assert np.array_equal(F16.astype(np.float32), np.arange(10, dtype=np.float32))


def test_contig_simple(oracle):           # check_elemwise.c:39-93
    a, b, c = farr([1, 2, 3], 3), farr([4, 5, 6], 3), np.zeros(3, np.uint32)
    assert oracle.elemwise(oracle.ADD_U32, [a, b, c], [0, 0, 1], NOCOLLAPSE) == 0
    assert c.tolist() == [5, 7, 9]


def test_contig_f16(oracle):              # check_elemwise.c:95-154
    a, b = F16[[1, 2, 3]].copy(), F16[[4, 5, 6]].copy()
    c = np.zeros(3, np.float16)
    assert oracle.elemwise(oracle.ADD_F16, [a, b, c], [0, 0, 1], NOCOLLAPSE) == 0
    assert np.array_equal(c.view(np.uint16), F16[[5, 7, 9]].view(np.uint16))


def test_zero_sized(oracle):              # check_elemwise.c:156-198, 837-880
    a, b, c = (np.zeros(0, np.uint32) for _ in range(3))
    assert oracle.elemwise(oracle.ADD_U32, [a, b, c], [0, 0, 1], NOCOLLAPSE) == 0
    a = np.zeros((0, 3), np.uint32)
    b = np.zeros((0, 3), np.uint32, order="F")
    c = np.zeros((0, 3), np.uint32)
    assert oracle.elemwise(oracle.ADD_U32, [a, b, c], [0, 0, 1], 0) == 0


def test_basic_simple_mixed_orders(oracle):   # check_elemwise.c:200-256
    a = farr([1, 2, 3], (1, 3))
    b = farr([4, 5, 6], (1, 3), "F")
    c = np.zeros((1, 3), np.uint32)
    assert oracle.elemwise(oracle.ADD_U32, [a, b, c], [0, 0, 1], NOCOLLAPSE) == 0
    assert c.ravel().tolist() == [5, 7, 9]


def test_basic_offset(oracle):            # check_elemwise.c:320-383: a starts 12 bytes in
    buf = np.zeros(6, np.uint32)
    buf[3:] = [1, 2, 3]
    a = buf[3:].reshape(1, 3)
    b = farr([4, 5, 6], (1, 3), "F")
    c = np.zeros((1, 3), np.uint32)
    assert oracle.elemwise(oracle.ADD_U32, [a, b, c], [0, 0, 1], NOCOLLAPSE) == 0
    assert c.ravel().tolist() == [5, 7, 9]


def test_basic_scalar(oracle):            # check_elemwise.c:385-455: c = a + x*b, x = 2
    a = farr([1, 2, 3], (1, 3))
    b = farr([4, 5], (2, 1), "F")
    c = np.zeros((2, 3), np.uint32)
    assert oracle.elemwise(oracle.AXPB_U32, [a, b, c], [0, 0, 1], BCAST,
                           scalar=np.uint32(2)) == 0
    assert c.ravel().tolist() == [9, 10, 11, 11, 12, 13]


def test_basic_scalar_dtype(oracle):      # check_elemwise.c:457-509: y = a*x + y, a = 1.1f
    x = farr([0, 1, 2, 3], (2, 2), dtype=np.int32)
    y = farr([2.0, 2.0, 2.0, 2.0], (2, 2), "F", dtype=np.float32)
    assert oracle.elemwise(oracle.SAXPY_I32_F32, [x, y], [0, 1], 0, scalar=np.float32(1.1)) == 0
    got = y.ravel(order="K")              # memory order, as GpuArray_read returns it
    want = np.array([2.0, 4.2, 3.1, 5.3], dtype=np.float32)
    assert np.array_equal(got, want)


def test_basic_remove1(oracle):           # check_elemwise.c:511-571
    a = farr([1, 2, 3, 4, 5, 6], (1, 3, 2, 1))
    b = farr([7, 8, 9, 10, 11, 12], (1, 3, 2, 1), "F")
    c = np.zeros((1, 3, 2, 1), np.uint32)
    assert oracle.elemwise(oracle.ADD_U32, [a, b, c], [0, 0, 1], 0) == 0
    assert c.ravel().tolist() == [8, 12, 11, 15, 14, 18]


def test_basic_broadcast(oracle):         # check_elemwise.c:573-639
    a = farr([1, 2, 3], (1, 3))
    b = farr([4, 5], (2, 1), "F")
    c = np.zeros((2, 3), np.uint32)
    assert oracle.elemwise(oracle.ADD_U32, [a, b, c], [0, 0, 1], NOCOLLAPSE) == 2   # GA_VALUE_ERROR
    assert oracle.elemwise(oracle.ADD_U32, [a, b, c], [0, 0, 1], NOCOLLAPSE | BCAST) == 0
    assert c.ravel().tolist() == [5, 6, 7, 6, 7, 8]


def test_basic_padshape(oracle):          # check_elemwise.c:641-706
    a = farr([1, 2, 3], (3,))
    b = farr([4, 5], (2, 1), "F")
    c = np.zeros((2, 3), np.uint32)
    assert oracle.elemwise(oracle.ADD_U32, [a, b, c], [0, 0, 1], NOCOLLAPSE) == 2
    assert oracle.elemwise(oracle.ADD_U32, [a, b, c], [0, 0, 1], NOCOLLAPSE | BCAST | PAD) == 0
    assert c.ravel().tolist() == [5, 6, 7, 6, 7, 8]


def test_basic_collapse(oracle):          # check_elemwise.c:708-766
    a = farr([1, 2, 3, 4, 5, 6], (2, 3))
    b = farr([7, 8, 9, 10, 11, 12], (2, 3))
    c = np.zeros((2, 3), np.uint32)
    assert oracle.elemwise(oracle.ADD_U32, [a, b, c], [0, 0, 1], 0) == 0
    assert c.ravel().tolist() == [8, 10, 12, 14, 16, 18]


def test_basic_neg_strides(oracle):       # check_elemwise.c:768-835
    a = farr([1, 2, 3, 4, 5, 6], (6,))
    b = farr([7, 8, 9, 10, 11, 12], (6,))[::-1]
    c = np.zeros(6, np.uint32)
    assert oracle.elemwise(oracle.ADD_U32, [a, b, c], [0, 0, 1], 0) == 0
    assert c.tolist() == [13] * 6


# ---- pygpu/tests/test_tools.py check_args vectors -----------------------------

@pytest.mark.parametrize("case", KATS["check_args"]["cases"], ids=lambda c: c["name"])
def test_check_args_vectors(case, oracle):
    # the Python-level check (pygpu/tools.py:68-168), vector for vector
    n, nd, dims, strs = oracle.check_args(case["shapes"], case["strides"], case["collapse"],
                                          case["broadcast"])
    assert (n, nd, list(dims)) == (case["n"], case["nd"], case["dims"])
    assert [list(s) for s in strs] == case["strs"]


@pytest.mark.parametrize("case", KATS["check_args"]["cases"], ids=lambda c: c["name"])
def test_c_check_agrees_with_the_python_check(case, oracle):
    # same layouts through the C-level check (src/gpuarray_elemwise.c:272-383).
    # It needs an output (the full-shaped array) and zeroes the stride of every
    # size-1 dim (:357-359), which the Python check does not; elsewhere the
    # two must agree.
    from numpy.lib.stride_tricks import as_strided
    arrays = []
    for shp, st in zip(case["shapes"], case["strides"]):
        span = sum((d - 1) * abs(s) for d, s in zip(shp, st)) // 4 + 1
        arrays.append(as_strided(np.zeros(span, dtype=np.float32), shape=shp, strides=st))
    flags = (BCAST if case["broadcast"] else 0) | (0 if case["collapse"] else NOCOLLAPSE)
    out = case.get("out", len(arrays) - 1)
    err, nd, dims, strs, n, call32 = oracle.check_basic(
        arrays, [i == out for i in range(len(arrays))], flags)
    assert err == 0 and call32 == 1
    assert (n, nd, list(dims)) == (case["n"], case["nd"], case["dims"])
    for got, want in zip(strs, case["strs"]):
        assert [g for g, d in zip(got, dims) if d != 1] == [w for w, d in zip(want, dims) if d != 1]
        assert all(g == 0 for g, d in zip(got, dims) if d == 1)


@pytest.mark.parametrize("case", KATS["planned_iteration_spaces"]["cases"], ids=lambda c: c["name"][:12])
def test_planned_iteration_space_of_the_strided_configurations(case, oracle):
    """The iteration space the reference plans for configuration 2 (two
    dimensions that do not merge, 32-bit offsets) and for the stride-2 views of
    configuration 5 (one dimension of 67 108 864 elements, source stride twice
    the item size): the checker's check_basic and the library's exported
    gpuarray_elemwise_collapse both have to arrive there."""
    from numpy.lib.stride_tricks import as_strided
    from test_types_util import lib_collapse
    dt = {1: np.uint8, 2: np.float16, 4: np.float32}[case["itemsize"]]
    # views of a one-element buffer: only shapes and strides are looked at
    arrays = [as_strided(np.zeros(1, dtype=dt), shape=a["shape"], strides=a["strides"], writeable=False)
              for a in case["arrays"]]
    is_out = [i == case["out"] for i in range(len(arrays))]
    err, nd, dims, strs, n, call32 = oracle.check_basic(arrays, is_out, BCAST if case["broadcast"] else 0)
    assert err == 0
    assert (nd, list(dims), n, call32) == (case["nd"], case["dims"], case["n"], case["call32"])
    assert [list(s) for s in strs] == case["strs"]
    # the library's collapse on the broadcast-adjusted strides (a size-1 input dim has stride 0)
    full = case["arrays"][case["out"]]["shape"]
    rows = [[0 if a["shape"][i] == 1 and full[i] != 1 else a["strides"][i] for i in range(len(full))]
            for a in case["arrays"]]
    lnd, ldims, lstrs = lib_collapse(list(full), rows)
    assert (lnd, list(ldims)) == (case["nd"], case["dims"])
    assert [list(s) for s in lstrs] == case["strs"]


def test_checker_elemwise_equals_numpy_on_random_views(oracle):
    rng = np.random.default_rng(21)
    for _ in range(60):
        nd = int(rng.integers(1, 4))
        shape = tuple(int(x) for x in rng.integers(1, 7, nd))
        a = rng.normal(size=shape).astype(np.float32)
        if rng.random() < 0.5:
            a = np.asfortranarray(a)
        bshape = tuple(d if rng.random() < 0.6 else 1 for d in shape)
        cshape = tuple(d if rng.random() < 0.6 else 1 for d in shape)
        b = rng.normal(size=bshape).astype(np.float32)
        c = rng.normal(size=cshape).astype(np.float32)[tuple(slice(None, None, -1) for _ in shape)]
        out = np.zeros(shape, np.float32)
        assert oracle.elemwise(oracle.A_PLUS_BC_F32, [a, b, c, out], [0, 0, 0, 1], BCAST) == 0
        assert np.array_equal(out, a + b * c)


# ---- maxandargmax -------------------------------------------------------------

def np_maxandargmax(x, redux):
    """Independent formulation: move the free axes first and the reduced axes
    after them IN reduxList ORDER, flatten the latter, and let NumPy scan."""
    free = [i for i in range(x.ndim) if i not in redux]
    y = x.transpose(free + list(redux)).reshape([x.shape[i] for i in free] + [-1])
    return y.max(-1), y.argmax(-1)


@pytest.mark.parametrize("shape,redux", [
    ((32, 50, 79), [0, 2]),      # check_reduction.c:66-154  test_reduction
    ((32, 50, 79), [2, 0]),      # :156-244  test_idxtranspose
    ((32, 50, 79), [0, 1, 2]),   # :345-431  test_alldimsreduced
    ((37, 13, 2, 1, 2, 1, 2, 1), [2, 4, 7, 5]),   # :246-343 test_veryhighrank, smaller lead dims
])
def test_maxandargmax_on_reference_data(shape, redux, oracle):
    x = oracle.pcg_fill_f32(int(np.prod(shape)), seed=1).reshape(shape)
    m, a = oracle.maxandargmax(x, redux)
    wm, wa = np_maxandargmax(x, redux)
    assert np.array_equal(m, wm) and np.array_equal(a, wa)


def test_pcg_stream_is_the_published_generator(oracle):
    # PCG-XSH-RR 64/32 with the reference's constants, restated in Python ints
    s = 1
    M, A = 6364136223846793005, 1442695040888963407
    out = []
    for _ in range(8):
        vals = []
        for _k in range(2):
            s = (s * M + A) & (2 ** 64 - 1)
            x = ((s ^ (s >> 18)) >> 27) & 0xffffffff
            r = s >> 59
            vals.append(((x >> r) | (x << ((32 - r) & 31))) & 0xffffffff if r else x)
        out.append(np.float32(((vals[0] << 32) | vals[1]) / 18446744073709551616.0))
    assert np.array_equal(oracle.pcg_fill_f32(8, 1), np.array(out, dtype=np.float32))


def test_maxandargmax_closed_forms(oracle):
    const = np.full((5, 40), 3.0, np.float32)
    m, a = oracle.maxandargmax(const, [1])
    assert np.all(m == 3.0) and np.all(a == 0)              # ties -> first index
    inc = np.tile(np.arange(40, dtype=np.float32), (5, 1))
    m, a = oracle.maxandargmax(inc, [1])
    assert np.all(a == 39)
    planted = np.zeros((4, 100), np.float32)
    planted[:, [70, 20, 90]] = 9.0
    assert np.all(oracle.maxandargmax(planted, [1])[1] == 20)
    # NaN is ignored unless it is the first element scanned (strict '>')
    x = np.array([[1.0, np.nan, 5.0, 2.0], [np.nan, 7.0, 1.0, 0.0]], np.float32)
    m, a = oracle.maxandargmax(x, [1])
    assert m[0] == 5.0 and a[0] == 2 and np.isnan(m[1]) and a[1] == 0
    # -0.0 vs +0.0: equal, so the first one scanned stays
    z = np.array([[-0.0, 0.0], [0.0, -0.0]], np.float32)
    m, a = oracle.maxandargmax(z, [1])
    assert np.signbit(m[0]) and not np.signbit(m[1]) and a.tolist() == [0, 0]


def test_maxandargmax_strided_and_other_types(oracle):
    rng = np.random.default_rng(8)
    base = rng.integers(-50, 50, (6, 9, 14)).astype(np.int32)
    for view in (base[:, :, ::2], base.transpose(2, 0, 1), base[::-1, :, 1:]):
        for redux in ([1], [2, 0], [0, 1, 2]):
            m, a = oracle.maxandargmax(view, redux)
            wm, wa = np_maxandargmax(view, redux)
            assert np.array_equal(m, wm) and np.array_equal(a, wa)
    h = rng.normal(size=(7, 33)).astype(np.float16)
    m, a = oracle.maxandargmax(h, [1])
    assert np.array_equal(m, h.max(1)) and np.array_equal(a, h.argmax(1))


# ---- the Python reduction template ----------------------------------------------

@pytest.mark.parametrize("shape,redux", [
    ((10,), [True]), ((20, 30), [True, True]), ((20, 30), [True, False]), ((20, 30), [False, True]),
    ((8, 5, 10), [True, True, True]), ((8, 5, 10), [True, True, False]),
    ((8, 5, 10), [True, False, True]), ((8, 5, 10), [False, True, True]),
    ((8, 5, 10), [True, False, False]), ((8, 5, 10), [False, True, False]),
    ((8, 5, 10), [False, False, True]),
])                                                  # pygpu/tests/test_reduction.py:12-27
def test_reduk_sum_masks(shape, redux, oracle):
    rng = np.random.default_rng(1)
    axes = [i for i, r in enumerate(redux) if r]
    for dt in ("float32", "float64", "int32"):
        x = (rng.uniform(0, 10, shape)).astype(dt)
        for ls in (1, 32, 256):
            got = oracle.reduk("sum", x, axes, dt, ls=ls)
            want = x.sum(axis=tuple(axes))
            assert got.shape == want.shape
            if dt == "int32":
                assert np.array_equal(got, want.astype(dt))
            else:
                assert np.allclose(got, want, rtol=2e-5)   # the reference's own tolerance


def test_reduk_closed_forms(oracle):
    ones = np.ones((7, 1000), np.float32)
    assert np.all(oracle.reduk("sum", ones, [1], "float32") == 1000.0)
    ar = np.arange(4096, dtype=np.int32)
    assert oracle.reduk("sum", ar, [0], "int64") == 4096 * 4095 // 2
    pm = np.concatenate([np.arange(1, 501), -np.arange(1, 501)]).astype(np.float32)
    assert oracle.reduk("sum", pm, [0], "float32") == 0.0
    assert oracle.reduk("prod", np.array([1, 2, 3, 4, 5], np.int32), [0], "int64") == 120
    b = np.zeros((3, 50), np.uint8)
    b[1, 49] = 1
    b[2, :] = 1
    assert oracle.reduk("any", b, [1], "bool").tolist() == [False, True, True]
    assert oracle.reduk("all", b, [1], "bool").tolist() == [False, False, True]
    # accumulate in the OUTPUT type (pygpu/reduction.py:83): int32 values that
    # overflow 32 bits are fine in an int64 result
    big = np.full(10, 2 ** 30, np.int32)
    assert oracle.reduk("sum", big, [0], "int64") == 10 * 2 ** 30
    assert oracle.reduk("sum", big, [0], "int32") == np.int32((10 * 2 ** 30) % 2 ** 32 - 2 ** 32
                                                              if (10 * 2 ** 30) % 2 ** 32 >= 2 ** 31
                                                              else (10 * 2 ** 30) % 2 ** 32)


def test_reduk_order_is_the_templates(oracle):
    # with one lane the template is a plain left-to-right float32 sum
    rng = np.random.default_rng(3)
    x = rng.normal(0, 1, 5000).astype(np.float32)
    seq = np.float32(0)
    for v in x:
        seq = np.float32(seq + v)
    assert oracle.reduk("sum", x, [0], "float32", ls=1) == seq
    # with 4 lanes: four interleaved partial sums, then (l0+l2)+(l1+l3)
    parts = []
    for lid in range(4):
        s = np.float32(0)
        for v in x[lid::4]:
            s = np.float32(s + v)
        parts.append(s)
    want = np.float32(np.float32(parts[0] + parts[2]) + np.float32(parts[1] + parts[3]))
    assert oracle.reduk("sum", x, [0], "float32", ls=4) == want


def test_contig_muladd_two_roundings(oracle):
    rng = np.random.default_rng(0)
    a = rng.uniform(-1, 1, 1 << 16).astype(np.float32)
    b = rng.uniform(-1, 1, 1 << 16).astype(np.float32)
    c = np.empty_like(a)
    oracle.elemwise_contig_muladd(a, b, c)
    assert np.array_equal(c, a * b + np.float32(0.5))
    # a fused multiply-add would differ somewhere on this input
    fused = (a.astype(np.float64) * b.astype(np.float64) + 0.5).astype(np.float32)
    assert not np.array_equal(c, fused)


# ---- take1: tests/check_array.c:17-250 and pygpu/tests/test_gpu_ndarray.py:740-754 ----

@pytest.mark.parametrize("case", KATS["take1"]["cases"], ids=lambda c: "x".join(map(str, c["v_shape"])))
def test_take1_reference_vectors(oracle, case):
    v = np.arange(case["v_elems"], dtype=np.uint32).reshape(case["v_shape"])
    got, err = oracle.take1(v, np.array(case["index"], dtype=np.int64))
    assert err == 0
    assert got.ravel().tolist() == case["expect"]


@pytest.mark.parametrize("case", KATS["take1"]["pygpu_cases"]["cases"],
                         ids=lambda c: "x".join(map(str, c["shape"])))
def test_take1_is_numpy_take(oracle, case):
    rng = np.random.default_rng(5)
    v = rng.standard_normal(case["shape"]).astype(np.float32)
    idx = np.array(case["index"])
    got, err = oracle.take1(v, idx)
    assert err == 0 and np.array_equal(got, v.take(idx, axis=0))


def test_take1_strided_source_wrap_and_bounds(oracle):
    rng = np.random.default_rng(6)
    base = rng.integers(0, 1 << 30, size=(9, 6, 10), dtype=np.int32)
    v = base[::2, ::-1, 1::3]                       # (5, 6, 3), mixed-sign strides
    for dt in (np.int8, np.uint8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64):
        idx = np.array([4, 0, 3, 3, 1], dtype=dt)
        got, err = oracle.take1(v, idx)
        assert err == 0 and np.array_equal(got, v[idx.astype(np.int64)])
    idx = np.array([-1, -5, 2], dtype=np.int32)
    got, err = oracle.take1(v, idx)
    assert err == 0 and np.array_equal(got, v[[4, 0, 2]])
    # one wrap only: -6 and 5 are outside [0, 5); those rows are left alone
    out = np.full((4, 6, 3), -7, dtype=np.int32)
    got, err = oracle.take1(v, np.array([1, -6, 5, 2], dtype=np.int64), out=out)
    assert err == -1
    assert np.array_equal(got[[0, 3]], v[[1, 2]]) and np.all(got[[1, 2]] == -7)


# ---- map + reduce in one kernel: pygpu/reduction.py:33-134 with map_expr -------

def test_reduk_map_is_numpy_on_exact_data(oracle):
    """Small integers in float: every product and partial sum is exact, so the
    template's order does not matter and NumPy is the answer bit for bit.  The
    shapes are the reference's own broadcast case
    (pygpu/tests/test_reduction.py:57-84: (5,10,15) * (1,10,15), axis 1)."""
    rng = np.random.default_rng(21)
    for dt in (np.float32, np.float64):
        x = rng.integers(-8, 9, size=(5, 10, 15)).astype(dt)
        y = rng.integers(-8, 9, size=(1, 10, 15)).astype(dt)
        for axes in ([1], [0], [2], [0, 2], [0, 1, 2]):
            got = oracle.reduk_map2(oracle.MAP_MUL, oracle.RED_ADD, x, y, 0.0, axes, ls=16)
            assert np.array_equal(got, (x * y).sum(axis=tuple(axes)))
            got = oracle.reduk_map2(oracle.MAP_ABSDIFF, oracle.RED_MAX, x, y, 0.0, axes, ls=8)
            assert np.array_equal(got, np.abs(x - y).max(axis=tuple(axes)))
            got = oracle.reduk_map2(oracle.MAP_SAXPY, oracle.RED_ADD, x, y, 3.0, axes, ls=4)
            assert np.array_equal(got, (dt(3) * x + y).sum(axis=tuple(axes)))
            got = oracle.reduk_map2(oracle.MAP_SQUARE, oracle.RED_ADD, x, y, 0.0, axes, ls=1)
            assert np.array_equal(got, np.broadcast_to(x * x, (5, 10, 15)).sum(axis=tuple(axes)))


def test_reduk_map_strided_views_and_tolerance(oracle):
    rng = np.random.default_rng(22)
    xb = rng.standard_normal((12, 9, 14))
    yb = rng.standard_normal((14, 9, 12))
    x, y = xb[::2, ::-1, 1::3], yb.T[::2, :, 1::3]          # both (6, 9, 5)
    got = oracle.reduk_map2(oracle.MAP_MUL, oracle.RED_ADD, x, y, 0.0, [0, 2], ls=32)
    np.testing.assert_allclose(got, (x * y).sum(axis=(0, 2)), rtol=1e-12, atol=1e-12)
    # one lane per group is the plain left-to-right loop
    got1 = oracle.reduk_map2(oracle.MAP_MUL, oracle.RED_ADD, x, y, 0.0, [1], ls=1)
    want = np.zeros((6, 5))
    for j in range(9):
        want = want + x[:, j, :] * y[:, j, :]
    assert np.array_equal(got1, want)
