"""GpuArray_take1 on the device against the CPU checker and the reference's own
vectors (tests/check_array.c:17-294, pygpu/tests/test_gpu_ndarray.py:740-754).
Every call goes through the C entry point; results are bit-exact."""
import ctypes as C
import json
import os

import numpy as np
import pytest

import libgpuarray_amd as ga
from libgpuarray_amd import _lib, gpuarray
from support import to_gpu_view

pytestmark = pytest.mark.gpu
KATS = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kats.json")))


@pytest.mark.parametrize("case", KATS["take1"]["cases"], ids=lambda c: "x".join(map(str, c["v_shape"])))
def test_reference_vectors(ctx, case):
    v = np.arange(case["v_elems"], dtype=np.uint32).reshape(case["v_shape"])
    g = gpuarray.array(v, context=ctx)
    gi = gpuarray.array(np.array(case["index"], dtype=np.int64), context=ctx)
    assert np.asarray(g.take1(gi)).ravel().tolist() == case["expect"]


@pytest.mark.parametrize("case", KATS["take1"]["pygpu_cases"]["cases"],
                         ids=lambda c: "x".join(map(str, c["shape"])))
@pytest.mark.parametrize("offseted", [False, True])
def test_pygpu_cases(ctx, case, offseted):
    rng = np.random.default_rng(11)
    shp = list(case["shape"])
    host = rng.standard_normal([shp[0] + 1] + shp[1:]).astype(np.float32)
    v = host[1:] if offseted else host[:-1]
    g, _ = to_gpu_view(v, ctx)
    idx = np.array(case["index"])
    got = np.asarray(g.take1(gpuarray.array(idx, context=ctx)))
    assert np.array_equal(got, v.take(idx, axis=0))


def test_offset_index_does_not_trip_the_bounds_check(ctx):     # check_array.c:252-279
    v = gpuarray.array(np.arange(4, dtype=np.uint32), context=ctx)
    i = gpuarray.array(np.array([20, 3, 3, 2], dtype=np.uint32), context=ctx)
    got = np.asarray(v.take1(i[2:]))
    assert got.tolist() == [3, 2]


INDEX_TYPES = [np.int8, np.uint8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64]


@pytest.mark.parametrize("itype", INDEX_TYPES, ids=lambda t: np.dtype(t).name)
def test_index_types_and_strided_sources(ctx, oracle, itype):
    rng = np.random.default_rng(12)
    base = rng.integers(0, 1 << 30, size=(9, 6, 10), dtype=np.int32)
    for v in (base, base[::2, ::-1, 1::3], base[::-1], base.transpose(0, 2, 1), base[:, :, ::2],
              base[:, 2], base[:, 1, 3]):
        n = v.shape[0]
        idx = rng.integers(0, n, size=17).astype(itype)
        g, _ = to_gpu_view(v, ctx)
        got = np.asarray(g.take1(gpuarray.array(idx, context=ctx)))
        want, err = oracle.take1(v, idx)
        assert err == 0 and np.array_equal(got, want)
        if np.dtype(itype).kind == "i":
            neg = (idx.astype(np.int64) - n).astype(itype)
            got = np.asarray(g.take1(gpuarray.array(neg, context=ctx)))
            assert np.array_equal(got, want)


@pytest.mark.parametrize("dtype", ["uint8", "float16", "int16", "float32", "float64"])
def test_element_types_and_wide_rows(ctx, oracle, dtype):
    rng = np.random.default_rng(13)
    dt = np.dtype(dtype)
    raw = rng.integers(0, 256, size=(37, 3001 * dt.itemsize), dtype=np.uint8)
    v = raw.view(dt)                        # arbitrary bit patterns, NaN payloads included
    idx = rng.integers(-37, 37, size=50)
    got = np.asarray(gpuarray.array(v, context=ctx).take1(gpuarray.array(idx, context=ctx)))
    want, err = oracle.take1(v, idx)
    assert err == 0
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))


def test_complex_is_refused_like_other_kernels(ctx):
    v = gpuarray.array(np.zeros((3, 2), np.complex64), context=ctx)
    with pytest.raises(_lib.UnsupportedException):
        v.take1(gpuarray.array(np.array([0]), context=ctx))


def test_out_of_bounds_reports_and_skips(ctx, oracle):
    v = np.arange(40, dtype=np.float32).reshape(5, 8)
    g = gpuarray.array(v, context=ctx)
    for bad in ([1, 5, 2], [1, -6, 2], [np.iinfo(np.int64).min, 0, 1]):
        with pytest.raises(IndexError, match="Index out of bounds"):
            g.take1(gpuarray.array(np.array(bad, dtype=np.int64), context=ctx))
    # the error word was reset: the next checked call passes
    assert np.array_equal(np.asarray(g.take1(gpuarray.array(np.array([4, -5]), context=ctx))),
                          v[[4, 0]])
    # unchecked call: rows with a bad index keep what the destination held
    out = gpuarray.array(np.full((4, 8), -7, dtype=np.float32), context=ctx)
    gi = gpuarray.array(np.array([1, -6, 5, 2], dtype=np.int64), context=ctx)
    assert _lib.lib.GpuArray_take1(out._ptr(), g._ptr(), gi._ptr(), 0) == _lib.GA_NO_ERROR
    want, err = oracle.take1(v, np.array([1, -6, 5, 2]), out=np.full((4, 8), -7, dtype=np.float32))
    assert err == -1 and np.array_equal(np.asarray(out), want)
    # the flag is still set; a checked call reports it once and clears it
    good = gpuarray.array(np.array([0]), context=ctx)
    with pytest.raises(IndexError):
        g.take1(good)
    assert np.array_equal(np.asarray(g.take1(good)), v[[0]])


def test_argument_rules(ctx):                      # src/gpuarray_array.c:408-446
    L = _lib.lib
    v = gpuarray.array(np.zeros((4, 6), np.float32), context=ctx)
    i = gpuarray.array(np.array([0, 1, 2]), context=ctx)

    def call(a, v_, i_):
        return L.GpuArray_take1(a._ptr(), v_._ptr(), i_._ptr(), 1)

    ok = gpuarray.empty((3, 6), "float32", context=ctx)
    assert call(ok, v, i) == _lib.GA_NO_ERROR
    assert call(gpuarray.empty((3, 5), "float32", context=ctx), v, i) == _lib.GA_INVALID_ERROR
    assert call(gpuarray.empty((2, 6), "float32", context=ctx), v, i) == _lib.GA_INVALID_ERROR
    assert call(gpuarray.empty((3,), "float32", context=ctx), v, i) == _lib.GA_INVALID_ERROR
    i2 = gpuarray.array(np.zeros((3, 1), np.int64), context=ctx)
    assert call(ok, v, i2) == _lib.GA_INVALID_ERROR
    assert call(gpuarray.empty((6, 6), "float32", context=ctx)[::2], v, i) == _lib.GA_INVALID_ERROR
    i6 = gpuarray.array(np.zeros(6, np.int64), context=ctx)
    assert call(ok, v, i6[::2]) == _lib.GA_INVALID_ERROR
    ro = gpuarray.empty((3, 6), "float32", context=ctx)
    ro.ga.flags &= ~_lib.GA_WRITEABLE
    assert call(ro, v, i) == _lib.GA_VALUE_ERROR
    raw = gpuarray.array(np.zeros(4 * 6 * 4 + 8, np.uint8), context=ctx)
    un = gpuarray.from_strided(raw, 2, (4, 6), (24, 4), dtype=np.float32)
    assert call(ok, un, i) == _lib.GA_UNALIGNED_ERROR
    fi = gpuarray.array(np.zeros(3, np.float32), context=ctx)
    assert call(ok, v, fi) == _lib.GA_VALUE_ERROR
    with pytest.raises(ValueError):
        v.take1(i2)
    # empty index and empty rows are not an error
    e = gpuarray.array(np.zeros(0, np.int64), context=ctx)
    assert v.take1(e).shape == (0, 6)
    z = gpuarray.empty((4, 0), "float32", context=ctx)
    assert z.take1(i).shape == (3, 0)


def test_large_gather_roundtrip(ctx):
    """2^26 floats: a permutation gather followed by the inverse permutation
    returns the source bit for bit."""
    rng = np.random.default_rng(14)
    n0, n1 = 1 << 14, 1 << 12
    v = rng.integers(0, 1 << 32, size=(n0, n1), dtype=np.uint32).view(np.float32)
    perm = rng.permutation(n0)
    inv = np.empty_like(perm)
    inv[perm] = np.arange(n0)
    g = gpuarray.array(v, context=ctx)
    t = g.take1(gpuarray.array(perm, context=ctx))
    back = t.take1(gpuarray.array(inv, context=ctx))
    assert np.array_equal(np.asarray(back).view(np.uint32), v.view(np.uint32))
    assert np.array_equal(np.asarray(t[:64]).view(np.uint32), v[perm[:64]].view(np.uint32))


@pytest.mark.parametrize("width", [4, 12, 32, 100, 256, 512, 516])
def test_short_dense_rows(ctx, oracle, width):
    """Rows of at most 128 sixteen-byte chunks take their own kernel (a lane
    moves one chunk of four rows): widths around its limits, row counts that
    leave groups partly empty, negative indices, and rows with a bad index
    left untouched."""
    rng = np.random.default_rng(width)
    for rows, n in ((1000, 1), (37, 5), (300, 1027), (5000, 4099)):
        v = rng.integers(0, 1 << 30, size=(rows, width), dtype=np.int32)
        idx = rng.integers(-rows, rows, size=n)
        g = gpuarray.array(v, context=ctx)
        got = np.asarray(g.take1(gpuarray.array(idx, context=ctx)))
        want, err = oracle.take1(v, idx)
        assert err == 0 and np.array_equal(got, want), (rows, n)
    bad = idx.copy()
    bad[[0, n // 2, n - 1]] = [rows, -rows - 1, rows + 7]
    out = gpuarray.array(np.full((n, width), -7, dtype=np.int32), context=ctx)
    gi = gpuarray.array(bad, context=ctx)
    assert _lib.lib.GpuArray_take1(out._ptr(), g._ptr(), gi._ptr(), 0) == _lib.GA_NO_ERROR
    want, err = oracle.take1(v, bad, out=np.full((n, width), -7, dtype=np.int32))
    assert err == -1 and np.array_equal(np.asarray(out), want)
    with pytest.raises(IndexError):                 # the flag the unchecked call left
        g.take1(gpuarray.array(np.array([0]), context=ctx))
