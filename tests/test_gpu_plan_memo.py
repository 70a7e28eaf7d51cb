"""Operators keep the plans of the last few layouts they were called on, and a
call on a layout seen before launches from the kept plan.  What these tests
hold: calls that differ in a single input of the planners (alignment of the
first element, step, order of the axes, how far the buffer extends behind the
last element, a tuning knob) each get their own plan, in any order of calls
and after more layouts than an operator keeps; results are compared with
NumPy every time.  (Run with GPUARRAY_REDUX_MEMO=2 and GPUARRAY_ELEMWISE_MEMO=2
in the environment, the library also plans every remembered call anew and
stops the process if the two plans differ.)"""
import numpy as np
import pytest

import libgpuarray_amd as ga
from libgpuarray_amd import gpuarray, reduction as R

pytestmark = pytest.mark.gpu


def _layouts(rng, rows, cols, dtype):
    """Views of one logical shape (rows, cols) that differ in one property each."""
    def fresh():
        return rng.integers(-20, 21, size=(rows, cols)).astype(dtype)

    out = []
    h = fresh()
    out.append(("dense, aligned", h, lambda g: g))
    big = rng.integers(-20, 21, size=(rows, cols + 1)).astype(dtype)
    out.append(("rows one element off", big[:, 1:], lambda g: g[:, 1:]))
    flat = rng.integers(-20, 21, size=rows * cols + 3).astype(dtype)
    out.append(("dense, first element off a 16-byte boundary", flat[3:].reshape(rows, cols),
                lambda g: g[3:].reshape((rows, cols))))
    wide = rng.integers(-20, 21, size=(rows, 2 * cols)).astype(dtype)
    out.append(("every other column", wide[:, ::2], lambda g: g[:, ::2]))
    t = rng.integers(-20, 21, size=(cols, rows)).astype(dtype)
    out.append(("transposed", t.T, lambda g: g.T))
    tall = rng.integers(-20, 21, size=(rows + 5, cols)).astype(dtype)
    out.append(("the last rows of a longer buffer", tall[5:], lambda g: g[5:]))
    out.append(("the first rows of a longer buffer", tall[:rows], lambda g: g[:rows]))
    return out


@pytest.mark.parametrize("dtype,cols", [("float32", 1023), ("int32", 250), ("uint8", 4099), ("float64", 33)])
def test_reductions_on_alternating_layouts(ctx, dtype, cols):
    rng = np.random.default_rng(4242)
    rows = 257
    cases = []
    for name, host, view in _layouts(rng, rows, cols, dtype):
        base = host.base if host.base is not None else host
        while base.base is not None:
            base = base.base
        g = view(gpuarray.array(base, context=ctx))
        assert g.shape == host.shape, name
        cases.append((name, host, g))
    order = list(range(len(cases)))
    for rep in range(4):
        rng.shuffle(order)
        for k in order + order[:3]:          # some layouts twice in a row, all of them again later
            name, host, g = cases[k]
            for axes in ((1,), (0,), (0, 1)):
                if host.dtype.kind == "f":
                    got = np.asarray(R.sum(g, axis=axes))
                    assert np.array_equal(got, host.sum(axis=axes)), (name, axes, rep)    # small integers: exact
                else:
                    got = np.asarray(R.sum(g, axis=axes, dtype="int64"))
                    assert np.array_equal(got, host.sum(axis=axes, dtype=np.int64)), (name, axes, rep)
            v, i = R.maxandargmax(g, axis=(1,))
            assert np.array_equal(np.asarray(v), host.max(axis=1)), (name, rep)
            assert np.array_equal(np.asarray(i), host.argmax(axis=1)), (name, rep)


@pytest.mark.parametrize("dtype,cols", [("float32", 1024), ("float32", 1023), ("int16", 300), ("float64", 64)])
def test_elementwise_on_alternating_layouts(ctx, dtype, cols):
    rng = np.random.default_rng(4343)
    rows = 130
    k = ga.GpuElemwise(ctx, "c = a + b * s", [ga.arg("a", dtype, read=True), ga.arg("b", dtype, read=True),
                                             ga.arg("s", dtype, scalar=True), ga.arg("c", dtype, write=True)])
    cases = []
    for name, host, view in _layouts(rng, rows, cols, dtype):
        base = host
        while base.base is not None:
            base = base.base
        cases.append((name, host, view(gpuarray.array(base, context=ctx))))
    outs = [("dense result", lambda: gpuarray.empty((rows, cols), dtype, context=ctx), lambda g: g),
            ("result rows one element off", lambda: gpuarray.empty((rows, cols + 1), dtype, context=ctx),
             lambda g: g[:, 1:]),
            ("transposed result", lambda: gpuarray.empty((cols, rows), dtype, context=ctx), lambda g: g.T)]
    order = [(i, j, o) for i in range(len(cases)) for j in (0, 4) for o in range(len(outs))]
    for rep in range(3):
        rng.shuffle(order)
        for i, j, o in order:
            (na, ha, gaa), (nb, hb, gb) = cases[i], cases[j]
            c = outs[o][2](outs[o][1]())
            s = int(rng.integers(-3, 4))           # the scalar changes from call to call
            k(gaa, gb, np.dtype(dtype).type(s), c)
            want = (ha + hb * np.dtype(dtype).type(s)).astype(dtype)
            assert np.array_equal(np.asarray(c), want), (na, nb, outs[o][0], rep)
    # broadcast operands: a row and a column against the dense array
    kb = ga.GpuElemwise(ctx, "c = a + b", [ga.arg("a", dtype, read=True), ga.arg("b", dtype, read=True),
                                           ga.arg("c", dtype, write=True)])
    ha = cases[0][1]
    row = rng.integers(-5, 6, size=(1, cols)).astype(dtype)
    col = rng.integers(-5, 6, size=(rows, 1)).astype(dtype)
    grow, gcol = gpuarray.array(row, context=ctx), gpuarray.array(col, context=ctx)
    for rep in range(6):
        for hb, gbb in ((row, grow), (col, gcol), (ha, cases[0][2])):
            c = gpuarray.empty((rows, cols), dtype, context=ctx)
            kb(cases[0][2], gbb, c, broadcast=True)
            assert np.array_equal(np.asarray(c), (ha + hb).astype(dtype)), rep


def test_a_tuning_knob_read_again_is_a_new_plan(ctx, knobs):
    """The kept plans belong to the tuning table they were made under."""
    x = np.random.default_rng(7).integers(-9, 10, size=1 << 22).astype(np.float32)
    g = gpuarray.array(x, context=ctx)
    want = x.sum(dtype=np.float64)

    def launches():
        ctx.kernel_timing(True)
        got = R.sum(g)
        n = len(ctx.kernel_times())
        ctx.kernel_timing(False)
        assert float(np.asarray(got)) == want          # small integers: exact
        return n
    assert launches() == 1 and launches() == 1         # a split sum that ends in its own launch
    knobs(REDUX_FUSED=0)
    assert launches() == 2 and launches() == 2         # the same call, planned again: a second launch
    knobs(REDUX_FUSED=None)
    assert launches() == 1
    # and the elementwise side: the transposed-tile size is part of the plan's geometry
    a = np.random.default_rng(8).integers(0, 50, size=(700, 900)).astype(np.float32)
    k = ga.GpuElemwise(ctx, "dst = src", [ga.arg("src", "float32", read=True), ga.arg("dst", "float32", write=True)])
    gi = gpuarray.array(a, context=ctx)
    for tile in (64, 128, None, 64):
        knobs(ELEMWISE_TTILE=tile)
        for _ in range(2):
            o = gpuarray.empty((900, 700), "float32", context=ctx)
            k(gi.T, o)
            assert np.array_equal(np.asarray(o), a.T), tile
