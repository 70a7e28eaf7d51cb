"""Random reductions against NumPy: element type, rank, extents (chosen to land
in every kernel family: rows sharing a wavefront, rows staged in LDS, shifted
rows, long split rows, columns with one or several outputs per lane), slicing
steps, transposition and axis sets are drawn per case.  Integers, booleans
and arg-reductions must match bit for bit; float sums within 2e-5 of the
float64 sum relative to the sum of magnitudes."""
import numpy as np
import pytest

from libgpuarray_amd import reduction as R
from support import to_gpu_view

pytestmark = pytest.mark.gpu

EXTENTS = [1, 2, 3, 4, 5, 7, 8, 16, 17, 31, 32, 33, 64, 100, 129, 250, 256, 257, 1000, 1023, 4099]
DTYPES = ["int8", "uint8", "int16", "int32", "int64", "float16", "float32", "float64", "bool"]


def draw(rng):
    nd = int(rng.integers(1, 5))
    while True:
        shape = tuple(int(rng.choice(EXTENTS)) for _ in range(nd))
        if np.prod(shape) <= 3_000_000:
            break
    dt = str(rng.choice(DTYPES))
    base_shape = tuple(s * int(rng.choice([1, 1, 2])) + int(rng.choice([0, 0, 1, 3])) for s in shape)
    if dt == "bool":
        base = rng.random(base_shape) < 0.5
    elif dt.startswith("float"):
        base = rng.integers(-20, 20, size=base_shape).astype(dt)
    else:
        info = np.iinfo(dt)
        base = rng.integers(max(info.min, -1000), min(info.max, 1000) + 1, size=base_shape).astype(dt)
    cut = []
    for s, b in zip(shape, base_shape):
        step = 2 if b >= 2 * s and rng.random() < 0.7 else 1
        start = int(rng.integers(0, b - (s - 1) * step))
        cut.append(slice(start, start + (s - 1) * step + 1, step))
    view = base[tuple(cut)]
    if nd > 1 and rng.random() < 0.3:
        view = view.transpose(rng.permutation(nd))
    k = int(rng.integers(1, nd + 1))
    axes = tuple(sorted(rng.choice(nd, k, replace=False).tolist()))
    return dt, view, axes


@pytest.mark.parametrize("seed", range(6))
def test_random_reductions_match_numpy(ctx, seed, knobs):
    knobs(REDUX_SROWS_MIN_ROWS=1)    # staged rows at test sizes too
    rng = np.random.default_rng(1000 + seed)
    for case in range(10):
        dt, view, axes = draw(rng)
        nd = view.ndim
        what = (seed, case, dt, view.shape, view.strides, axes)
        g, _ = to_gpu_view(view, ctx)
        if dt.startswith("float"):
            got = np.asarray(R.sum(g, axis=axes, dtype="float32" if dt == "float16" else None))
            want = view.astype(np.float64).sum(axis=axes)
            scale = np.abs(view.astype(np.float64)).sum(axis=axes)
            assert np.all(np.abs(got - want) <= 2e-5 * np.maximum(scale, 1e-30)), ("sum",) + what
        else:
            got = np.asarray(R.sum(g, axis=axes, dtype="int64"))
            assert np.array_equal(got, view.sum(axis=axes, dtype=np.int64)), ("sum",) + what
        assert np.array_equal(np.asarray(R.any(g, axis=axes)), view.any(axis=axes)), ("any",) + what
        assert np.array_equal(np.asarray(R.all(g, axis=axes)), view.all(axis=axes)), ("all",) + what
        if dt == "bool":
            continue
        assert np.array_equal(np.asarray(R.max(g, axis=axes)), view.max(axis=axes)), ("max",) + what
        assert np.array_equal(np.asarray(R.min(g, axis=axes)), view.min(axis=axes)), ("min",) + what
        moved = np.moveaxis(view, axes, range(nd - len(axes), nd))
        flat = moved.reshape(moved.shape[:nd - len(axes)] + (-1,))
        assert np.array_equal(np.asarray(R.argmax(g, axis=axes)), flat.argmax(axis=-1)), ("argmax",) + what
        assert np.array_equal(np.asarray(R.argmin(g, axis=axes)), flat.argmin(axis=-1)), ("argmin",) + what
