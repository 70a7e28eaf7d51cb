"""Random elementwise calls against NumPy: element type, rank, extents,
broadcast operands, slicing steps (negative ones too), C- or Fortran-ordered
roots and a common transposition are drawn per case.  The destination's whole
root buffer is compared, so that a write outside the view shows as well."""
import numpy as np
import pytest

import libgpuarray_amd as ga
from support import to_gpu_view, read_root, root_of, arg

pytestmark = pytest.mark.gpu

EXTENTS = [1, 2, 3, 4, 5, 7, 8, 16, 17, 31, 32, 33, 64, 65, 100, 128, 129, 256, 257, 1000, 1024, 4099]
DTYPES = ["int8", "uint8", "int16", "int32", "int64", "float16", "float32", "float64"]


def operand(rng, shape, dt, may_broadcast):
    own = tuple(1 if (may_broadcast and rng.random() < 0.25) else s for s in shape)
    room = tuple(s * int(rng.choice([1, 1, 2])) + int(rng.choice([0, 0, 1, 3])) for s in own)
    if dt.startswith("float"):
        base = rng.integers(-50, 50, size=room).astype(dt)
    else:
        info = np.iinfo(dt)
        base = rng.integers(info.min, int(info.max) + 1, size=room, dtype=np.int64).astype(dt)
    base = np.asarray(base, order="F" if rng.random() < 0.25 else "C")
    cut = []
    for s, b in zip(own, room):
        step = int(rng.choice([1, 1, 2, -1])) if b >= 2 * s else int(rng.choice([1, 1, -1]))
        span = (s - 1) * abs(step) + 1
        start = int(rng.integers(0, b - span + 1))
        if step > 0:
            cut.append(slice(start, start + span, step))
        else:
            cut.append(slice(start + span - 1, start - 1 if start > 0 else None, step))
    view = base[tuple(cut)]
    assert view.shape == own
    return view


@pytest.mark.parametrize("seed", range(6))
def test_random_elementwise_matches_numpy(ctx, seed):
    rng = np.random.default_rng(2000 + seed)
    kernels = {}
    for case in range(10):
        nd = int(rng.integers(1, 5))
        while True:
            shape = tuple(int(rng.choice(EXTENTS)) for _ in range(nd))
            if np.prod(shape) <= 2_000_000:
                break
        dt = str(rng.choice(DTYPES))
        if dt not in kernels:
            kernels[dt] = ga.GpuElemwise(ctx, "c = a + b", [arg("a", dt, read=True), arg("b", dt, read=True),
                                                            arg("c", dt, write=True)], convert_f16=True)
        a, b = operand(rng, shape, dt, True), operand(rng, shape, dt, True)
        c = operand(rng, shape, dt, False)
        perm = rng.permutation(nd) if (nd > 1 and rng.random() < 0.3) else np.arange(nd)
        a, b, c = a.transpose(perm), b.transpose(perm), c.transpose(perm)
        what = (seed, case, dt, c.shape, a.strides, b.strides, c.strides)
        root = root_of(c)
        expected = root.copy(order="K")
        ga_, gb = to_gpu_view(a, ctx)[0], to_gpu_view(b, ctx)[0]
        gc, croot = to_gpu_view(c, ctx)
        kernels[dt](ga_, gb, gc)
        if dt == "float16":
            want = (a.astype(np.float32) + b.astype(np.float32)).astype(np.float16)
        else:
            with np.errstate(over="ignore"):
                want = (a + b).astype(dt)
        offset = c.__array_interface__["data"][0] - root.__array_interface__["data"][0]
        memory = expected if expected.flags.c_contiguous else expected.T
        np.ndarray(c.shape, dtype=c.dtype, buffer=memory, offset=offset, strides=c.strides)[...] = want
        assert np.array_equal(read_root(croot, root), expected), what
