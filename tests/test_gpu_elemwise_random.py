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


@pytest.mark.parametrize("seed", range(3))
def test_large_planes_and_flat_size_classes_match_numpy(ctx, knobs, seed):
    """The paths whose launch shape depends on size: transposed operands over
    planes of up to 14 x 14 large tiles with ragged edges (tile size, band
    height, diagonal order and panel width drawn per case, or left to the
    library), a transposed result, several planes; and the flat kernel at two
    to eight million elements, where it moves two or four adjacent chunks per
    lane, with views that start off a 16-byte boundary.  Values are small
    integers, so every type's result is exact: bit for bit against NumPy."""
    from libgpuarray_amd import gpuarray
    rng = np.random.default_rng(700 + seed)
    kernels = {}

    def kernel(dt, expr, names):
        if (dt, expr) not in kernels:
            args = [arg(n, dt, read=True) for n in names[:-1]] + [arg(names[-1], dt, write=True)]
            kernels[(dt, expr)] = ga.GpuElemwise(ctx, expr, args, convert_f16=True)
        return kernels[(dt, expr)]

    def values(shape, dt):
        return rng.integers(0, 11, size=shape).astype(dt)

    for case in range(10):
        knobs(ELEMWISE_TTILE=None, ELEMWISE_BAND=None, ELEMWISE_PANEL=None)
        dt = str(rng.choice(["float32", "float32", "float64", "int16"]))
        mode = int(rng.integers(0, 4))
        if mode <= 1:
            if rng.random() < 0.5:
                knobs(ELEMWISE_TTILE=rng.choice([64, 128]))
            if rng.random() < 0.6:
                knobs(ELEMWISE_BAND=rng.choice([0, 0, 1, 2, 8]), ELEMWISE_PANEL=rng.choice([0, 0, 1, 3, 16]))
            ny = int(rng.integers(1, 14)) * 128 + int(rng.choice([0, 0, 4, 8, 60, 100]))
            nx = int(rng.integers(1, 14)) * 128 + int(rng.choice([0, 0, 4, 12, 64, 124]))
            planes = int(rng.choice([1, 1, 1, 2, 5]))
            lead = (planes,) if planes > 1 else ()
            swap = list(range(len(lead))) + [len(lead) + 1, len(lead)]
            a = values(lead + (nx, ny), dt)
            a_t = np.swapaxes(a, -1, -2)
            g_t = gpuarray.array(a, context=ctx).transpose(swap)
            if mode == 0:       # transposed input, two broadcast inputs
                b, c = values((1,) * len(lead) + (1, nx), dt), values((1,) * len(lead) + (ny, 1), dt)
                out = gpuarray.empty(lead + (ny, nx), dt, context=ctx)
                kernel(dt, "o = a + b*c", "abco")(g_t, gpuarray.array(b, context=ctx), gpuarray.array(c, context=ctx), out)
                want = (a_t + b * c).astype(dt)
            else:               # transposed result, a plain and a transposed input
                x = values(lead + (ny, nx), dt)
                out = gpuarray.empty(lead + (nx, ny), dt, context=ctx).transpose(swap)
                kernel(dt, "o = a + b", "abo")(gpuarray.array(x, context=ctx), g_t, out)
                want = (x + a_t).astype(dt)
            assert np.array_equal(np.asarray(out), want), (seed, case, dt, mode, ny, nx, planes)
        else:
            n = int(rng.choice([1 << 21, 3 << 20, 1 << 22, 3 << 21, 1 << 23])) + int(rng.integers(-3000, 3000))
            off = int(rng.choice([0, 0, 1, 3]))
            dst_off = off if mode == 2 else 0       # mode 3: the result starts at another offset than the inputs
            a, b = values(n + 4, dt), values(n + 4, dt)
            whole = gpuarray.zeros((n + 4,), dt, context=ctx)
            kernel(dt, "o = a + b", "abo")(gpuarray.array(a, context=ctx)[off:off + n],
                                           gpuarray.array(b, context=ctx)[off:off + n], whole[dst_off:dst_off + n])
            got = np.asarray(whole)
            assert np.array_equal(got[dst_off:dst_off + n], (a[off:off + n] + b[off:off + n]).astype(dt)), (seed, case, dt, n, off)
            assert not got[:dst_off].any() and not got[dst_off + n:].any(), (seed, case, "outside the view")
