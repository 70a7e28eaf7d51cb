"""Helper of test_host_logic_without_device.py (not collected by pytest): random
chains of basic indexing, transposition and reshaping on a GpuArray and on the
NumPy array of the same shape, side by side.  The reference's own tests hold
shape, strides and flags to NumPy's (pygpu/tests/test_gpu_ndarray.py:460-579);
here every step of a chain is held to them, and the byte offset as well.  No
kernel result is looked at, so the stand-in runtime is enough."""
import sys

import numpy as np

sys.path.insert(0, ".")
import libgpuarray_amd as ga                      # noqa: E402

ctx = ga.init("hip0")
rng = np.random.default_rng(int(sys.argv[1]))
chains = int(sys.argv[2])


def random_key(shape):
    key = []
    for d in shape:
        r = rng.random()
        if r < 0.15 and d > 0:
            key.append(int(rng.integers(-d, d)))
        elif r < 0.85:
            step = int(rng.choice([1, 1, 2, 3, -1, -2]))
            a = int(rng.integers(-d - 1, d + 2))
            b = int(rng.integers(-d - 1, d + 2))
            key.append(slice(a if rng.random() < 0.7 else None, b if rng.random() < 0.7 else None, step))
        else:
            key.append(slice(None))
    cut = int(rng.integers(0, len(key) + 1))
    if rng.random() < 0.3:
        key = key[:cut] + [Ellipsis]          # trailing dims in full
    if rng.random() < 0.2:
        key.insert(int(rng.integers(0, len(key) + 1)), None)
    return tuple(key)


def same(g, h, base_ptr, what):
    assert g.shape == h.shape, (what, g.shape, h.shape)
    if h.size > 0:
        # NumPy normalises the strides of size-1 dims only for contiguity; compare where extent > 1
        for d, (sg, sh) in enumerate(zip(g.strides, h.strides)):
            assert h.shape[d] <= 1 or sg == sh, (what, g.strides, h.strides, h.shape)
        assert g.offset == h.__array_interface__["data"][0] - base_ptr, (what, g.offset)
        assert bool(g.flags.c_contiguous) == h.flags.c_contiguous, (what, "C", h.shape, h.strides)
        assert bool(g.flags.f_contiguous) == h.flags.f_contiguous, (what, "F", h.shape, h.strides)


for chain in range(chains):
    nd = int(rng.integers(1, 5))
    shape = tuple(int(rng.integers(1, 7)) for _ in range(nd))
    dt = str(rng.choice(["float32", "int8", "float64", "int16"]))
    order = str(rng.choice(["C", "F"]))
    h0 = np.zeros(shape, dt, order=order)
    g = ga.zeros(shape, dt, order=order, context=ctx)
    h = h0
    # (a fresh array starts at offset 0, or at 64 in a DEBUG build of the library)
    base_ptr = h0.__array_interface__["data"][0] - g.offset
    trail = [(shape, dt, order)]
    same(g, h, base_ptr, trail)
    for step in range(int(rng.integers(1, 6))):
        if h.ndim == 0:
            break
        r = rng.random()
        if r < 0.5:
            key = random_key(h.shape)
            trail.append(("index", key))
            h = h[key]
            g = g[key]
            if not isinstance(h, np.ndarray):      # NumPy hands out a scalar for a 0-d result
                assert g.shape == ()
                break
        elif r < 0.75:
            perm = tuple(int(x) for x in rng.permutation(h.ndim))
            trail.append(("transpose", perm))
            h = h.transpose(perm)
            g = g.transpose(*perm) if rng.random() < 0.5 else g.transpose(perm)
        else:
            # a shape with the same element count: merge two neighbours or split one dim
            dims = list(h.shape)
            if len(dims) >= 2 and rng.random() < 0.5:
                i = int(rng.integers(0, len(dims) - 1))
                dims[i:i + 2] = [dims[i] * dims[i + 1]]
            else:
                i = int(rng.integers(0, len(dims)))
                f = [k for k in (2, 3) if dims[i] % k == 0]
                if f:
                    k = int(rng.choice(f))
                    dims[i:i + 1] = [k, dims[i] // k]
            ro = str(rng.choice(["C", "F"]))
            trail.append(("reshape", tuple(dims), ro))
            h2 = h.reshape(dims, order=ro)
            g2 = g.reshape(tuple(dims), order=ro)
            assert g2.shape == h2.shape, trail
            if not np.shares_memory(h2, h0) and h2.size > 0:
                break            # NumPy had to copy: the chain's memory ends here
            if h2.size > 0 and h.size > 1:
                # NumPy found a view; the reference's rule is NumPy's (src/gpuarray_array.c:611-772)
                h, g = h2, g2
            else:
                break
        same(g, h, base_ptr, trail)
print("views ok")
