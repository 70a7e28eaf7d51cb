"""Helper of test_host_logic_without_device.py (not collected by pytest): drives
the reduction and elementwise planners over random element types, shapes,
steps, offsets and axis sets against the stand-in runtime, whose launches do
nothing.  What is asked is that every call returns (no crash in the host
arithmetic that picks vector widths, lane geometry and splits) with a result
of the right shape."""
import sys

import numpy as np

sys.path.insert(0, ".")
sys.path.insert(0, "tests")
import libgpuarray_amd as ga                      # noqa: E402
from libgpuarray_amd import reduction as R        # noqa: E402
from libgpuarray_amd.elemwise import elemwise2    # noqa: E402
from support import to_gpu_view                   # noqa: E402

ctx = ga.init("hip0")
rng = np.random.default_rng(int(sys.argv[1]))
cases = int(sys.argv[2])
pool = [1, 2, 3, 4, 5, 7, 8, 16, 17, 31, 32, 33, 64, 100, 129, 250, 256, 257, 1000, 1023, 4099]
types = ["int8", "uint8", "int16", "int32", "int64", "float16", "float32", "float64", "bool"]
for case in range(cases):
    nd = int(rng.integers(1, 5))
    while True:
        shape = tuple(int(rng.choice(pool)) for _ in range(nd))
        if np.prod(shape) <= 2_000_000:
            break
    dt = str(rng.choice(types))
    steps = [int(rng.choice([1, 1, 2, 3, 4])) for _ in shape]
    base = np.zeros(tuple(s * st + int(rng.integers(0, 4)) for s, st in zip(shape, steps)), dt)
    idx = []
    for s, st, b in zip(shape, steps, base.shape):
        start = int(rng.integers(0, b - (s - 1) * st))
        idx.append(slice(start, start + (s - 1) * st + 1, st))
    view = base[tuple(idx)]
    if nd > 1 and rng.random() < 0.3:
        view = view.transpose(rng.permutation(nd))
    k = int(rng.integers(1, nd + 1))
    axes = tuple(sorted(rng.choice(nd, k, replace=False).tolist()))
    g, _ = to_gpu_view(view, ctx)
    want = view.sum(axis=axes).shape
    print(case, dt, view.shape, view.strides, axes, flush=True)
    assert np.asarray(R.sum(g, axis=axes)).shape == want
    assert np.asarray(R.any(g, axis=axes)).shape == want
    if dt != "bool":
        assert np.asarray(R.max(g, axis=axes)).shape == want
        v, i = R.maxandargmax(g, axis=axes)
        assert np.asarray(i).shape == want
    if dt != "bool":
        assert elemwise2(g, "+", g, g).shape == view.shape
    # the copy family: a contiguous copy in either order, a cast, an assignment
    # through a stepped key, a gather along the first axis
    assert g.copy("C").shape == view.shape and g.copy("F").shape == view.shape
    assert g.astype("float32" if dt != "float32" else "int32").shape == view.shape
    if view.shape[0] > 1:
        g[::2] = g[::2].copy()
        picks = rng.integers(0, view.shape[0], size=int(rng.integers(1, 40)))
        assert g.take1(ga.array(picks, context=ctx)).shape == (len(picks),) + view.shape[1:]
# fixed shapes that take the planners' special routes: rows of at most 32 bytes
# walked in registers, leading dims over short kept rows (folded), a flat kernel
# with a narrow side beyond one fill of the chip, an outer product
if int(sys.argv[1]) == 0:
    for dt, shape in (("float32", (20000, 3)), ("float16", (20011, 6)), ("uint8", (70001, 12)), ("int64", (16385, 2))):
        g = ga.zeros(shape, dt, context=ctx)
        assert np.asarray(R.sum(g, axis=(1,))).shape == shape[:1]
        v, i = R.maxandargmax(g, axis=(1,))
        assert np.asarray(i).shape == shape[:1]
    for dt, shape, axes in (("float32", (1 << 20, 10), (0,)), ("int8", (1 << 22, 3), (0,)), ("float32", (1024, 1024, 4), (0, 1))):
        g = ga.zeros(shape, dt, context=ctx)
        assert np.asarray(R.sum(g, axis=axes)).shape == tuple(d for k, d in enumerate(shape) if k not in axes)
    g = ga.zeros((3 << 20,), "uint8", context=ctx)
    assert g.astype("float32").shape == g.shape and g.astype("float32").astype("float16").shape == g.shape
    col, row = ga.zeros((2048, 1), "float32", context=ctx), ga.zeros((1, 2048), "float32", context=ctx)
    assert elemwise2(col, "*", row, col, broadcast=True).shape == (2048, 2048)
print("planner ok")
