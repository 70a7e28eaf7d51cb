"""Calls recorded into a HIP graph and replayed.

A caller that holds the context's stream (extension "hip_get_stream", the
counterpart of the reference's cuda_get_stream, src/gpuarray/ext_cuda.h) can
put it into capture mode, issue GpuElemwise / GpuReduction calls on arrays
that already exist, and replay the recorded launches with one graph launch.
That only works if a call on warmed-up operators does nothing but launch
kernels on that stream: no allocation, no memset node (GpuArray_memset fills with a
kernel while the stream records), no synchronisation.  Each
replay here follows eager work (new input contents, a synchronisation) and is
compared bit for bit with the same calls issued eagerly."""
import ctypes as C

import numpy as np
import pytest

import libgpuarray_amd as ga
from libgpuarray_amd import _lib, gpuarray
from libgpuarray_amd import reduction as R
from support import arg

pytestmark = pytest.mark.gpu


def test_elemwise_and_reductions_replay_from_a_graph(ctx):
    hip = C.CDLL("libamdhip64.so")
    stream = C.c_void_p(_lib.extension("hip_get_stream", C.c_void_p, [C.c_void_p])(ctx.ctx))
    rows, cols = 384, 1000            # ragged rows: shifted vector loads
    n = rows * cols
    f32 = "float32"
    e1 = ga.GpuElemwise(ctx, "c = a*b + 0.5f", [arg("a", f32, read=True), arg("b", f32, read=True),
                                               arg("c", f32, write=True)])
    e2 = ga.GpuElemwise(ctx, "d = c*c - s", [arg("c", f32, read=True), arg("s", f32, scalar=True),
                                            arg("d", f32, write=True)])
    rsum = ga.GpuReduction(ctx, "sum", f32)
    rmax = ga.GpuReduction(ctx, "maxandargmax", f32)
    a = gpuarray.zeros((n,), f32, context=ctx)
    b = gpuarray.zeros((n,), f32, context=ctx)

    fold_rows = 1 << 19               # sum over a batch of rows of 10 floats: folded rows, three launches
    wide = gpuarray.zeros((fold_rows, 10), f32, context=ctx)
    wide_fill = ga.GpuElemwise(ctx, "w = a * 3.0f", [arg("a", f32, read=True), arg("w", f32, write=True)])

    bump = ga.GpuElemwise(ctx, "z = z + 1", [arg("z", "uint8", read=True, write=True)])

    def outputs():
        return dict(c=gpuarray.zeros((n,), f32, context=ctx), d=gpuarray.zeros((n,), f32, context=ctx),
                    z=gpuarray.zeros((100003,), "uint8", context=ctx),
                    ws=gpuarray.zeros((10,), f32, context=ctx),
                    rs=gpuarray.zeros((rows,), f32, context=ctx), tot=gpuarray.zeros((), f32, context=ctx),
                    cs=gpuarray.zeros((cols,), f32, context=ctx),
                    mv=gpuarray.zeros((rows,), f32, context=ctx),
                    mi=gpuarray.zeros((rows,), "int64", context=ctx))

    def issue(o):
        e1(a, b, o["c"])
        e2(o["c"], np.float32(0.25), o["d"])
        d2 = o["d"].reshape((rows, cols))
        rsum(d2, [1], d0=o["rs"])
        rsum(o["d"], [0], d0=o["tot"])          # split over many groups: two kernels, scratch partials
        rsum(d2, [0], d0=o["cs"])               # column kernel
        rmax(d2, [1], d0=o["mv"], d1=o["mi"])
        flat = wide.reshape((fold_rows * 10,))
        wide_fill(a[:n // 4], flat[:n // 4])        # part of `wide` follows the inputs
        rsum(wide, [0], d0=o["ws"])
        o["z"].memset(5)                            # recorded as a kernel of the library, not as a memset node
        bump(o["z"])

    eager, replayed = outputs(), outputs()
    issue(eager)                                 # compiles everything, sizes the scratch buffer
    issue(replayed)
    ctx.sync()

    graph, gexec = C.c_void_p(), C.c_void_p()
    assert hip.hipStreamBeginCapture(stream, 0) == 0            # hipStreamCaptureModeGlobal
    try:
        issue(replayed)
    finally:
        rc = hip.hipStreamEndCapture(stream, C.byref(graph))
    assert rc == 0, "a call did something a capturing stream does not allow (hip error %d)" % rc
    assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, C.c_size_t(0)) == 0
    try:
        rng = np.random.default_rng(90)
        for k in range(4):
            ha = rng.standard_normal(n).astype(np.float32)
            hb = rng.standard_normal(n).astype(np.float32)
            a.write(ha)
            b.write(hb)
            for v in replayed.values():          # stale results must not pass for fresh ones
                v.write(np.full(v.shape, 249 if v.dtype == np.uint8 else -7, v.dtype))
            ctx.sync()
            assert hip.hipGraphLaunch(gexec, stream) == 0
            ctx.sync()
            issue(eager)
            ctx.sync()
            for name in eager:
                assert np.array_equal(np.asarray(eager[name]), np.asarray(replayed[name])), (k, name)
            c = ha * hb + np.float32(0.5)
            d = c * c - np.float32(0.25)
            assert np.array_equal(np.asarray(replayed["d"]), d)
            assert np.all(np.asarray(replayed["z"]) == 6)
            assert np.array_equal(np.asarray(replayed["mi"]), d.reshape(rows, cols).argmax(axis=1))
    finally:
        hip.hipGraphExecDestroy(gexec)
        hip.hipGraphDestroy(graph)


def test_scratch_that_a_graph_recorded_is_never_handed_out_again(monkeypatch):
    """A graph holds the address of the scratch buffer its split reductions
    write partials to.  When a later, larger split reduction outgrows that
    buffer, the old one must stay out of circulation: were it given back to
    the memory cache, the caller's next array could land on it and every
    replay would write partials into that array.  A context of its own, so
    that the scratch buffer starts at its smallest size whatever ran before."""
    if ga.count_devices() == 0:
        pytest.skip("no HIP device")
    ctx = ga.init("hip0")
    hip = C.CDLL("libamdhip64.so")
    stream = C.c_void_p(_lib.extension("hip_get_stream", C.c_void_p, [C.c_void_p])(ctx.ctx))
    f32 = "float32"
    rsum = ga.GpuReduction(ctx, "sum", f32)
    n = 1 << 24
    hx = np.random.default_rng(91).standard_normal(n).astype(np.float32)
    x = gpuarray.array(hx, context=ctx)
    tot = gpuarray.zeros((), f32, context=ctx)
    rsum(x, [0], d0=tot)                 # two launches: partials rest in the scratch buffer (1 MiB)
    ctx.sync()
    want = float(np.asarray(tot))
    assert abs(want - float(hx.sum(dtype=np.float64))) <= 1e-5 * abs(float(hx.sum(dtype=np.float64)))
    graph, gexec = C.c_void_p(), C.c_void_p()
    assert hip.hipStreamBeginCapture(stream, 0) == 0
    try:
        rsum(x, [0], d0=tot)
    finally:
        rc = hip.hipStreamEndCapture(stream, C.byref(graph))
    assert rc == 0
    assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, C.c_size_t(0)) == 0
    try:
        # an eager split reduction whose partials outgrow that buffer: 8 pieces
        # for each of 65536 columns, 6 MiB
        monkeypatch.setenv("GPUARRAY_REDUX_GROUPS_PER_CU", "256")
        ctx.reload_tuning()
        wide = gpuarray.zeros((512, 65536), f32, context=ctx)
        cols = gpuarray.empty((65536,), f32, context=ctx)
        rsum(wide, [0], d0=cols)
        monkeypatch.delenv("GPUARRAY_REDUX_GROUPS_PER_CU")
        ctx.reload_tuning()
        ctx.sync()
        # arrays made now take whatever blocks the cache has free
        fresh = [gpuarray.array(np.full(1 << 16, 5.0, np.float32), context=ctx) for _ in range(32)]
        for k in range(3):
            tot.write(np.float32(-1))
            ctx.sync()
            assert hip.hipGraphLaunch(gexec, stream) == 0
            ctx.sync()
            assert float(np.asarray(tot)) == want, k
            for f in fresh:
                assert np.all(np.asarray(f) == 5.0), "a replay wrote into an array allocated after the capture"
    finally:
        hip.hipGraphExecDestroy(gexec)
        hip.hipGraphDestroy(graph)
