"""Buffers, contexts, kernels and array views on the device, through the C
ABI.  Scenarios: tests/check_buffer.c:21-177, tests/check_array.c:280-292 and
the view checks of pygpu/tests/test_gpu_ndarray.py:410-579 (NumPy's shape /
strides / flags are the expected values)."""
import ctypes as C
import itertools

import numpy as np
import pytest

import libgpuarray_amd as ga
from libgpuarray_amd import _lib, gpuarray
from support import to_gpu_view, gen_gpuarray

pytestmark = pytest.mark.gpu
lib = _lib.lib


def refcnt(b):
    r = C.c_uint()
    assert lib.gpudata_property(b, _lib.GA_BUFFER_PROP_REFCNT, C.byref(r)) == 0
    return r.value


def test_context_properties(ctx):
    assert ctx.bin_id == "gfx950"
    assert ctx.numprocs == 256
    assert ctx.maxlsize0 == 1024 and ctx.lmemsize >= 64 * 1024
    assert ctx.total_gmem >= ctx.free_gmem > 0
    bad = C.c_size_t()
    assert lib.gpucontext_property(ctx.ctx, 99, C.byref(bad)) == _lib.GA_INVALID_ERROR
    assert lib.gpucontext_property(ctx.ctx, 9999, C.byref(bad)) == _lib.GA_VALUE_ERROR


def test_buffer_alloc_retain_release(ctx):      # check_buffer.c:21-77
    for sz in (0, 1, 1024):
        d = lib.gpudata_alloc(ctx.ctx, sz, None, 0, None)
        assert d and refcnt(d) == 1
        lib.gpudata_release(d)
    d = lib.gpudata_alloc(ctx.ctx, 1024, None, 0, None)
    d2 = lib.gpudata_alloc(ctx.ctx, 1024, None, 0, None)
    lib.gpudata_retain(d)
    assert refcnt(d) == 2
    lib.gpudata_release(d)
    assert refcnt(d) == 1
    lib.gpudata_retain(d); lib.gpudata_retain(d2); lib.gpudata_retain(d)
    assert (refcnt(d), refcnt(d2)) == (3, 2)
    lib.gpudata_release(d)
    assert (refcnt(d), refcnt(d2)) == (2, 2)
    lib.gpudata_release(d); lib.gpudata_release(d2)
    assert (refcnt(d), refcnt(d2)) == (1, 1)
    # share (check_buffer.c:79-93)
    assert lib.gpudata_share(d, d2, None) == 0
    assert lib.gpudata_share(d, d, None) == 1
    lib.gpudata_release(d); lib.gpudata_release(d2)


def test_buffer_read_write_move(ctx):           # check_buffer.c:95-177
    data = np.arange(8, dtype=np.int32)
    d = lib.gpudata_alloc(ctx.ctx, data.nbytes, None, 0, None)
    assert lib.gpudata_write(d, 0, data.ctypes.data, data.nbytes) == 0
    buf = np.zeros(8, np.int32)
    assert lib.gpudata_read(buf.ctypes.data, d, 0, data.nbytes) == 0
    assert np.array_equal(buf, data)
    buf[:] = 0
    assert lib.gpudata_read(buf.ctypes.data, d, 4, data.nbytes - 4) == 0
    assert np.array_equal(buf[:7], data[1:])
    assert lib.gpudata_write(d, 8, data.ctypes.data, data.nbytes - 8) == 0
    assert lib.gpudata_read(buf.ctypes.data, d, 0, data.nbytes) == 0
    assert np.array_equal(buf[2:], data[:6]) and np.array_equal(buf[:2], data[:2])
    d2 = lib.gpudata_alloc(ctx.ctx, data.nbytes * 2, None, 0, None)
    assert lib.gpudata_write(d, 0, data.ctypes.data, data.nbytes) == 0
    assert lib.gpudata_move(d2, data.nbytes, d, 0, data.nbytes) == 0
    assert lib.gpudata_read(buf.ctypes.data, d2, data.nbytes, data.nbytes) == 0
    assert np.array_equal(buf, data)
    assert lib.gpudata_move(d2, 0, d, 4, data.nbytes - 4) == 0
    assert lib.gpudata_read(buf.ctypes.data, d2, 0, data.nbytes) == 0
    assert np.array_equal(buf[:7], data[1:])
    # out-of-range accesses are refused, not executed
    assert lib.gpudata_read(buf.ctypes.data, d, 8, data.nbytes) == _lib.GA_VALUE_ERROR
    assert lib.gpudata_move(d2, data.nbytes * 2, d, 0, 4) == _lib.GA_VALUE_ERROR
    # init flag and its misuse (src/gpuarray_buffer_opencl.c:488-508)
    e = C.c_int(0)
    d3 = lib.gpudata_alloc(ctx.ctx, data.nbytes, data.ctypes.data, _lib.GA_BUFFER_INIT, C.byref(e))
    assert d3
    assert lib.gpudata_read(buf.ctypes.data, d3, 0, data.nbytes) == 0 and np.array_equal(buf, data)
    assert not lib.gpudata_alloc(ctx.ctx, 8, None, _lib.GA_BUFFER_INIT, C.byref(e))
    assert e.value == _lib.GA_VALUE_ERROR
    # memset fills to the END of the buffer
    assert lib.gpudata_memset(d3, 8, 0xAB) == 0
    raw = np.zeros(data.nbytes, np.uint8)
    assert lib.gpudata_read(raw.ctypes.data, d3, 0, data.nbytes) == 0
    assert np.array_equal(raw[:8], data.view(np.uint8)[:8]) and np.all(raw[8:] == 0xAB)
    for b in (d, d2, d3):
        lib.gpudata_release(b)


def test_large_moves_take_the_copy_kernel(ctx, knobs):
    """buffer_move copies large ranges with the library's own kernel when source
    and destination sit equally far from a 16-byte boundary (here from the
    first byte on), with the driver's copy otherwise: same bytes either way,
    nothing outside the range, and a cleared array struct is refused."""
    knobs(MOVE_KERNEL_MIN=1)
    rng = np.random.default_rng(31)
    total = (1 << 20) + 200
    h = rng.integers(0, 256, total).astype(np.uint8)
    src = gpuarray.array(h, context=ctx)
    for so, do, m in ((0, 0, 1 << 20), (3, 3, (1 << 20) + 17), (5, 21, (1 << 19) + 3), (7, 8, 1 << 19),
                      (1, 1, 1), (2, 18, 15), (0, 16, 16), (9, 9, 40), (4, 4, 4099)):
        dst = gpuarray.zeros((total,), "uint8", context=ctx)
        dv, sv = dst[do:do + m], src[so:so + m]          # the views must outlive the call
        assert lib.GpuArray_move(dv._ptr(), sv._ptr()) == 0
        got = np.asarray(dst)
        assert np.array_equal(got[do:do + m], h[so:so + m]), (so, do, m)
        assert not got[:do].any() and not got[do + m:].any(), (so, do, m)
    f = gpuarray.array(rng.standard_normal((700, 300)).astype(np.float32), context=ctx)
    assert np.array_equal(np.asarray(f.copy()), np.asarray(f))
    cleared = _lib.GpuArrayStruct()
    assert lib.GpuArray_move(C.byref(cleared), f._ptr()) == _lib.GA_INVALID_ERROR
    assert lib.GpuArray_read(h.ctypes.data, 4, C.byref(cleared)) == _lib.GA_INVALID_ERROR


def test_user_kernel_written_against_the_toolchain_headers(ctx):
    """Kernel text that leans on the toolchain's HIP headers (half types,
    cross-lane shuffles, float4, the cooperative-groups header) fails against
    the library's own small device runtime and gets a second compile through
    hipRTC: GpuKernel_init accepts any source the backend's compiler accepts
    (reference src/gpuarray/kernel.h:54-70)."""
    src = b"""#include <hip/hip_fp16.h>
#include <hip/hip_cooperative_groups.h>
extern "C" __global__ void lanes(float *out, __half *h, float4 *q, unsigned int n) {
  auto block = cooperative_groups::this_thread_block();
  unsigned int i = blockIdx.x * blockDim.x + block.thread_rank();
  if (i >= n) return;
  float from_left = __shfl_up((float)i, 1);          // lane 0 of a wavefront keeps its own
  out[i] = from_left;
  h[i] = __float2half(0.5f * (float)(i % 7));
  if (i < n / 4) q[i] = make_float4(i, i + 1.0f, i + 2.0f, i + 3.0f);
}"""
    n = 1024
    out = gpuarray.zeros((n,), "float32", context=ctx)
    h = gpuarray.zeros((n,), "float16", context=ctx)
    q = gpuarray.zeros((n,), "float32", context=ctx)
    k = _lib.GpuKernelStruct()
    types = (C.c_int * 4)(_lib.GA_BUFFER, _lib.GA_BUFFER, _lib.GA_BUFFER, _lib.GA_UINT)
    strs = (C.c_char_p * 1)(src)
    log = C.c_char_p()
    rc = lib.GpuKernel_init(C.byref(k), ctx.ctx, 1, strs, None, b"lanes", 4, types, _lib.GA_USE_HALF, C.byref(log))
    assert rc == 0, (log.value or b"").decode(errors="replace")[-800:]
    nn = C.c_uint(n)
    for i, a in enumerate((out.ga.data, h.ga.data, q.ga.data, C.byref(nn))):
        assert lib.GpuKernel_setarg(C.byref(k), i, a) == 0
    gs, ls = C.c_size_t(n // 256), C.c_size_t(256)
    assert lib.GpuKernel_call(C.byref(k), 1, C.byref(gs), C.byref(ls), 0, None) == 0
    idx = np.arange(n)
    want = np.where(idx % 64 == 0, idx, idx - 1).astype(np.float32)
    assert np.array_equal(np.asarray(out), want)
    assert np.array_equal(np.asarray(h), (0.5 * (idx % 7)).astype(np.float16))
    wq = np.zeros(n, np.float32)
    wq[:n] = (np.arange(n // 4)[:, None] + np.arange(4)[None, :]).reshape(-1)[:n]
    assert np.array_equal(np.asarray(q), wq)
    lib.GpuKernel_clear(C.byref(k))
    # text that is simply wrong still fails, and the log holds both tries
    bad = (C.c_char_p * 1)(b'extern "C" __global__ void k(int *p) { p[0] = no_such_thing(3); }')
    assert lib.GpuKernel_init(C.byref(k), ctx.ctx, 1, bad, None, b"k", 1, types, 0, C.byref(log)) == _lib.GA_IMPL_ERROR
    text = (log.value or b"").decode(errors="replace")
    assert "no_such_thing" in text and "second try" in text


def test_user_kernel_through_gpukernel(ctx):
    # a kernel in the reference's dialect, launched with explicit geometry and
    # with GpuKernel_sched's geometry
    src = b"""#include "cluda.h"
KERNEL void axpy(GLOBAL_MEM ga_float *y, GLOBAL_MEM ga_float *x, ga_float a, ga_size n) {
  for (ga_size i = GID_0 * LDIM_0 + LID_0; i < n; i += GDIM_0 * LDIM_0) y[i] = a * x[i] + y[i];
}"""
    n = 100003
    x = np.random.default_rng(0).normal(size=n).astype(np.float32)
    y = np.ones(n, np.float32)
    gx, gy = gpuarray.array(x, context=ctx), gpuarray.array(y, context=ctx)
    k = _lib.GpuKernelStruct()
    types = (C.c_int * 4)(_lib.GA_BUFFER, _lib.GA_BUFFER, _lib.GA_FLOAT, _lib.GA_SIZE)
    strs = (C.c_char_p * 1)(src)
    assert lib.GpuKernel_init(C.byref(k), ctx.ctx, 1, strs, None, b"axpy", 4, types, 0, None) == 0
    a, nn = C.c_float(2.0), C.c_size_t(n)
    assert lib.GpuKernel_setarg(C.byref(k), 0, gy.ga.data) == 0
    assert lib.GpuKernel_setarg(C.byref(k), 1, gx.ga.data) == 0
    assert lib.GpuKernel_setarg(C.byref(k), 2, C.byref(a)) == 0
    assert lib.GpuKernel_setarg(C.byref(k), 3, C.byref(nn)) == 0
    assert lib.GpuKernel_setarg(C.byref(k), 4, C.byref(nn)) == _lib.GA_VALUE_ERROR
    gs, ls = C.c_size_t(0), C.c_size_t(0)
    assert lib.GpuKernel_sched(C.byref(k), n, C.byref(gs), C.byref(ls)) == 0
    assert ls.value == 256 and gs.value == (n + 255) // 256
    assert lib.GpuKernel_call(C.byref(k), 1, C.byref(gs), C.byref(ls), 0, None) == 0
    assert np.array_equal(np.asarray(gy), np.float32(2.0) * x + y)
    # caller-fixed sizes are kept
    gs, ls = C.c_size_t(7), C.c_size_t(0)
    assert lib.GpuKernel_sched(C.byref(k), n, C.byref(gs), C.byref(ls)) == 0 and gs.value == 7
    gs, ls = C.c_size_t(0), C.c_size_t(64)
    assert lib.GpuKernel_sched(C.byref(k), 1 << 28, C.byref(gs), C.byref(ls)) == 0
    assert ls.value == 64 and gs.value == 256 * 16
    # a launch that cannot run is an error code, not a fault
    big = C.c_size_t(4096)
    one = C.c_size_t(1)
    assert lib.GpuKernel_call(C.byref(k), 1, C.byref(one), C.byref(big), 0, None) == _lib.GA_VALUE_ERROR
    assert lib.GpuKernel_call(C.byref(k), 4, C.byref(one), C.byref(one), 0, None) == _lib.GA_VALUE_ERROR
    lib.GpuKernel_clear(C.byref(k))
    # compile errors come back with a log the caller owns
    bad = (C.c_char_p * 1)(b'#include "cluda.h"\nKERNEL void k(int *p) { p[0] = nope; }')
    log = C.c_char_p()
    t1 = (C.c_int * 1)(_lib.GA_BUFFER)
    assert lib.GpuKernel_init(C.byref(k), ctx.ctx, 1, bad, None, b"k", 1, t1, 0, C.byref(log)) \
        == _lib.GA_IMPL_ERROR
    assert b"nope" in log.value
    assert not k.k and not k.args
    # kernels marked as CUDA/OpenCL text are refused
    assert lib.GpuKernel_init(C.byref(k), ctx.ctx, 1, strs, None, b"axpy", 4, types,
                              _lib.GA_USE_CUDA, None) == _lib.GA_DEVSUP_ERROR


def check_meta(g, n):
    assert g.shape == n.shape and g.dtype == n.dtype
    if n.size > 0:   # NumPy zeroes the strides of empty arrays; the C rule does not
        assert g.strides == n.strides
        assert g.flags.c_contiguous == n.flags.c_contiguous
        assert g.flags.f_contiguous == n.flags.f_contiguous


def test_empty_zeros_orders_and_errors(ctx):
    for shape in [(), (5,), (3, 4), (2, 3, 4), (0, 3), (1, 1)]:
        for order in "CF":
            g = gpuarray.zeros(shape, "float32", order, context=ctx)
            n = np.zeros(shape, np.float32, order=order)
            check_meta(g, n)
            assert np.array_equal(np.asarray(g), n)
            assert g.flags.aligned and g.flags.writeable
    a = _lib.GpuArrayStruct()
    dims = (C.c_size_t * 2)(1 << 40, 1 << 40)
    assert lib.GpuArray_empty(C.byref(a), ctx.ctx, _lib.GA_FLOAT, 2, dims, 0) == _lib.GA_XLARGE_ERROR
    assert lib.GpuArray_empty(C.byref(a), ctx.ctx, _lib.GA_SIZE, 1, dims, 0) == _lib.GA_VALUE_ERROR
    assert lib.GpuArray_empty(C.byref(a), ctx.ctx, _lib.GA_FLOAT, 1, dims, 5) == _lib.GA_VALUE_ERROR


def test_transpose_all_permutations(ctx):       # test_gpu_ndarray.py:526-579
    rng = np.random.default_rng(2)
    for shape in [(4,), (3, 5), (2, 3, 4), (2, 3, 1, 4)]:
        for order in "cf":
            for sliced in (1, 2, -2, -1):
                n, g = gen_gpuarray(shape, "float32", sliced=sliced, order=order, ctx=ctx, rng=rng)
                check_meta(g.T, n.T)
                assert np.array_equal(np.asarray(g.T), n.T)
                for perm in itertools.permutations(range(len(shape))):
                    check_meta(g.transpose(perm), n.transpose(perm))
                    assert np.array_equal(np.asarray(g.transpose(perm)), n.transpose(perm))
    with pytest.raises(ValueError):
        g.transpose((0, 0, 1, 2))


def test_indexing_matches_numpy(ctx):
    rng = np.random.default_rng(3)
    n, g = gen_gpuarray((6, 7, 8), "int32", ctx=ctx, rng=rng, high=100)
    keys = [np.s_[1], np.s_[1:4], np.s_[::2], np.s_[::-1], np.s_[5:1:-2], np.s_[..., 3],
            np.s_[2, 3, 4], np.s_[:, 2:5, ::3], np.s_[-1, ..., -2], np.s_[3:3], np.s_[:, ::-1, 1:],
            np.s_[4:1], np.s_[1:-1, -3:, ::-3]]
    for k in keys:
        check_meta(g[k], n[k])
        assert np.array_equal(np.asarray(g[k]), n[k])
    assert g[::-1].offset == 5 * n.strides[0]
    with pytest.raises(IndexError):
        g[6]
    # the raw entry point validates ranges (src/gpuarray_array.c:264-300)
    r = _lib.GpuArrayStruct()
    st = (_lib.c_ssize_t * 3)(0, 0, 9)
    sp = (_lib.c_ssize_t * 3)(6, 7, 8)
    se = (_lib.c_ssize_t * 3)(1, 1, 1)
    assert lib.GpuArray_index(C.byref(r), g._ptr(), st, sp, se) == _lib.GA_VALUE_ERROR
    assert lib.GpuArray_index(C.byref(r), g._ptr(), None, sp, se) == _lib.GA_VALUE_ERROR


def test_reshape_matches_numpy(ctx):            # test_gpu_ndarray.py:460-497
    rng = np.random.default_rng(4)
    cases = [((6,), (2, 3)), ((2, 3), (6,)), ((2, 3, 4), (6, 4)), ((2, 3, 4), (2, 12)),
             ((2, 3, 4), (4, 3, 2)), ((12,), (1, 12, 1)), ((1, 6, 1), (6,)), ((4, 6), (2, 2, 3, 2)),
             ((2, 3, 4), (-1,)), ((0, 3), (3, 0))]
    for shape, new in cases:
        for order in "cf":
            n, g = gen_gpuarray(shape, "float32", order=order, ctx=ctx, rng=rng)
            for ro in "CF":
                rn, rg = n.reshape(new, order=ro), g.reshape(new, order=ro)
                assert rg.shape == rn.shape
                assert np.array_equal(np.asarray(rg), rn)
    # a sliced array reshapes without a copy exactly when NumPy can
    n, g = gen_gpuarray((4, 6), "float32", sliced=2, ctx=ctx, rng=rng)
    rg = g.reshape((4, 2, 3))
    rn = n.reshape((4, 2, 3))
    assert rg.strides == rn.strides and np.array_equal(np.asarray(rg), rn)
    r = _lib.GpuArrayStruct()
    dims = (C.c_size_t * 1)(24)
    assert lib.GpuArray_reshape(C.byref(r), g._ptr(), 1, dims, 0, 1) == _lib.GA_COPY_ERROR
    assert lib.GpuArray_reshape(C.byref(r), g._ptr(), 1, dims, 0, 0) == 0
    lib.GpuArray_clear(C.byref(r))
    dims = (C.c_size_t * 1)(25)
    assert lib.GpuArray_reshape(C.byref(r), g._ptr(), 1, dims, 0, 0) == _lib.GA_INVALID_ERROR


def test_copy_move_astype_setitem(ctx):
    rng = np.random.default_rng(5)
    for shape in [(7,), (5, 6), (3, 4, 5)]:
        for sliced, oi in [(1, False), (2, True), (-1, False)]:
            n, g = gen_gpuarray(shape, "float32", sliced=sliced, offseted_inner=oi, ctx=ctx, rng=rng)
            for order in "CF":
                c = g.copy(order)
                assert (c.flags.c_contiguous if order == "C" else c.flags.f_contiguous)
                assert np.array_equal(np.asarray(c), n)
            for dt in ("float64", "int32", "float16", "uint8", "int64"):
                assert np.array_equal(np.asarray(g.astype(dt)), n.astype(dt)), dt
    # views alias, copies do not (test_gpu_ndarray.py:410-457)
    n, g = gen_gpuarray((4, 5), "float32", ctx=ctx, rng=rng)
    v, c = g.view(), g.copy()
    assert lib.GpuArray_share(v._ptr(), g._ptr()) == 1 and lib.GpuArray_share(c._ptr(), g._ptr()) == 0
    g[1:3, ::2] = np.float32(7)
    n[1:3, ::2] = 7
    assert np.array_equal(np.asarray(v), n) and not np.array_equal(np.asarray(c), n)
    row = gpuarray.array(np.arange(5, dtype=np.float32), context=ctx)
    g[...] = row                                   # broadcast along the first axis
    assert np.array_equal(np.asarray(g), np.tile(np.arange(5, dtype=np.float32), (4, 1)))
    # one-segment rules (src/gpuarray_array.c:879-900)
    buf = np.zeros(10, np.float32)
    assert lib.GpuArray_read(buf.ctypes.data, 40, g[:, ::2]._ptr()) == _lib.GA_UNSUPPORTED_ERROR
    assert lib.GpuArray_memset(g[:, ::2]._ptr(), 0) == _lib.GA_UNSUPPORTED_ERROR
    # shape mismatch in move (src/gpuarray_array.c:859-868)
    assert lib.GpuArray_move(g._ptr(), row._ptr()) == _lib.GA_VALUE_ERROR


def test_split_and_concatenate(ctx):
    rng = np.random.default_rng(6)
    n, g = gen_gpuarray((6, 5), "int32", ctx=ctx, rng=rng, high=50)
    outs = [_lib.GpuArrayStruct() for _ in range(3)]
    ptrs = (_lib.PA * 3)(*[C.pointer(o) for o in outs])
    cuts = (C.c_size_t * 2)(2, 3)
    assert lib.GpuArray_split(ptrs, g._ptr(), 2, cuts, 0) == 0
    want = np.split(n, [2, 3], axis=0)
    for o, w in zip(outs, want):
        assert tuple(o.dimensions[i] for i in range(2)) == w.shape
    r = _lib.GpuArrayStruct()
    ins = (_lib.PA * 3)(*[C.pointer(o) for o in outs])
    assert lib.GpuArray_concatenate(C.byref(r), ins, 3, 0, _lib.GA_LONG) == 0
    back = np.empty((6, 5), np.int64)
    assert lib.GpuArray_read(back.ctypes.data, back.nbytes, C.byref(r)) == 0
    assert np.array_equal(back, n.astype(np.int64))
    lib.GpuArray_clear(C.byref(r))
    for o in outs:
        lib.GpuArray_clear(C.byref(o))


def test_memory_cache_reuses_and_never_overlaps(ctx):
    # freed blocks come back without a trip to the driver, live blocks never
    # overlap, and their contents survive neighbours being split and merged
    rng = np.random.default_rng(12)
    ptr_of = _lib.extension("hip_get_ptr", C.c_void_p, [C.c_void_p])
    size_of = _lib.extension("hip_get_sz", C.c_size_t, [C.c_void_p])
    d = lib.gpudata_alloc(ctx.ctx, 1 << 20, None, 0, None)
    p0 = ptr_of(d)
    lib.gpudata_release(d)
    d = lib.gpudata_alloc(ctx.ctx, 1 << 20, None, 0, None)
    assert ptr_of(d) == p0                       # best fit finds the block just freed
    assert size_of(d) == 1 << 20 and ptr_of(d) % 256 == 0
    lib.gpudata_release(d)
    live = {}
    for step in range(400):
        if live and rng.random() < 0.45:
            key = list(live)[int(rng.integers(len(live)))]
            buf, pattern = live.pop(key)
            back = np.empty_like(pattern)
            assert lib.gpudata_read(back.ctypes.data, buf, 0, back.nbytes) == 0
            assert np.array_equal(back, pattern)
            lib.gpudata_release(buf)
        else:
            n = int(rng.choice([1, 7, 255, 256, 257, 4096, 70000, 1 << 20, (1 << 22) + 5]))
            buf = lib.gpudata_alloc(ctx.ctx, n, None, 0, None)
            assert buf and ptr_of(buf) % 256 == 0
            pattern = rng.integers(0, 256, n, dtype=np.uint8)
            assert lib.gpudata_write(buf, 0, pattern.ctypes.data, n) == 0
            live[step] = (buf, pattern)
        spans = sorted((ptr_of(b), ptr_of(b) + size_of(b)) for b, _ in live.values())
        assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:]))
    for buf, pattern in live.values():
        back = np.empty_like(pattern)
        assert lib.gpudata_read(back.ctypes.data, buf, 0, back.nbytes) == 0
        assert np.array_equal(back, pattern)
        lib.gpudata_release(buf)


def test_memory_cache_limits():
    # reference rules: max bounds what is taken from the device and the error
    # is "Maximum cache size reached" (src/gpuarray_buffer_cuda.c:649-653);
    # max == 0 turns the cache off; initial must not exceed max
    c = ga.GpuContext("hip", 0, initial_cache_size=1 << 20, max_cache_size=16 << 20)
    e = C.c_int(0)
    bufs = []
    while True:
        b = lib.gpudata_alloc(c.ctx, 4 << 20, None, 0, C.byref(e))
        if not b:
            break
        bufs.append(b)
        assert len(bufs) <= 4                    # 16 MiB cap, 4 MiB each
    assert len(bufs) >= 3                        # the context's own 8-byte buffer sits in one segment
    assert e.value == _lib.GA_VALUE_ERROR and "Maximum cache size reached" in c.error()
    lib.gpudata_release(bufs.pop())
    again = lib.gpudata_alloc(c.ctx, 3 << 20, None, 0, None)      # fits in what was freed
    assert again
    for b in bufs + [again]:
        lib.gpudata_release(b)
    nocache = ga.GpuContext("hip", 0, max_cache_size=0)
    a = gpuarray.array(np.arange(1000, dtype=np.float32), context=nocache)
    assert np.array_equal(np.asarray(a), np.arange(1000, dtype=np.float32))
    with pytest.raises(ga.GpuArrayException):
        ga.GpuContext("hip", 0, initial_cache_size=2, max_cache_size=1)


def test_disk_kernel_cache(tmp_path):
    import glob, os, time
    d = str(tmp_path / "kcache")
    expr = "c = a*b + 0.25f /* disk cache test */"
    spec = [ga.arg("a", "float32", read=True), ga.arg("b", "float32", read=True),
            ga.arg("c", "float32", write=True)]

    def run(c):
        t0 = time.perf_counter()
        k = ga.GpuElemwise(c, expr, spec)
        dt = time.perf_counter() - t0
        a = gpuarray.array(np.arange(1000, dtype=np.float32), context=c)
        out = gpuarray.empty((1000,), "float32", context=c)
        k(a, a, out)
        want = np.arange(1000, dtype=np.float32) ** 2 + np.float32(0.25)
        assert np.array_equal(np.asarray(out), want)
        return dt

    cold = run(ga.GpuContext("hip", 0, kernel_cache_path=d))
    files = [f for f in glob.glob(os.path.join(d, "*", "*")) if ".tmp." not in f]
    assert len(files) == 1
    # entry layout: 8-byte big-endian key and value lengths, key, value, checksum
    raw = open(files[0], "rb").read()
    kl, vl = int.from_bytes(raw[:8], "big"), int.from_bytes(raw[8:16], "big")
    assert len(raw) == 16 + kl + vl + 8 and expr.encode() in raw[16:16 + kl]
    assert raw[16 + kl:16 + kl + 4] == b"\x7fELF"
    warm = run(ga.GpuContext("hip", 0, kernel_cache_path=d))     # new context: module comes from disk
    assert warm < cold / 3, (cold, warm)
    # a damaged entry fails its checksum: it is recompiled and replaced, and
    # the damaged code never reaches the loader
    with open(files[0], "r+b") as f:
        f.seek(16 + kl + 64)
        f.write(b"\0" * 256)
    run(ga.GpuContext("hip", 0, kernel_cache_path=d))
    assert open(files[0], "rb").read()[16 + kl:] == raw[16 + kl:]


class _TwoQ(object):
    """The reference's policy restated from src/cache/twoq.c:232-316, to
    predict what the module cache holds."""

    def __init__(self, hot, warm, cold, elasticity):
        self.sizes = (hot, warm, cold, elasticity)
        self.hot, self.warm, self.cold = [], [], []

    def add(self, k):
        hot, _, cold, el = self.sizes
        self.hot.append(k)
        while len(self.hot) > hot:
            self.cold.append(self.hot.pop(0))
        if len(self.cold) > cold + el:
            while len(self.cold) > cold:
                self.cold.pop(0)

    def get(self, k):
        if k in self.hot:
            self.hot.remove(k); self.hot.append(k)
        elif k in self.warm:
            self.warm.remove(k); self.warm.append(k)
        elif k in self.cold:
            self.cold.remove(k); self.warm.append(k)
            if len(self.warm) > self.sizes[1]:
                self.cold.append(self.warm.pop(0))
        else:
            return False
        return True

    def cached(self):
        return set(self.hot) | set(self.warm) | set(self.cold)


def test_module_cache_follows_the_2q_policy(monkeypatch, tmp_path):
    monkeypatch.setenv("GPUARRAY_MODULE_CACHE", "2,2,1,1")
    c = ga.GpuContext("hip", 0, kernel_cache_path=str(tmp_path / "k"))
    stats_fn = _lib.extension("hip_module_cache_stats", C.c_int, [C.c_void_p, C.POINTER(C.c_size_t)])

    def stats():
        out = (C.c_size_t * 4)()
        assert stats_fn(c.ctx, out) == 0
        return list(out)

    base = stats()                       # whatever the context itself has built
    assert base[3] == sum(base[:3])
    model = _TwoQ(2, 2, 1, 1)
    spec = [ga.arg("a", "float32", read=True), ga.arg("c", "float32", write=True)]
    a = gpuarray.array(np.arange(100, dtype=np.float32), context=c)
    out = gpuarray.empty((100,), "float32", context=c)
    held = {}

    def make(i):
        k = ga.GpuElemwise(c, "c = a + %d.0f /* 2q test */" % i, spec)
        if not model.get(i):
            model.add(i)
        return k

    def check_counts(nheld_uncached):
        s = stats()
        assert s[:3] == [len(model.hot), len(model.warm), len(model.cold)], (s, model.__dict__)
        assert s[3] == len(model.cached()) + nheld_uncached

    assert base[:3] == [0, 0, 0]
    for i in range(6):
        held[i] = make(i)
        uncached = [j for j in held if j not in model.cached()]
        check_counts(len(uncached))
    # entries that fell out stay loaded while an operator uses them, and run
    uncached = [j for j in held if j not in model.cached()]
    assert uncached, "the sizes above must have evicted something"
    for j in held:
        held[j](a, out)
        assert np.array_equal(np.asarray(out), np.arange(100, dtype=np.float32) + j)
    # dropping the operator of an evicted module unloads it
    del held[uncached[0]]
    check_counts(len(uncached) - 1)
    # a hit in cold promotes to warm; making the same operator again compiles nothing new
    cold_key = model.cold[0]
    again = make(cold_key)
    check_counts(len(uncached) - 1)
    again(a, out)
    assert np.array_equal(np.asarray(out), np.arange(100, dtype=np.float32) + cold_key)
