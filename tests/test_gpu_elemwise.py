"""GpuElemwise on the device, through the C ABI, against
  - the literal results of the reference's tests (tests/check_elemwise.c:39-880),
  - the CPU checker (oracle/) on seeded random layouts, bit for bit,
  - NumPy at the benchmark's shapes.
Float expressions are compiled without contraction, so a*b+c is two roundings
and results are bit-identical to the checker and to NumPy."""
import ctypes as C

import numpy as np
import pytest

import libgpuarray_amd as ga
from libgpuarray_amd import _lib, gpuarray
from support import to_gpu_view, read_root, root_of, arg

pytestmark = pytest.mark.gpu
lib = _lib.lib
F16 = np.array([0x0000, 0x3c00, 0x4000, 0x4200, 0x4400, 0x4500, 0x4600, 0x4700, 0x4800, 0x4880],
               dtype=np.uint16).view(np.float16)
@pytest.mark.parametrize("dts", [("uint8", "uint8", "uint8"), ("float16", "float16", "float16"),
                                 ("float64", "float64", "float64"), ("float32", "float16", "float32"),
                                 ("int16", "int64", "int32")])
def test_views_cut_the_same_way_keep_vector_access(ctx, dts):
    """Arrays that start the same number of elements off a chunk boundary
    (x[k:] of aligned arrays) take vector access after a short head; other
    combinations fall back to element access.  Either way every element is
    computed once and nothing outside the views is written."""
    rng = np.random.default_rng(77)
    ta, tb, tc = dts
    ge = ga.GpuElemwise(ctx, "c = a + b", [arg("a", ta, read=True), arg("b", tb, read=True),
                                           arg("c", tc, write=True)], convert_f16=True)
    pad = 40
    for n in (1, 2, 5, 15, 16, 17, 31, 33, 1000, 4099, 100003):
        a = rng.integers(0, 50, n + pad).astype(ta)
        b = rng.integers(0, 50, n + pad).astype(tb)
        for oa, ob, oc in ((1, 1, 1), (3, 3, 3), (15, 15, 15), (17, 17, 17), (1, 17, 33), (2, 1, 0),
                           (0, 0, 5), (4, 4, 4), (8, 0, 0)):
            ga_v, gb_v = to_gpu_view(a[oa:oa + n], ctx)[0], to_gpu_view(b[ob:ob + n], ctx)[0]
            gc = gpuarray.zeros((n + pad,), tc, context=ctx)
            ge(ga_v, gb_v, gc[oc:oc + n])
            got = np.asarray(gc)
            want = (a[oa:oa + n].astype(np.float64) + b[ob:ob + n].astype(np.float64)).astype(tc)
            assert np.array_equal(got[oc:oc + n], want), (n, oa, ob, oc)
            assert not got[:oc].any() and not got[oc + n:].any(), (n, oa, ob, oc)


BCAST, NOCOLLAPSE, PAD = _lib.GE_BROADCAST, _lib.GE_NOCOLLAPSE, _lib.GE_PADSHAPE


def raw_call(ge, arrays_and_scalars, flags):
    """GpuElemwise_call with explicit flags; returns the error code."""
    keep = []
    ptrs = (C.c_void_p * len(arrays_and_scalars))()
    for i, v in enumerate(arrays_and_scalars):
        if isinstance(v, ga.GpuArray):
            ptrs[i] = C.addressof(v.ga)
        else:
            keep.append(np.ascontiguousarray(v))
            ptrs[i] = keep[-1].ctypes.data
    return lib.GpuElemwise_call(ge.ge, ptrs, flags)


def dev(values, shape, order="C", dtype=np.uint32, ctx=None):
    """Device array whose MEMORY holds `values` in order (GpuArray_write into a
    C- or F-ordered array, as the reference tests do)."""
    g = gpuarray.empty(shape, dtype, order, context=ctx)
    flat = np.array(values, dtype=dtype)
    assert lib.GpuArray_write(g._ptr(), flat.ctypes.data, flat.nbytes) == 0
    return g


def mem(g, count, dtype=np.uint32):
    out = np.zeros(count, dtype)
    assert lib.GpuArray_read(out.ctypes.data, out.nbytes, g._ptr()) == 0
    return out


def add_u32(ctx, nd=0, flags=0, expr="c = a + b", dt="uint32"):
    return ga.GpuElemwise(ctx, expr, [arg("a", dt, read=True), arg("b", dt, read=True),
                                      arg("c", dt, write=True)], nd=nd,
                          convert_f16=bool(flags & _lib.GE_CONVERT_F16))


# ---- the reference's scenarios ---------------------------------------------------

def test_contig_simple(ctx):
    a, b = dev([1, 2, 3], (3,), ctx=ctx), dev([4, 5, 6], (3,), ctx=ctx)
    c = gpuarray.empty((3,), "uint32", context=ctx)
    assert raw_call(add_u32(ctx, 1), [a, b, c], NOCOLLAPSE) == 0
    assert mem(c, 3).tolist() == [5, 7, 9]


def test_contig_and_basic_f16(ctx):
    ge = add_u32(ctx, 1, _lib.GE_CONVERT_F16, dt="float16")
    a = dev(F16[[1, 2, 3]], (3,), dtype=np.float16, ctx=ctx)
    b = dev(F16[[4, 5, 6]], (3,), dtype=np.float16, ctx=ctx)
    c = gpuarray.empty((3,), "float16", context=ctx)
    assert raw_call(ge, [a, b, c], NOCOLLAPSE) == 0
    assert np.array_equal(mem(c, 3, np.float16).view(np.uint16), F16[[5, 7, 9]].view(np.uint16))
    a = dev(F16[[1, 2, 3]], (1, 3), dtype=np.float16, ctx=ctx)
    b = dev(F16[[4, 5, 6]], (1, 3), "F", dtype=np.float16, ctx=ctx)
    c = gpuarray.empty((1, 3), "float16", context=ctx)
    assert raw_call(ge, [a, b, c], NOCOLLAPSE) == 0
    assert np.array_equal(mem(c, 3, np.float16).view(np.uint16), F16[[5, 7, 9]].view(np.uint16))


def test_zero_sized(ctx):
    ge = add_u32(ctx, 1)
    z = [gpuarray.empty((0,), "uint32", context=ctx) for _ in range(3)]
    assert raw_call(ge, z, NOCOLLAPSE) == 0
    a = gpuarray.empty((0, 3), "uint32", "C", context=ctx)
    b = gpuarray.empty((0, 3), "uint32", "F", context=ctx)
    c = gpuarray.empty((0, 3), "uint32", "C", context=ctx)
    assert raw_call(ge, [a, b, c], 0) == 0


def test_basic_simple_and_offset(ctx):
    ge = add_u32(ctx, 2)
    a = dev([1, 2, 3], (1, 3), ctx=ctx)
    b = dev([4, 5, 6], (1, 3), "F", ctx=ctx)
    c = gpuarray.empty((1, 3), "uint32", context=ctx)
    assert raw_call(ge, [a, b, c], NOCOLLAPSE) == 0
    assert mem(c, 3).tolist() == [5, 7, 9]
    # "simulate indexing": offset 12 bytes into a 6-element row (check_elemwise.c:339-345)
    a = gpuarray.empty((1, 6), "uint32", context=ctx)
    a.ga.offset = 12
    a.ga.dimensions[1] = 3
    lib.GpuArray_fix_flags(a._ptr())
    data = np.array([1, 2, 3], np.uint32)
    assert lib.GpuArray_write(a._ptr(), data.ctypes.data, 12) == 0
    c = gpuarray.empty((1, 3), "uint32", context=ctx)
    assert raw_call(ge, [a, b, c], NOCOLLAPSE) == 0
    assert mem(c, 3).tolist() == [5, 7, 9]
    a.ga.offset = 0   # restore before the array is released


def test_basic_scalar(ctx):
    ge = ga.GpuElemwise(ctx, "c = a + x * b",
                        [arg("a", "uint32", read=True), arg("x", "uint32", scalar=True),
                         arg("b", "uint32", read=True), arg("c", "uint32", write=True)], nd=2)
    a = dev([1, 2, 3], (1, 3), ctx=ctx)
    b = dev([4, 5], (2, 1), "F", ctx=ctx)
    c = gpuarray.empty((2, 3), "uint32", context=ctx)
    assert raw_call(ge, [a, np.uint32(2), b, c], BCAST) == 0
    assert mem(c, 6).tolist() == [9, 10, 11, 11, 12, 13]


def test_basic_scalar_dtype(ctx):
    ge = ga.GpuElemwise(ctx, "y = a * x + y",
                        [arg("a", "float32", scalar=True), arg("x", "int32", read=True),
                         arg("y", "float32", read=True, write=True)], nd=2)
    x = dev([0, 1, 2, 3], (2, 2), dtype=np.int32, ctx=ctx)
    y = dev([2.0, 2.0, 2.0, 2.0], (2, 2), "F", dtype=np.float32, ctx=ctx)
    assert raw_call(ge, [np.float32(1.1), x, y], 0) == 0
    assert np.array_equal(mem(y, 4, np.float32), np.array([2.0, 4.2, 3.1, 5.3], np.float32))


def test_basic_remove1_and_collapse(ctx):
    ge = add_u32(ctx, 0)
    a = dev([1, 2, 3, 4, 5, 6], (1, 3, 2, 1), ctx=ctx)
    b = dev([7, 8, 9, 10, 11, 12], (1, 3, 2, 1), "F", ctx=ctx)
    c = gpuarray.empty((1, 3, 2, 1), "uint32", context=ctx)
    assert raw_call(ge, [a, b, c], 0) == 0
    assert mem(c, 6).tolist() == [8, 12, 11, 15, 14, 18]
    a = dev([1, 2, 3, 4, 5, 6], (2, 3), ctx=ctx)
    b = dev([7, 8, 9, 10, 11, 12], (2, 3), ctx=ctx)
    c = gpuarray.empty((2, 3), "uint32", context=ctx)
    assert raw_call(ge, [a, b, c], 0) == 0
    assert mem(c, 6).tolist() == [8, 10, 12, 14, 16, 18]


def test_basic_broadcast_and_padshape(ctx):
    ge = add_u32(ctx, 2)
    a = dev([1, 2, 3], (1, 3), ctx=ctx)
    b = dev([4, 5], (2, 1), "F", ctx=ctx)
    c = gpuarray.empty((2, 3), "uint32", context=ctx)
    assert raw_call(ge, [a, b, c], NOCOLLAPSE) == _lib.GA_VALUE_ERROR
    assert "Mismatched dimension" in ctx.error()
    assert raw_call(ge, [a, b, c], NOCOLLAPSE | BCAST) == 0
    assert mem(c, 6).tolist() == [5, 6, 7, 6, 7, 8]
    a1 = dev([1, 2, 3], (3,), ctx=ctx)
    c = gpuarray.empty((2, 3), "uint32", context=ctx)
    assert raw_call(ge, [a1, b, c], NOCOLLAPSE) == _lib.GA_VALUE_ERROR
    assert raw_call(ge, [a1, b, c], NOCOLLAPSE | BCAST | PAD) == 0
    assert mem(c, 6).tolist() == [5, 6, 7, 6, 7, 8]
    # outputs never broadcast (src/gpuarray_elemwise.c:348-354)
    c1 = gpuarray.empty((1, 3), "uint32", context=ctx)
    big = gpuarray.empty((2, 3), "uint32", context=ctx)
    assert raw_call(ge, [big, a, c1], BCAST) == _lib.GA_VALUE_ERROR


def test_basic_neg_strides(ctx):
    ge = add_u32(ctx, 1)
    a = dev([1, 2, 3, 4, 5, 6], (6,), ctx=ctx)
    b = dev([7, 8, 9, 10, 11, 12], (6,), ctx=ctx)
    st, sp, se = (_lib.c_ssize_t * 1)(5), (_lib.c_ssize_t * 1)(-1), (_lib.c_ssize_t * 1)(-1)
    assert lib.GpuArray_index_inplace(b._ptr(), st, sp, se) == 0
    c = gpuarray.empty((6,), "uint32", context=ctx)
    assert raw_call(ge, [a, b, c], 0) == 0
    assert mem(c, 6).tolist() == [13] * 6


def test_new_reports_compile_errors(ctx):
    with pytest.raises(ga.GpuArrayException) as e:
        add_u32(ctx, expr="c = a + not_a_name")
    assert "not_a_name" in str(e.value)
    # no output array at all (src/gpuarray_elemwise.c:301-302)
    ge = ga.GpuElemwise(ctx, "a + b", [arg("a", "uint32", read=True), arg("b", "uint32", read=True)])
    a = dev([1, 2, 3], (1, 3), ctx=ctx)
    b = dev([4, 5], (2, 1), "F", ctx=ctx)
    assert raw_call(ge, [a, b], BCAST) == _lib.GA_VALUE_ERROR


# ---- parity with the CPU checker on random layouts ---------------------------------

def random_view(rng, shape, dtype):
    """A view of `shape` with random memory order, steps, reversals and offset."""
    nd = len(shape)
    perm = rng.permutation(nd)
    steps = [int(rng.choice([1, 1, 2, 3])) for _ in range(nd)]
    pad = [int(rng.integers(0, 3)) for _ in range(nd)]
    big = [shape[perm[i]] * steps[i] + pad[i] for i in range(nd)]
    base = rng.normal(0, 1, big).astype(dtype)
    idx = tuple(slice(pad[i], pad[i] + shape[perm[i]] * steps[i], steps[i]) for i in range(nd))
    v = base[idx].transpose(np.argsort(perm))
    for ax in range(nd):
        if rng.random() < 0.25:
            v = np.flip(v, ax)
    assert v.shape == tuple(shape)
    return v


@pytest.mark.parametrize("seed", range(6))
def test_random_layouts_bit_exact_vs_checker(seed, ctx, oracle):
    rng = np.random.default_rng(100 + seed)
    ge = ga.GpuElemwise(ctx, "out = a + b*c",
                        [arg("a", "float32", read=True), arg("b", "float32", read=True),
                         arg("c", "float32", read=True), arg("out", "float32", write=True)])
    for _ in range(12):
        nd = int(rng.integers(1, 5))
        shape = [int(x) for x in rng.integers(1, [40, 20, 9, 5][:nd])]
        rng.shuffle(shape)
        ins = []
        for _k in range(3):
            shp = [d if rng.random() < 0.7 else 1 for d in shape]
            ins.append(random_view(rng, shp, np.float32))
        out = random_view(rng, shape, np.float32)
        g_in = [to_gpu_view(v, ctx)[0] for v in ins]
        g_out, g_root = to_gpu_view(out, ctx)
        # the checker runs on a host copy of the output's whole buffer, viewed
        # with the same offset and strides
        want_root = np.ascontiguousarray(root_of(out).reshape(-1, order="A")).copy()
        off = out.__array_interface__["data"][0] - root_of(out).__array_interface__["data"][0]
        host_out = np.ndarray(shape=out.shape, dtype=np.float32, buffer=want_root.data,
                              offset=off, strides=out.strides)
        assert oracle.elemwise(oracle.A_PLUS_BC_F32, ins + [host_out], [0, 0, 0, 1],
                               flags=BCAST) == 0
        assert raw_call(ge, g_in + [g_out], BCAST) == 0
        got_root = np.asarray(g_root)[:want_root.nbytes].view(np.float32)
        assert np.array_equal(got_root, want_root), (shape, [v.strides for v in ins], out.strides)
        assert np.array_equal(host_out, np.broadcast_to(ins[0] + ins[1] * ins[2], out.shape))


def test_dtype_matrix_copy_cast_vs_numpy(ctx):
    rng = np.random.default_rng(7)
    dts = ["bool", "int8", "uint8", "int16", "uint16", "int32", "uint32", "int64", "uint64",
           "float16", "float32", "float64"]
    src = rng.uniform(0, 100, (33, 17))
    for sd in dts:
        n = src.astype(sd)
        g = gpuarray.array(n, context=ctx)
        for dd in dts:
            got = np.asarray(g.T.astype(dd))       # transposed source -> tiled kernel
            assert np.array_equal(got, n.T.astype(dd)), (sd, dd)
            got = np.asarray(g.astype(dd))         # flat kernel
            assert np.array_equal(got, n.astype(dd)), (sd, dd)


def test_cast_to_bool_stores_the_truth_value_not_the_low_byte(ctx):
    """A deliberate difference from the reference.  Its GA_BOOL is an unsigned
    char (`ga_bool`, src/cluda_opencl.h:26), so a casting copy `dst = src` into
    a bool array converts to unsigned char: 62.5 becomes 62, 256 becomes 0, 257
    becomes 1.  Here the copy stores `src != 0`, NumPy's astype(bool): 1, 1, 1.
    Both results are spelled out so that the difference stays visible."""
    for dtype, values in (("float32", [0.0, 1.0, 62.5, -3.0, 0.25]),
                          ("int32", [0, 1, 255, 256, 257, 512, -1]),
                          ("int64", [0, 1 << 8, 1 << 32, 3])):
        host = np.array(values, dtype=dtype)
        got = np.asarray(gpuarray.array(host, context=ctx).astype("bool")).view(np.uint8)
        with np.errstate(invalid="ignore"):
            reference_would_store = host.astype(np.int64).astype(np.uint8)   # C's conversion to unsigned char
        here = (host != 0).astype(np.uint8)
        assert np.array_equal(got, here), (dtype, got)
        if dtype == "int32":
            assert reference_would_store.tolist() == [0, 1, 255, 0, 1, 0, 255]
            assert here.tolist() == [0, 1, 1, 1, 1, 1, 1]
        assert np.array_equal(got != 0, host.astype(bool))


def test_all_fortran_inputs_take_the_flat_path(ctx):
    rng = np.random.default_rng(8)
    a = np.asfortranarray(rng.normal(size=(130, 70)).astype(np.float32))
    b = np.asfortranarray(rng.normal(size=(130, 70)).astype(np.float32))
    ga_, gb = gpuarray.array(a, order="F", context=ctx), gpuarray.array(b, order="F", context=ctx)
    gc = gpuarray.empty((130, 70), "float32", "F", context=ctx)
    ge = ga.GpuElemwise(ctx, "c = a*b + 0.5f", [arg("a", "float32", read=True),
                                                arg("b", "float32", read=True),
                                                arg("c", "float32", write=True)])
    ge(ga_, gb, gc)
    assert np.array_equal(np.asarray(gc), a * b + np.float32(0.5))
    # C output, F inputs: general path, dims sorted by the output's strides
    gc2 = gpuarray.empty((130, 70), "float32", "C", context=ctx)
    ge(ga_, gb, gc2)
    assert np.array_equal(np.asarray(gc2), a * b + np.float32(0.5))


@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 63, 64, 65, 255, 256, 257, 1023, 4095, 4096, 4097,
                               65535, 1 << 20, (1 << 20) + 1, (1 << 22) + 3,
                               # grids of one to four chip fills: two / four adjacent chunks per lane
                               (1 << 21) + 1021, (3 << 20) + 1, (1 << 22) - 5, (3 << 21) + 3, (1 << 23) - 1,
                               (1 << 23) + 1])
def test_flat_sizes_tails_and_misalignment(n, ctx, oracle):
    rng = np.random.default_rng(n)
    a = rng.uniform(-1, 1, n + 3).astype(np.float32)
    b = rng.uniform(-1, 1, n + 3).astype(np.float32)
    ge = ga.GpuElemwise(ctx, "c = a*b + 0.5f", [arg("a", "float32", read=True),
                                                arg("b", "float32", read=True),
                                                arg("c", "float32", write=True)])
    want = np.empty(n, np.float32)
    for off in (0, 1, 3):          # element offsets: 0 keeps 16-byte alignment, 1 and 3 break it
        av, bv = a[off:off + n], b[off:off + n]
        oracle.elemwise_contig_muladd(np.ascontiguousarray(av), np.ascontiguousarray(bv), want)
        gav, gbv = to_gpu_view(av, ctx)[0], to_gpu_view(bv, ctx)[0]
        gc = gpuarray.zeros((n + 3,), "float32", context=ctx)
        ge(gav, gbv, gc[off:off + n])
        got = np.asarray(gc)
        assert np.array_equal(got[off:off + n], want)
        assert np.all(got[:off] == 0) and np.all(got[off + n:] == 0)   # nothing outside the view


def test_small_types_vectorised_flat_path(ctx):
    rng = np.random.default_rng(9)
    for dt in ("uint8", "int16", "float16", "float64", "int64"):
        n = 100003
        a = rng.integers(0, 50, n).astype(dt)
        b = rng.integers(0, 50, n).astype(dt)
        ge = ga.GpuElemwise(ctx, "c = a + b", [arg("a", dt, read=True), arg("b", dt, read=True),
                                               arg("c", dt, write=True)], convert_f16=True)
        gc = gpuarray.empty((n,), dt, context=ctx)
        ge(gpuarray.array(a, context=ctx), gpuarray.array(b, context=ctx), gc)
        assert np.array_equal(np.asarray(gc), (a + b).astype(dt)), dt


@pytest.mark.parametrize("n", [(5 << 20) + 7, (1 << 24) + 5])
def test_flat_kernel_with_a_narrow_side_takes_two_chunks_per_lane(ctx, n):
    # bytes to floats, floats to bytes / halves, comparisons to a byte: beyond one
    # fill of the chip these run with two chunks per lane; offsets break the alignment
    rng = np.random.default_rng(n)
    f = rng.uniform(-100, 100, n + 3).astype(np.float32)
    g = rng.uniform(-100, 100, n + 3).astype(np.float32)
    u = rng.integers(0, 256, n + 3).astype(np.uint8)
    cases = [("o = a * 0.5f", [("a", u)], "float32", lambda a: a.astype(np.float32) * np.float32(0.5)),
             ("o = a + b", [("a", u), ("b", u[::-1].copy())], "float32",
              lambda a, b: a.astype(np.float32) + b.astype(np.float32)),
             ("o = a", [("a", f)], "float16", lambda a: a.astype(np.float16)),
             ("o = a", [("a", np.abs(f))], "uint8", lambda a: a.astype(np.uint8)),
             ("o = a > b", [("a", f), ("b", g)], "bool", lambda a, b: a > b),
             ("o = a", [("a", f.astype(np.float64))], "float32", lambda a: a.astype(np.float32))]
    for expr, ins, odt, ref in cases:
        ge = ga.GpuElemwise(ctx, expr, [arg(nm, v.dtype.name, read=True) for nm, v in ins] +
                            [arg("o", odt, write=True)], convert_f16=True)
        for off_in, off_out in ((0, 0), (1, 0), (0, 3), (2, 2)):
            gins = [gpuarray.array(v, context=ctx)[off_in:off_in + n] for _, v in ins]
            go = gpuarray.zeros((n + 3,), odt, context=ctx)
            ge(*gins, go[off_out:off_out + n])
            got = np.asarray(go)
            want = ref(*[v[off_in:off_in + n] for _, v in ins])
            assert np.array_equal(got[off_out:off_out + n], want), (expr, odt, off_in, off_out)
            assert not got[:off_out].any() and not got[off_out + n:].any()


@pytest.mark.parametrize("pairs", ["1", "0"])
def test_eight_byte_elements_in_views_move_two_per_lane(ctx, knobs, pairs):
    # doubles and 64-bit integers in views that are not dense: two elements per
    # lane (inner extents that are a multiple of 2, not of 4, qualify), also
    # next to narrower types; four per lane with the switch off
    knobs(ELEMWISE_PAIRS=pairs, ELEMWISE_PERIODIC=0)
    rng = np.random.default_rng(23)
    for rows, cols, width in ((130, 1002, 500), (67, 2052, 1026), (300, 516, 258), (33, 4100, 2048)):
        a = rng.standard_normal((rows, cols))
        b = rng.standard_normal((rows, cols))
        r = rng.standard_normal((1, width)).astype(np.float32)
        c = rng.standard_normal((rows, 1))
        ga_, gb, gr, gc = (gpuarray.array(v, context=ctx) for v in (a, b, r, c))
        ge = ga.GpuElemwise(ctx, "o = (a * b + r) - c",
                            [arg("a", "float64", read=True), arg("b", "float64", read=True),
                             arg("r", "float32", read=True), arg("c", "float64", read=True),
                             arg("o", "float64", write=True)])
        for lo in (0, 2, 1):                      # 16-byte boundary kept, kept, broken
            out = gpuarray.zeros((rows, cols), "float64", context=ctx)
            ge(ga_[:, lo:lo + width], gb[:, cols - width:], gr, gc, out[:, lo:lo + width], broadcast=True)
            want = np.zeros((rows, cols))
            want[:, lo:lo + width] = (a[:, lo:lo + width] * b[:, cols - width:] + r.astype(np.float64)) - c
            assert np.array_equal(np.asarray(out), want), (rows, cols, width, lo)
        i = rng.integers(-2**40, 2**40, size=(rows, cols))
        gi = gpuarray.array(i, context=ctx)
        gk = ga.GpuElemwise(ctx, "o = a - b", [arg("a", "int64", read=True), arg("b", "int64", read=True),
                                               arg("o", "int64", write=True)])
        out = gpuarray.zeros((rows, width), "int64", context=ctx)
        gk(gi[:, :width], gi[:, cols - width:], out)
        assert np.array_equal(np.asarray(out), i[:, :width] - i[:, cols - width:])


def test_inplace_and_multiple_outputs(ctx):
    rng = np.random.default_rng(10)
    x = rng.normal(size=(257, 33)).astype(np.float32)
    g = gpuarray.array(x, context=ctx)
    s = gpuarray.empty(x.shape, "float32", context=ctx)
    d = gpuarray.empty(x.shape, "float64", "F", context=ctx)
    ge = ga.GpuElemwise(ctx, "s = x * 2.0f; d = (ga_double)x - 1.0; x = -x",
                        [arg("x", "float32", read=True, write=True), arg("s", "float32", write=True),
                         arg("d", "float64", write=True)])
    ge(g, s, d)
    assert np.array_equal(np.asarray(g), -x)
    assert np.array_equal(np.asarray(s), x * np.float32(2))
    assert np.array_equal(np.asarray(d), x.astype(np.float64) - 1.0)


def test_zero_dimensional_and_size_one(ctx):
    ge = add_u32(ctx, dt="float32")
    a = gpuarray.array(np.float32(2.5), context=ctx)
    b = gpuarray.array(np.float32(4.0), context=ctx)
    c = gpuarray.empty((), "float32", context=ctx)
    ge(a, b, c)
    assert np.asarray(c) == np.float32(6.5)
    c3 = gpuarray.empty((1, 1, 1), "float32", context=ctx)
    ge(a, b, c3)                                      # padshape + broadcast defaults
    assert np.asarray(c3).ravel()[0] == np.float32(6.5)


# ---- the benchmark's shapes -----------------------------------------------------------------

def test_config1_contiguous_2p24(ctx, oracle):
    rng = np.random.default_rng(0)
    n = 1 << 24
    a = rng.uniform(-1, 1, n).astype(np.float32)
    b = rng.uniform(-1, 1, n).astype(np.float32)
    ge = ga.GpuElemwise(ctx, "c = a*b + 0.5f", [arg("a", "float32", read=True),
                                                arg("b", "float32", read=True),
                                                arg("c", "float32", write=True)])
    gc = gpuarray.empty((n,), "float32", context=ctx)
    ge(gpuarray.array(a, context=ctx), gpuarray.array(b, context=ctx), gc)
    got = np.asarray(gc)
    want = np.empty(n, np.float32)
    oracle.elemwise_contig_muladd(a, b, want)
    assert np.array_equal(got, want)
    assert np.array_equal(got, a * b + np.float32(0.5))


def test_config2_transposed_broadcast_4096(ctx, oracle):
    rng = np.random.default_rng(1)
    a = rng.normal(0, 1, (4096, 4096)).astype(np.float32)
    b = rng.normal(0, 1, (1, 4096)).astype(np.float32)
    c = rng.normal(0, 1, (4096, 1)).astype(np.float32)
    ge = ga.GpuElemwise(ctx, "out = a + b*c",
                        [arg("a", "float32", read=True), arg("b", "float32", read=True),
                         arg("c", "float32", read=True), arg("out", "float32", write=True)])
    g_a = gpuarray.array(a, context=ctx).T
    assert g_a.strides == (4, 16384) and g_a.flags.f_contiguous and not g_a.flags.c_contiguous
    out = gpuarray.empty((4096, 4096), "float32", context=ctx)
    # without GE_BROADCAST the call is refused, as in the reference
    assert raw_call(ge, [g_a, gpuarray.array(b, context=ctx), gpuarray.array(c, context=ctx), out],
                    0) == _lib.GA_VALUE_ERROR
    ge(g_a, gpuarray.array(b, context=ctx), gpuarray.array(c, context=ctx), out)
    got = np.asarray(out)
    assert np.array_equal(got, a.T + b * c)
    # the checker, on a corner that it finishes quickly
    sub = np.zeros((256, 256), np.float32)
    assert oracle.elemwise(oracle.A_PLUS_BC_F32, [a.T[:256, :256], b[:, :256], c[:256], sub],
                           [0, 0, 0, 1], flags=BCAST) == 0
    assert np.array_equal(got[:256, :256], sub)


def test_config5_strided_copy_of_the_view(ctx):
    rng = np.random.default_rng(6)
    base = rng.integers(-1000, 1001, (64, 128, 1024), dtype=np.int32)
    g = gpuarray.array(base, context=ctx)[:, :, ::2]
    assert g.strides == (128 * 1024 * 4, 4096, 8)
    c = g.copy()
    assert c.flags.c_contiguous and np.array_equal(np.asarray(c), base[:, :, ::2])


def test_linearity_at_full_size(ctx):
    # size-independent property at the 2^28 target shape: (a*b + 0.5) with
    # b == 1 is a + 0.5 exactly, and with a == 0 is 0.5 everywhere
    n = 1 << 28
    ge = ga.GpuElemwise(ctx, "c = a*b + 0.5f", [arg("a", "float32", read=True),
                                                arg("b", "float32", read=True),
                                                arg("c", "float32", write=True)])
    a = gpuarray.zeros((n,), "float32", context=ctx)
    b = gpuarray.empty((n,), "float32", context=ctx)
    c = gpuarray.empty((n,), "float32", context=ctx)
    ge(a, b, c)                                   # a == 0 but b is garbage: NaN/inf can appear
    fill = ga.GpuElemwise(ctx, "b = 1.0f", [arg("b", "float32", write=True)])
    fill(b)
    iota = ga.GpuElemwise(ctx, "a = (ga_float)(i & 1023)", [arg("a", "float32", write=True)])
    iota(a)
    ge(a, b, c)
    # sample three windows, including the very end
    for lo in (0, n // 2 - 5000, n - 10000):
        got = np.asarray(c[lo:lo + 10000])
        want = (np.arange(lo, lo + 10000) & 1023).astype(np.float32) + np.float32(0.5)
        assert np.array_equal(got, want)


@pytest.mark.parametrize("tile,band,panel", [(64, 0, 0), (64, 0, 3), (64, 1, 0), (64, 3, 0), (64, 8, 0),
                                             (128, 0, 0), (128, 0, 2), (128, 1, 0), (128, 2, 0), (128, 5, 0)])
def test_transposed_tiles_and_bands(ctx, knobs, tile, band, panel):
    """Every tile size and tile order of the transposed kernels (bands of
    `band` tile rows; 0: diagonals, within panels of `panel` tile columns), on
    extents that leave ragged tiles, a partial last band and a narrower last
    panel, with one and with two transposed operands, a transposed result,
    several planes and 8-byte elements: bit-exact against NumPy."""
    knobs(ELEMWISE_TTILE=tile, ELEMWISE_BAND=band, ELEMWISE_PANEL=panel)
    rng = np.random.default_rng(40 + tile + band)
    f32 = "float32"
    k2 = ga.GpuElemwise(ctx, "out = a + b*c", [arg("a", f32, read=True), arg("b", f32, read=True),
                                               arg("c", f32, read=True), arg("out", f32, write=True)])
    for ny, nx in ((516, 260), (128, 128), (1100, 68), (68, 1100), (644, 388)):
        a = rng.standard_normal((nx, ny)).astype(np.float32)        # used as a.T: (ny, nx)
        b = rng.standard_normal((1, nx)).astype(np.float32)
        c = rng.standard_normal((ny, 1)).astype(np.float32)
        out = gpuarray.empty((ny, nx), f32, context=ctx)
        k2(gpuarray.array(a, context=ctx).T, gpuarray.array(b, context=ctx),
           gpuarray.array(c, context=ctx), out)
        assert np.array_equal(np.asarray(out), a.T + b * c), (ny, nx)
        # an operand that is constant along both axes
        s11 = rng.standard_normal((1, 1)).astype(np.float32)
        k2(gpuarray.array(a, context=ctx).T, gpuarray.array(s11, context=ctx),
           gpuarray.array(c, context=ctx), out)
        assert np.array_equal(np.asarray(out), a.T + s11 * c), (ny, nx)
        # two transposed inputs
        a2 = rng.standard_normal((nx, ny)).astype(np.float32)
        k2(gpuarray.array(a, context=ctx).T, gpuarray.array(a2, context=ctx).T,
           gpuarray.array(c, context=ctx), out)
        assert np.array_equal(np.asarray(out), a.T + a2.T * c), (ny, nx)
        # transposed result: out.T written from C-ordered inputs
        outT = gpuarray.empty((nx, ny), f32, context=ctx)
        x = rng.standard_normal((ny, nx)).astype(np.float32)
        k2(gpuarray.array(x, context=ctx), gpuarray.array(b, context=ctx),
           gpuarray.array(c, context=ctx), outT.T)
        assert np.array_equal(np.asarray(outT), (x + b * c).T), (ny, nx)
    # planes (nd = 3) and 8-byte elements
    kd = ga.GpuElemwise(ctx, "o = p * 2.0", [arg("p", "float64", read=True), arg("o", "float64", write=True)])
    p = rng.standard_normal((3, 264, 392))
    o = gpuarray.empty((3, 392, 264), "float64", context=ctx)
    kd(gpuarray.array(p, context=ctx).transpose(0, 2, 1), o)
    assert np.array_equal(np.asarray(o), p.transpose(0, 2, 1) * 2.0)


@pytest.mark.parametrize("skew", [1, 0])
@pytest.mark.parametrize("tile", [64, 128])
def test_tile_windows_follow_result_rows_off_the_64_byte_blocks(ctx, knobs, tile, skew):
    """A result whose rows do not start on 64-byte blocks of memory: the
    transposed kernels move a tile's window on every row to the block
    boundary before it (ELEMWISE_SKEW).  Every phase of the first row (base 0
    to 12 floats into a block), pitches that walk through the phases from row
    to row, extents around a tile's width and around the extra columns the
    windows need, a row operand (its window moves with the row), several
    planes; with the rectangular tiles as well.  The whole buffer of the result
    is compared, so a store outside the view shows."""
    knobs(ELEMWISE_TTILE=tile, ELEMWISE_SKEW=skew, ELEMWISE_LOOSE_MIN_BYTES=1)
    rng = np.random.default_rng(700 + tile)
    k = ga.GpuElemwise(ctx, "o = a * r + c", [arg("a", "float32", read=True), arg("r", "float32", read=True),
                                              arg("c", "float32", read=True), arg("o", "float32", write=True)])
    cases = [(ny, nx, pad, lead) for ny in (36, 132) for nx in (4, 52, 116, 120, 124, 128, 132, 244, 252, 260)
             for pad, lead in ((4, 0), (8, 4), (12, 8), (20, 12), (16, 0), (0, 4))]
    for ny, nx, pad, lead in cases[::3] if tile == 64 else cases[1::3] + cases[2::3]:
        a = rng.integers(-9, 10, size=(nx, ny)).astype(np.float32)              # read as a.T
        r = rng.integers(-9, 10, size=(1, nx)).astype(np.float32)
        c = rng.integers(-9, 10, size=(ny, nx + 8)).astype(np.float32)[:, 4:4 + nx]   # its own phase
        root = rng.integers(-9, 10, size=(ny + 2, lead + nx + pad)).astype(np.float32)
        view = root[1:1 + ny, lead:lead + nx]
        go, groot = to_gpu_view(view, ctx)
        gc, _ = to_gpu_view(c, ctx)
        k(gpuarray.array(a, context=ctx).T, gpuarray.array(r, context=ctx), gc, go, broadcast=True)
        want = root.copy()
        want[1:1 + ny, lead:lead + nx] = a.T * r + c
        assert np.array_equal(read_root(groot, root), want), (ny, nx, pad, lead)
    # planes: the phase of a row depends on the plane too
    p = rng.integers(-9, 10, size=(3, 140, 76)).astype(np.float32)
    root = np.zeros((3, 76, 140 + 4), np.float32)
    go, groot = to_gpu_view(root[:, :, :140], ctx)
    kc = ga.GpuElemwise(ctx, "o = p", [arg("p", "float32", read=True), arg("o", "float32", write=True)])
    kc(gpuarray.array(p, context=ctx).transpose(0, 2, 1), go)
    want = root.copy()
    want[:, :, :140] = p.transpose(0, 2, 1)
    assert np.array_equal(read_root(groot, root), want)


@pytest.mark.parametrize("fill,tmin", [(1, 12), (0, 16), (1, 2)])
def test_transposed_operands_of_narrow_planes(ctx, knobs, fill, tmin):
    """(N, f) taken as its transpose with f from 3 to 130: the small tile where
    it is filled better than the large one (ELEMWISE_TTILE_FILL), tiles at all
    from ELEMWISE_TMIN elements along the narrow dim on (below, single elements
    per lane), with the kernel that holds very narrow planes in registers
    switched off; also the other way round, a narrow result of a wide transposed
    operand.  Floats and doubles, with a row operand; against NumPy, exact."""
    knobs(ELEMWISE_TTILE_FILL=fill, ELEMWISE_TMIN=tmin, ELEMWISE_TTILE_MIN=1, ELEMWISE_NARROW=0)
    rng = np.random.default_rng(830 + tmin)
    for dtype in ("float32", "float64"):
        k = ga.GpuElemwise(ctx, "o = a + r", [arg("a", dtype, read=True), arg("r", dtype, read=True),
                                               arg("o", dtype, write=True)])
        draw = lambda shape: rng.integers(-9, 10, size=shape).astype(dtype)
        for n, f in ((5000, 3), (4096, 8), (3001, 12), (2500, 13), (6000, 15), (4000, 16), (3333, 20),
                     (2048, 33), (2500, 48), (1999, 49), (1500, 100), (1111, 130)):
            a = draw((n, f))
            ga_ = gpuarray.array(a, context=ctx)
            r = draw((1, n))
            out = gpuarray.empty((f, n), dtype, context=ctx)
            k(ga_.transpose(1, 0), gpuarray.array(r, context=ctx), out, broadcast=True)
            assert np.array_equal(np.asarray(out), a.T + r), (dtype, n, f)
            b = draw((f, n))
            r2 = draw((1, f))
            out2 = gpuarray.empty((n, f), dtype, context=ctx)
            k(gpuarray.array(b, context=ctx).transpose(1, 0), gpuarray.array(r2, context=ctx), out2, broadcast=True)
            assert np.array_equal(np.asarray(out2), b.T + r2), (dtype, n, f, "wide")


@pytest.mark.parametrize("lds,nt,quads,wide", [(2, 3, 0, None), (3, 0, 1, 64), (0, 7, 1, None), (1, 1, 0, 64)])
def test_very_narrow_planes_held_in_registers(ctx, knobs, lds, nt, quads, wide):
    """(N, f) with f from 2 to 15 taken as its transpose, and written as one: a
    lane holds four positions of the long dim by all f of the short one
    (ELEMWISE_NARROW; the arrays with the short dim innermost directly or through
    the LDS, ELEMWISE_NARROW_LDS; the others as 16-byte chunks, on four-byte
    boundaries when N is no multiple of four).  f from 17 to 64: a group's piece
    of the arrays with the short dim innermost whole through the LDS
    (ELEMWISE_NARROW_STAGED for narrow results, _STAGED_WIDE for wide ones).  Long extents of whole and cut
    groups and lanes, a row operand, an array read and written, a result inside a
    larger buffer whose rows start off the 16-byte boundaries, batches of planes
    (channels last to channels first and back); floats and 32-bit integers against
    NumPy, exact."""
    knobs(ELEMWISE_NARROW_LDS=lds, ELEMWISE_NARROW_NT=nt, ELEMWISE_NARROW_QUADS=quads, ELEMWISE_NARROW_MIN=1024,
          ELEMWISE_NARROW_STAGED_WIDE=wide)
    rng = np.random.default_rng(900 + lds)
    for dtype in ("float32", "int32"):
        k = ga.GpuElemwise(ctx, "o = a + r", [arg("a", dtype, read=True), arg("r", dtype, read=True),
                                               arg("o", dtype, write=True)])
        kio = ga.GpuElemwise(ctx, "o = o - a", [arg("a", dtype, read=True), arg("o", dtype, read=True, write=True)])
        draw = lambda shape: rng.integers(-9, 10, size=shape).astype(dtype)
        for f in list(range(2, 16)) + [17, 20, 23, 31, 32, 33, 50, 63, 64]:
            for n in ((1024, 4099, 100001) if f % 3 else (2048, 5003, 8190)):
                a = draw((n, f))
                r = draw((1, n))
                out = gpuarray.empty((f, n), dtype, context=ctx)
                k(gpuarray.array(a, context=ctx).transpose(1, 0), gpuarray.array(r, context=ctx), out, broadcast=True)
                assert np.array_equal(np.asarray(out), a.T + r), (dtype, n, f)
                b = draw((f, n))
                r2 = draw((1, f))
                out2 = gpuarray.empty((n, f), dtype, context=ctx)
                k(gpuarray.array(b, context=ctx).transpose(1, 0), gpuarray.array(r2, context=ctx), out2, broadcast=True)
                assert np.array_equal(np.asarray(out2), b.T + r2), (dtype, n, f, "narrow result")
                o3 = draw((n, f))
                g3 = gpuarray.array(o3, context=ctx)
                kio(gpuarray.array(b, context=ctx).transpose(1, 0), g3)
                assert np.array_equal(np.asarray(g3), o3 - b.T), (dtype, n, f, "read and written")
        # the wide result inside a larger buffer: rows one element into pitches of n + 3
        n, f = 6001, 5
        a = draw((n, f))
        root = np.zeros((f, n + 3), dtype)
        go, groot = to_gpu_view(root[:, 1:n + 1], ctx)
        kc = ga.GpuElemwise(ctx, "o = a", [arg("a", dtype, read=True), arg("o", dtype, write=True)])
        kc(gpuarray.array(a, context=ctx).transpose(1, 0), go)
        want = root.copy()
        want[:, 1:n + 1] = a.T
        assert np.array_equal(read_root(groot, root), want), dtype
        # planes: channels last to channels first and back, (B, H, W, C) <-> (B, C, H, W); whole planes
        # of 1024 positions, cut ones, short ones, and planes inside a larger buffer
        for bsz, h, w, c in ((3, 32, 32, 3), (5, 17, 31, 7), (2, 40, 50, 4), (4, 16, 16, 5), (3, 20, 21, 18), (2, 16, 16, 35)):
            x = draw((bsz, h, w, c))
            out = gpuarray.empty((bsz, c, h, w), dtype, context=ctx)
            kc(gpuarray.array(x, context=ctx).transpose(0, 3, 1, 2), out)
            assert np.array_equal(np.asarray(out), x.transpose(0, 3, 1, 2)), (dtype, bsz, h, w, c)
            y = draw((bsz, c, h, w))
            out = gpuarray.empty((bsz, h, w, c), dtype, context=ctx)
            kc(gpuarray.array(y, context=ctx).transpose(0, 2, 3, 1), out)
            assert np.array_equal(np.asarray(out), y.transpose(0, 2, 3, 1)), (dtype, bsz, h, w, c, "back")
        xroot = draw((3, 1000 + 2, 6))
        gx_, _ = to_gpu_view(xroot[:, 2:], ctx)
        oroot = np.zeros((3, 6 + 1, 1000), dtype)
        go, groot = to_gpu_view(oroot[:, :6], ctx)
        kc(gx_.transpose(0, 2, 1), go)
        want = oroot.copy()
        want[:, :6] = xroot[:, 2:].transpose(0, 2, 1)
        assert np.array_equal(read_root(groot, oroot), want), dtype
        # the narrow operand as a view that starts off the 16-byte boundaries: the other kernels
        aroot = draw((n + 1, f))
        gv, _ = to_gpu_view(aroot[1:], ctx)
        out = gpuarray.empty((f, n), dtype, context=ctx)
        kc(gv.transpose(1, 0), out)
        assert np.array_equal(np.asarray(out), aroot[1:].T), dtype


@pytest.mark.parametrize("dtype", ["float64", "int64", "float16", "int16"])
def test_very_narrow_planes_of_two_and_eight_byte_elements(ctx, knobs, dtype):
    """The kernel that holds narrow planes in registers with two and eight elements
    to a 16-byte chunk: (N, f) as its transpose and written as one, f from 2 to 15, N
    with and without whole chunks (rows of the wide side off the 16-byte
    boundaries), an array read and written, planes; halves computed as floats.
    Against NumPy, exact (small integers)."""
    knobs(ELEMWISE_NARROW_MIN=1024, ELEMWISE_NARROW_QUADS=1)
    rng = np.random.default_rng(917)
    k = ga.GpuElemwise(ctx, "o = a + r", [arg("a", dtype, read=True), arg("r", dtype, read=True),
                                           arg("o", dtype, write=True)], convert_f16=True)
    kio = ga.GpuElemwise(ctx, "o = o - a", [arg("a", dtype, read=True), arg("o", dtype, read=True, write=True)],
                         convert_f16=True)
    draw = lambda shape: rng.integers(-9, 10, size=shape).astype(dtype)
    for f in (2, 3, 4, 5, 8, 11, 15):
        for n in (2048, 4099, 65537):
            a = draw((n, f))
            r = draw((1, n))
            out = gpuarray.empty((f, n), dtype, context=ctx)
            k(gpuarray.array(a, context=ctx).transpose(1, 0), gpuarray.array(r, context=ctx), out, broadcast=True)
            assert np.array_equal(np.asarray(out), a.T + r), (n, f)
            b = draw((f, n))
            r2 = draw((1, f))
            out2 = gpuarray.empty((n, f), dtype, context=ctx)
            k(gpuarray.array(b, context=ctx).transpose(1, 0), gpuarray.array(r2, context=ctx), out2, broadcast=True)
            assert np.array_equal(np.asarray(out2), b.T + r2), (n, f, "narrow result")
            o3 = draw((n, f))
            g3 = gpuarray.array(o3, context=ctx)
            kio(gpuarray.array(b, context=ctx).transpose(1, 0), g3)
            assert np.array_equal(np.asarray(g3), o3 - b.T), (n, f, "read and written")
    kc = ga.GpuElemwise(ctx, "o = a", [arg("a", dtype, read=True), arg("o", dtype, write=True)], convert_f16=True)
    for bsz, h, w, c in ((3, 32, 32, 3), (5, 17, 31, 7), (2, 40, 52, 2)):
        x = draw((bsz, h, w, c))
        out = gpuarray.empty((bsz, c, h, w), dtype, context=ctx)
        kc(gpuarray.array(x, context=ctx).transpose(0, 3, 1, 2), out)
        assert np.array_equal(np.asarray(out), x.transpose(0, 3, 1, 2)), (bsz, h, w, c)
        y = draw((bsz, c, h, w))
        out = gpuarray.empty((bsz, h, w, c), dtype, context=ctx)
        kc(gpuarray.array(y, context=ctx).transpose(0, 2, 3, 1), out)
        assert np.array_equal(np.asarray(out), y.transpose(0, 2, 3, 1)), (bsz, h, w, c, "back")


def test_very_narrow_planes_between_element_sizes(ctx, knobs):
    """Narrow planes in registers with arrays of different element sizes (images of
    bytes, halves and floats between channels last and channels first, also with one
    byte per element throughout): a lane's positions are a chunk of the smallest
    type, and of the wider arrays several chunks.  A wide result of wider elements
    than the operand's is the strided kernel's (its rows would be stored in pieces);
    checked all the same.  Against NumPy, exact (small integers)."""
    knobs(ELEMWISE_NARROW_MIN=1024)
    rng = np.random.default_rng(931)
    for di, do in (("uint8", "uint8"), ("uint8", "float32"), ("float32", "uint8"), ("float16", "float32"),
                   ("float32", "float16"), ("int16", "int64"), ("float64", "uint8")):
        kc = ga.GpuElemwise(ctx, "o = a + 1", [arg("a", di, read=True), arg("o", do, write=True)], convert_f16=True)
        for bsz, h, w, c in ((2, 40, 52, 3), (3, 33, 31, 4), (1, 70, 70, 7), (2, 64, 64, 1 + 14 * (di == do))):
            x = rng.integers(0, 10, size=(bsz, h, w, c)).astype(di)
            out = gpuarray.empty((bsz, c, h, w), do, context=ctx)
            kc(gpuarray.array(x, context=ctx).transpose(0, 3, 1, 2), out)
            assert np.array_equal(np.asarray(out), (x.transpose(0, 3, 1, 2) + 1).astype(do)), (di, do, bsz, h, w, c)
            y = rng.integers(0, 10, size=(bsz, c, h, w)).astype(di)
            out = gpuarray.empty((bsz, h, w, c), do, context=ctx)
            kc(gpuarray.array(y, context=ctx).transpose(0, 2, 3, 1), out)
            assert np.array_equal(np.asarray(out), (y.transpose(0, 2, 3, 1) + 1).astype(do)), (di, do, bsz, h, w, c, "back")
        # a per-channel shift and factor fused into the change of layout (fetched once per channel)
        kn = ga.GpuElemwise(ctx, "o = (a - m) * s", [arg("a", di, read=True), arg("m", do, read=True), arg("s", do, read=True),
                                                      arg("o", do, write=True)], convert_f16=True)
        for bsz, h, w, c in ((2, 40, 52, 3), (3, 33, 31, 5)):
            x = rng.integers(4, 10, size=(bsz, h, w, c)).astype(di)
            m = rng.integers(0, 4, size=(1, c, 1, 1)).astype(do)
            f_ = rng.integers(1, 4, size=(1, c, 1, 1)).astype(do)
            out = gpuarray.empty((bsz, c, h, w), do, context=ctx)
            kn(gpuarray.array(x, context=ctx).transpose(0, 3, 1, 2), gpuarray.array(m, context=ctx),
               gpuarray.array(f_, context=ctx), out, broadcast=True)
            want = ((x.transpose(0, 3, 1, 2).astype(np.float64) - m) * f_).astype(do)
            assert np.array_equal(np.asarray(out), want), (di, do, bsz, h, w, c, "normalised")
            y = rng.integers(4, 10, size=(bsz, c, h, w)).astype(di)
            ml, fl = m.reshape(1, 1, 1, c), f_.reshape(1, 1, 1, c)
            out = gpuarray.empty((bsz, h, w, c), do, context=ctx)
            kn(gpuarray.array(y, context=ctx).transpose(0, 2, 3, 1), gpuarray.array(ml, context=ctx),
               gpuarray.array(fl, context=ctx), out, broadcast=True)
            want = ((y.transpose(0, 2, 3, 1).astype(np.float64) - ml) * fl).astype(do)
            assert np.array_equal(np.asarray(out), want), (di, do, bsz, h, w, c, "normalised, back")
        for n, f in ((4099, 3), (70001, 5)):
            a = rng.integers(0, 10, size=(n, f)).astype(di)
            out = gpuarray.empty((f, n), do, context=ctx)
            kc(gpuarray.array(a, context=ctx).transpose(1, 0), out)
            assert np.array_equal(np.asarray(out), (a.T + 1).astype(do)), (di, do, n, f)
            b = rng.integers(0, 10, size=(f, n)).astype(di)
            out = gpuarray.empty((n, f), do, context=ctx)
            kc(gpuarray.array(b, context=ctx).transpose(1, 0), out)
            assert np.array_equal(np.asarray(out), (b.T + 1).astype(do)), (di, do, n, f, "narrow result")


@pytest.mark.parametrize("tile,nt,skew", [(0, 3, 1), (8, 0, 2), (64, 1, 0), (16, 6, 2), (0, 7, 0)])
def test_matrices_of_short_records_taken_as_their_transposes(ctx, knobs, tile, nt, skew):
    """(X, Y, f) with a short inner dim taken as (Y, X, f): images turned, sequences
    of short feature vectors between batch-major and time-major.  Tiles of records
    through the LDS (ELEMWISE_RECORDS; side of a tile ELEMWISE_RECORDS_TILE): whole
    and cut tiles, a second operand laid out like the result, a broadcast operand,
    planes, and an operand whose records start inside a larger buffer; rectangular
    tiles and windows moved onto the result's 64-byte blocks (ELEMWISE_RECORDS_SKEW:
    0 never, 1 where the result's rows start off them, 2 always; the same values
    for ELEMWISE_RECORDS_YMAJOR, tiles numbered along Y first), also with the
    result inside a larger buffer.  Floats and
    32-bit integers against NumPy, exact."""
    knobs(ELEMWISE_RECORDS_TILE=tile, ELEMWISE_RECORDS_NT=nt, ELEMWISE_RECORDS_MIN=1, ELEMWISE_RECORDS_SKEW=skew,
          ELEMWISE_RECORDS_YMAJOR=skew)
    rng = np.random.default_rng(950 + tile)
    for dtype in ("float32", "int32"):
        k = ga.GpuElemwise(ctx, "o = a + b * r", [arg("a", dtype, read=True), arg("b", dtype, read=True),
                                                   arg("r", dtype, read=True), arg("o", dtype, write=True)])
        kc = ga.GpuElemwise(ctx, "o = a", [arg("a", dtype, read=True), arg("o", dtype, write=True)])
        draw = lambda shape: rng.integers(-9, 10, size=shape).astype(dtype)
        for f in (2, 3, 5, 8, 13, 16, 33, 64):
            if tile == 64 and f > 4:
                continue          # (more LDS than a group has)
            for ny, nx in ((32, 32), (100, 257), (333, 64), (65, 1000)):
                a = draw((nx, ny, f))
                b = draw((ny, nx, f))
                r = draw((1, nx, 1))
                out = gpuarray.empty((ny, nx, f), dtype, context=ctx)
                k(gpuarray.array(a, context=ctx).transpose(1, 0, 2), gpuarray.array(b, context=ctx),
                  gpuarray.array(r, context=ctx), out, broadcast=True)
                assert np.array_equal(np.asarray(out), a.transpose(1, 0, 2) + b * r), (dtype, f, ny, nx)
                aroot = draw((3, nx, ny + 2, f))
                gv, _ = to_gpu_view(aroot[:, :, 1:ny + 1, :], ctx)
                out2 = gpuarray.empty((3, ny, nx, f), dtype, context=ctx)
                kc(gv.transpose(0, 2, 1, 3), out2)
                assert np.array_equal(np.asarray(out2), aroot[:, :, 1:ny + 1, :].transpose(0, 2, 1, 3)), (dtype, f, ny, nx, "planes")
            # the result inside a larger buffer: rows that start 1 + 2 f elements into pitches of (nx + 3) f
            ny, nx = 70, 130
            a = draw((nx, ny, f))
            oroot = np.zeros((ny, nx + 3, f), dtype)
            oroot.reshape(-1)[0] = 0
            go, groot = to_gpu_view(oroot[:, 2:nx + 2, :], ctx)
            kc(gpuarray.array(a, context=ctx).transpose(1, 0, 2), go)
            want = oroot.copy()
            want[:, 2:nx + 2, :] = a.transpose(1, 0, 2)
            assert np.array_equal(read_root(groot, oroot), want), (dtype, f, "result inside a larger buffer")


@pytest.mark.parametrize("skew", [1, 2])
@pytest.mark.parametrize("dtype", ["uint8", "int16", "float16", "float64"])
def test_matrices_of_short_records_of_other_element_sizes(ctx, knobs, dtype, skew):
    """The tiles of records with 16, 8 and 2 elements to a 16-byte chunk: byte images
    turned, records of halves and doubles; with a second operand laid out like the
    result and a broadcast one, planes, cut tiles; halves computed as floats."""
    knobs(ELEMWISE_RECORDS_MIN=1, ELEMWISE_RECORDS_SKEW=skew, ELEMWISE_RECORDS_YMAJOR=skew)
    rng = np.random.default_rng(977)
    k = ga.GpuElemwise(ctx, "o = a + b * r", [arg("a", dtype, read=True), arg("b", dtype, read=True),
                                               arg("r", dtype, read=True), arg("o", dtype, write=True)], convert_f16=True)
    kc = ga.GpuElemwise(ctx, "o = a", [arg("a", dtype, read=True), arg("o", dtype, write=True)], convert_f16=True)
    draw = lambda shape: rng.integers(0, 4, size=shape).astype(dtype)
    for f in (2, 3, 4, 8, 21, 32):
        for ny, nx in ((64, 64), (100, 257), (65, 1000)):
            a = draw((nx, ny, f))
            b = draw((ny, nx, f))
            r = draw((1, nx, 1))
            out = gpuarray.empty((ny, nx, f), dtype, context=ctx)
            k(gpuarray.array(a, context=ctx).transpose(1, 0, 2), gpuarray.array(b, context=ctx),
              gpuarray.array(r, context=ctx), out, broadcast=True)
            assert np.array_equal(np.asarray(out), a.transpose(1, 0, 2) + b * r), (f, ny, nx)
            aroot = draw((2, nx, ny + 2, f))
            gv, _ = to_gpu_view(aroot[:, :, 1:ny + 1, :], ctx)
            out2 = gpuarray.empty((2, ny, nx, f), dtype, context=ctx)
            kc(gv.transpose(0, 2, 1, 3), out2)
            assert np.array_equal(np.asarray(out2), aroot[:, :, 1:ny + 1, :].transpose(0, 2, 1, 3)), (f, ny, nx, "planes")


@pytest.mark.parametrize("loose", [1, 0])
@pytest.mark.parametrize("dtype", ["float32", "int32"])
def test_transposed_operands_of_four_byte_elements_on_any_layout(ctx, knobs, dtype, loose):
    """Transposed operands whose bases, pitches and extents are no multiples of
    four elements (ELEMWISE_LOOSE: four elements per lane through accesses that
    assume four-byte boundaries only, cut quads element by element; 0: one
    element per lane).  Odd extents around the tile sizes, every phase of the
    operand's and the result's first element, a row and a column operand, a
    second transposed operand, planes; the result's whole buffer is compared."""
    knobs(ELEMWISE_LOOSE=loose, ELEMWISE_LOOSE_MIN_BYTES=1)
    rng = np.random.default_rng(810 + loose)
    k = ga.GpuElemwise(ctx, "o = a * r + c", [arg("a", dtype, read=True), arg("r", dtype, read=True),
                                              arg("c", dtype, read=True), arg("o", dtype, write=True)])
    k2 = ga.GpuElemwise(ctx, "o = a - b", [arg("a", dtype, read=True), arg("b", dtype, read=True),
                                           arg("o", dtype, write=True)])
    draw = lambda shape: rng.integers(-9, 10, size=shape).astype(dtype)
    for ny, nx in ((17, 19), (63, 130), (129, 127), (131, 257), (250, 66), (61, 391), (257, 129)):
        for la, lo_, pad in ((0, 0, 0), (1, 0, 3), (2, 3, 1), (3, 1, 2), (0, 2, 5)):
            aroot = draw((nx + 1, la + ny + pad))
            a = aroot[1:, la:la + ny]                        # read as a.T: rows start at any element
            r = draw((1, nx))
            c = draw((ny, 1))
            root = draw((ny + 2, lo_ + nx + pad))
            view = root[1:1 + ny, lo_:lo_ + nx]
            go, groot = to_gpu_view(view, ctx)
            gat, _ = to_gpu_view(a.T, ctx)
            k(gat, gpuarray.array(r, context=ctx), gpuarray.array(c, context=ctx), go, broadcast=True)
            want = root.copy()
            want[1:1 + ny, lo_:lo_ + nx] = a.T * r + c
            assert np.array_equal(read_root(groot, root), want), (ny, nx, la, lo_, pad)
            b = draw((nx, ny + 1))[:, 1:]
            gbt, _ = to_gpu_view(b.T, ctx)
            k2(gat, gbt, go)
            want[1:1 + ny, lo_:lo_ + nx] = a.T - b.T
            assert np.array_equal(read_root(groot, root), want), (ny, nx, la, lo_, pad)
    p = draw((3, 133, 77))
    root = np.zeros((3, 77, 133 + 3), dtype)
    go, groot = to_gpu_view(root[:, :, 2:135], ctx)
    kc = ga.GpuElemwise(ctx, "o = p", [arg("p", dtype, read=True), arg("o", dtype, write=True)])
    kc(gpuarray.array(p, context=ctx).transpose(0, 2, 1), go)
    want = root.copy()
    want[:, :, 2:135] = p.transpose(0, 2, 1)
    assert np.array_equal(read_root(groot, root), want)


@pytest.mark.parametrize("loose", [1, 0])
def test_row_views_of_four_byte_elements_on_any_layout(ctx, knobs, loose):
    """Views without transposed operands whose rows start at any element and
    have any length: the quads of a row start on the result's 16-byte
    boundaries, before the row if need be, and the quads that an end of the
    row cuts move element by element (ELEMWISE_LOOSE; 0: one element per
    lane).  Rows of 1 to 9 elements in every phase (a cut quad can hold the
    whole row), longer odd rows, operands in other phases than the result,
    a stepped and a constant operand; the result's whole buffer is compared."""
    knobs(ELEMWISE_LOOSE=loose, ELEMWISE_LOOSE_MIN_BYTES=1)
    rng = np.random.default_rng(830 + loose)
    k = ga.GpuElemwise(ctx, "o = a * s + c", [arg("a", "float32", read=True), arg("s", "float32", read=True),
                                              arg("c", "float32", read=True), arg("o", "float32", write=True)])
    draw = lambda shape: rng.integers(-9, 10, size=shape).astype(np.float32)
    for rows in (1, 7, 300):
        for n in (1, 2, 3, 4, 5, 6, 7, 8, 9, 31, 130, 1001):
            for lo_, la, pad in ((0, 1, 1), (1, 0, 2), (2, 3, 1), (3, 2, 3)):
                root = draw((rows + 1, lo_ + n + pad))
                view = root[1:, lo_:lo_ + n]
                a = draw((rows, la + n + 2))[:, la:la + n]
                st = draw((rows, 2 * n + 1))[:, 1::2]                  # stepped along the row
                c = draw((rows, 1))                                    # constant along the row
                go, groot = to_gpu_view(view, ctx)
                k(to_gpu_view(a, ctx)[0], to_gpu_view(st, ctx)[0], gpuarray.array(c, context=ctx), go, broadcast=True)
                want = root.copy()
                want[1:, lo_:lo_ + n] = a * st + c
                assert np.array_equal(read_root(groot, root), want), (rows, n, lo_, la, pad)
    # rows that run backwards through memory, next to each other
    root = draw((40, 6))
    view = root[::-1, 1:4]
    a = draw((40, 3))
    go, groot = to_gpu_view(view, ctx)
    k(gpuarray.array(a, context=ctx), gpuarray.array(a, context=ctx), gpuarray.array(draw((40, 1)) * 0, context=ctx), go,
      broadcast=True)
    want = root.copy()
    want[::-1, 1:4] = a * a
    assert np.array_equal(read_root(groot, root), want)


def test_math_library_functions_match_numpy(ctx):
    """The C math library as kernels see it (the library's own device runtime
    maps it to compiler builtins and the device library): every function on
    float32 and float64 arrays against NumPy / SciPy, to a few units in the
    last place; the rounding functions, fabs, fmin / fmax, copysign, sqrt and
    fmod exactly."""
    import scipy.special as sp
    rng = np.random.default_rng(77)
    n = 4096
    pos = rng.uniform(0.05, 20.0, n)
    sym = rng.uniform(-6.0, 6.0, n)
    unit = rng.uniform(-0.98, 0.98, n)
    other = rng.uniform(0.5, 4.0, n)
    with np.errstate(all="ignore"):
        cases = [
            ("exp(a)", sym, None, np.exp, 4), ("exp2(a)", sym, None, np.exp2, 4),
            ("exp10(a)", sym, None, lambda x: np.power(x.dtype.type(10), x), 4),
            ("expm1(a)", sym, None, np.expm1, 4), ("log(a)", pos, None, np.log, 4),
            ("log2(a)", pos, None, np.log2, 4), ("log10(a)", pos, None, np.log10, 4),
            ("log1p(a)", pos, None, np.log1p, 4), ("sqrt(a)", pos, None, np.sqrt, 0),
            ("rsqrt(a)", pos, None, lambda x: 1 / np.sqrt(x), 4), ("cbrt(a)", sym, None, np.cbrt, 4),
            ("sin(a)", sym, None, np.sin, 4), ("cos(a)", sym, None, np.cos, 4),
            ("tan(a)", unit, None, np.tan, 6), ("asin(a)", unit, None, np.arcsin, 6),
            ("acos(a)", unit, None, np.arccos, 6), ("atan(a)", sym, None, np.arctan, 4),
            ("sinh(a)", sym, None, np.sinh, 6), ("cosh(a)", sym, None, np.cosh, 6),
            ("tanh(a)", sym, None, np.tanh, 6), ("asinh(a)", sym, None, np.arcsinh, 6),
            ("acosh(a)", other + 1, None, np.arccosh, 6), ("atanh(a)", unit, None, np.arctanh, 8),
            ("erf(a)", sym, None, sp.erf, 8), ("erfc(a)", unit, None, sp.erfc, 8),
            ("lgamma(a)", pos, None, sp.gammaln, 64), ("tgamma(a)", other, None, sp.gamma, 16),
            ("floor(a)", sym, None, np.floor, 0), ("ceil(a)", sym, None, np.ceil, 0),
            ("trunc(a)", sym, None, np.trunc, 0), ("rint(a)", sym, None, np.rint, 0),
            ("fabs(a)", sym, None, np.abs, 0),
            ("round(a)", sym, None, lambda x: np.copysign(np.floor(np.abs(x) + x.dtype.type(0.5)), x), 0),
            ("pow(a, b)", pos, other, np.power, 16), ("atan2(a, b)", sym, other, np.arctan2, 6),
            ("hypot(a, b)", sym, other, np.hypot, 4), ("fmod(a, b)", sym, other, np.fmod, 0),
            ("fmin(a, b)", sym, other, np.fmin, 0), ("fmax(a, b)", sym, other, np.fmax, 0),
            ("copysign(a, b)", sym, -other, np.copysign, 0),
        ]
        for dt in ("float32", "float64"):
            eps = np.finfo(dt).eps
            for expr, xa, xb, fn, ulps in cases:
                a = xa.astype(dt)
                b = (xb if xb is not None else other).astype(dt)
                want = fn(a, b) if xb is not None else fn(a)
                k = ga.GpuElemwise(ctx, "c = " + expr, [arg("a", dt, read=True), arg("b", dt, read=True),
                                                         arg("c", dt, write=True)])
                out = gpuarray.empty((n,), dt, context=ctx)
                k(gpuarray.array(a, context=ctx), gpuarray.array(b, context=ctx), out)
                got = np.asarray(out)
                assert got.dtype == np.dtype(dt)
                if ulps == 0:
                    assert np.array_equal(got, want.astype(dt)), (expr, dt)
                else:
                    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
                    tol = ulps * eps * np.maximum(np.abs(want.astype(np.float64)), 1e-30)
                    if expr in ("sin(a)", "cos(a)", "lgamma(a)"):
                        tol = np.maximum(tol, ulps * eps)      # results near a zero of the function
                    assert (err <= tol).all(), (expr, dt, float((err / tol).max()))
    # integer arguments go to the double function, as in <cmath>
    k = ga.GpuElemwise(ctx, "c = sqrt(a) + pow(a, 2)", [arg("a", "int32", read=True), arg("c", "float64", write=True)])
    ia = rng.integers(0, 1000, n).astype("int32")
    out = gpuarray.empty((n,), "float64", context=ctx)
    k(gpuarray.array(ia, context=ctx), out)
    assert np.allclose(np.asarray(out), np.sqrt(ia.astype(np.float64)) + ia.astype(np.float64) ** 2, rtol=1e-15)


@pytest.mark.parametrize("rowload", [8, 0])
def test_broadcast_rows_of_four_byte_elements_fetched_a_chunk_at_a_time(ctx, knobs, rowload):
    """A row operand broadcast against a dense array whose rows are no whole
    number of 16-byte chunks, or that does not start on a 16-byte boundary:
    the flat kernel fetches the chunks that lie inside one row with one load
    that assumes four-byte boundaries only, and the chunks that straddle two
    rows element by element (ELEMWISE_PERIODIC_ROWLOAD: the shortest row that
    is read this way, 1024 elements unless set; 0: none).  Row lengths around
    the multiples of four, every phase of the operand's first element, a
    dense array that starts off a chunk (a head of one to three elements), two
    and three dims, int32 as well; bit for bit against NumPy."""
    knobs(ELEMWISE_PERIODIC=2, ELEMWISE_PERIODIC_ROWLOAD=rowload)
    rng = np.random.default_rng(93 + rowload)
    for dt in ("float32", "int32"):
        k2 = ga.GpuElemwise(ctx, "o = a * b + c", [arg("a", dt, read=True), arg("b", dt, read=True),
                                                    arg("c", dt, read=True), arg("o", dt, write=True)])
        draw = lambda shape: rng.integers(-50, 51, size=shape).astype(dt)
        for R, Cn in ((300, 1001), (517, 10), (64, 17), (1000, 8), (77, 9), (4099, 11), (33, 1000), (129, 254), (5, 6)):
            for lead in (0, 1, 2, 3):
                a = draw((R, Cn))
                wide = draw((1, Cn + 4))
                row = wide[:, lead:lead + Cn]
                col = draw((R, 1))
                ga_, gw, gc = (gpuarray.array(x, context=ctx) for x in (a, wide, col))
                out = gpuarray.empty((R, Cn), dt, context=ctx)
                k2(ga_, gw[:, lead:lead + Cn], gc, out, broadcast=True)
                assert np.array_equal(np.asarray(out), a * row + col), (dt, R, Cn, lead)
            # the dense array starts one to three elements into its buffer
            for head in (1, 3):
                flat = draw((R * Cn + 4,))
                gf = gpuarray.array(flat, context=ctx)
                a = flat[head:head + R * Cn].reshape(R, Cn)
                row, col = draw((1, Cn)), draw((R, 1))
                out = gpuarray.empty((R, Cn), dt, context=ctx)
                k2(gf[head:head + R * Cn].reshape((R, Cn)), gpuarray.array(row, context=ctx),
                   gpuarray.array(col, context=ctx), out, broadcast=True)
                assert np.array_equal(np.asarray(out), a * row + col), (dt, R, Cn, "head", head)
        # three dims: an operand that varies along the outer and the inner dim, and a row of the inner dim
        for shape in ((33, 10, 257), (2, 5, 4099), (9, 6, 250), (7, 3, 9)):
            a = draw(shape)
            nb = draw((shape[0], 1, shape[2]))
            rw = draw((1, 1, shape[2]))
            out = gpuarray.empty(shape, dt, context=ctx)
            k2(gpuarray.array(a, context=ctx), gpuarray.array(nb, context=ctx), gpuarray.array(rw, context=ctx), out, broadcast=True)
            assert np.array_equal(np.asarray(out), a * nb + rw), (dt, shape)


@pytest.mark.parametrize("mode", ["1", "2", "0"])
def test_dense_arrays_with_broadcast_operands(ctx, oracle, knobs, mode):
    """Dense arrays combined with operands broadcast along some dims take the
    flat kernel, which reads the broadcast operands through the coordinates of
    the flat index (mode 1: where four elements per lane are not possible;
    2: always; 0: never): two and three collapsed dims, extents that are not
    multiples of 4, a misaligned first element, a strided column, several
    broadcast operands, mixed types, 8- and 1-byte elements; bit for bit
    against NumPy."""
    knobs(ELEMWISE_PERIODIC=mode)
    rng = np.random.default_rng(91)
    f32 = "float32"
    k3 = ga.GpuElemwise(ctx, "o = a * b + c", [arg("a", f32, read=True), arg("b", f32, read=True),
                                                arg("c", f32, read=True), arg("o", f32, write=True)])
    def run(k, ins, shape, dt=f32):
        out = gpuarray.empty(shape, dt, context=ctx)
        k(*ins, out, broadcast=True)
        return np.asarray(out)
    for R, Cn in ((1000, 3), (517, 10), (300, 1001), (64, 17), (5, 1), (1, 7), (4099, 5), (513, 1000), (37, 64)):
        a = rng.standard_normal((R, Cn)).astype(f32)
        row = rng.standard_normal((1, Cn)).astype(f32)
        col = rng.standard_normal((R, 1)).astype(f32)
        g = lambda x: gpuarray.array(x, context=ctx)
        assert np.array_equal(run(k3, [g(a), g(row), g(col)], (R, Cn)), a * row + col), (R, Cn)
        assert np.array_equal(run(k3, [g(row), g(a), g(a)], (R, Cn)), row * a + a), (R, Cn)
        # the dense operand starts off a 16-byte boundary; the column is a strided view
        wide = rng.standard_normal((R + 1, Cn)).astype(f32)
        mat = rng.standard_normal((R, 6)).astype(f32)
        gw, gm = g(wide), g(mat)
        got = run(k3, [gw[1:], g(row), gm[:, 2:3]], (R, Cn))
        assert np.array_equal(got, wide[1:] * row + mat[:, 2:3]), (R, Cn)
    # three dims: per-channel operands, and one that varies along two dims
    for shape in ((7, 3, 5), (33, 10, 257), (2, 5, 4099), (129, 3, 1), (9, 6, 256)):
        a = rng.standard_normal(shape).astype(f32)
        ch = rng.standard_normal((1, shape[1], 1)).astype(f32)
        nb = rng.standard_normal((shape[0], 1, shape[2])).astype(f32)
        g = lambda x: gpuarray.array(x, context=ctx)
        assert np.array_equal(run(k3, [g(a), g(ch), g(nb)], shape), a * ch + nb), shape
        assert np.array_equal(run(k3, [g(a), g(ch), g(ch)], shape), a * ch + ch), shape
    # other element sizes and mixed types
    kd = ga.GpuElemwise(ctx, "o = a + b", [arg("a", "float64", read=True), arg("b", f32, read=True),
                                            arg("o", "float64", write=True)])
    a = rng.standard_normal((257, 9)); b = rng.standard_normal((1, 9)).astype(f32)
    assert np.array_equal(run(kd, [gpuarray.array(a, context=ctx), gpuarray.array(b, context=ctx)], (257, 9), "float64"), a + b)
    kb = ga.GpuElemwise(ctx, "o = a ^ b", [arg("a", "uint8", read=True), arg("b", "uint8", read=True),
                                            arg("o", "uint8", write=True)])
    a = rng.integers(0, 256, (301, 37), dtype=np.uint8); b = rng.integers(0, 256, (301, 1), dtype=np.uint8)
    assert np.array_equal(run(kb, [gpuarray.array(a, context=ctx), gpuarray.array(b, context=ctx)], (301, 37), "uint8"), a ^ b)
