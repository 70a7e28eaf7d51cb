"""The array object's NumPy-facing behaviour, after the reference's Python
tests (pygpu/tests/test_gpu_ndarray.py:40-760): NumPy's own shape, strides,
flags and content are the expected values."""
import copy
import itertools

import numpy as np
import pytest

import libgpuarray_amd as ga
from libgpuarray_amd import gpuarray
from support import gen_gpuarray, to_gpu_view

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "float64", "int8", "int16", "uint8", "uint16", "int32", "int64", "uint32",
          "uint64", "float16"]
SHAPES = [(), (5,), (6, 7), (4, 8, 9), (1, 8, 9)]


def check_flags(x, y):
    """pygpu/tests/support.py:52-87: nothing is asked of empty arrays, and a
    C-ordered device copy of an array NumPy keeps in Fortran order is accepted."""
    if y.size == 0:
        pass
    elif x.flags["C_CONTIGUOUS"] != y.flags["C_CONTIGUOUS"]:
        assert x.flags["C_CONTIGUOUS"] is True and x.flags["F_CONTIGUOUS"] is False
        assert y.flags["C_CONTIGUOUS"] is False
    elif not any(s == 1 for s in x.shape):
        assert x.flags["F_CONTIGUOUS"] == y.flags["F_CONTIGUOUS"]
    assert x.flags["WRITEABLE"] == y.flags["WRITEABLE"] or x.ndim == 0
    assert x.flags["ALIGNED"] == y.flags["ALIGNED"]


def check_meta(x, y):
    assert x.shape == y.shape and x.dtype == y.dtype
    if y.size:
        assert x.strides == y.strides
    check_flags(x, y)


def check_all(x, y):
    check_meta(x, y)
    assert np.array_equal(np.asarray(x), y)


def test_hash_and_bool(ctx):                               # :40-53
    with pytest.raises(TypeError):
        hash(ga.empty((2, 3), context=ctx))
    for data in [np.empty((0, 33)), [[1]], [[0]], [], [0], [1], 0, 1]:
        assert bool(ga.asarray(data, context=ctx)) == bool(np.asarray(data).size and np.asarray(data).any())


@pytest.mark.parametrize("dtype", DTYPES)
def test_transfer(ctx, dtype):                             # :56-75, :94-136
    for shp in SHAPES:
        for offseted in (True, False):
            a, b = gen_gpuarray(shp, dtype, offseted, ctx=ctx)
            c = np.asarray(b)
            assert np.array_equal(np.asarray(b, dtype=dtype), a) and np.array_equal(c, a)
            assert a.shape == b.shape == c.shape and a.strides == b.strides == c.strides
            assert a.dtype == b.dtype == c.dtype == np.dtype(dtype) and c.flags.c_contiguous
    for shp in SHAPES[1:]:
        a = (np.random.default_rng(0).random(shp) * 10).astype(dtype)
        b = ga.array(a, context=ctx)
        ar, br = a[::-1], b[::-1]
        c = np.asarray(br)
        assert np.array_equal(c, ar) and c.flags.c_contiguous
        assert ar.strides == br.strides == (-c.strides[0],) + c.strides[1:]
        af, bf = np.asfortranarray(a), ga.asfortranarray(b)
        cf = np.asarray(bf)
        assert af.strides == bf.strides == cf.strides and cf.flags.f_contiguous
        assert np.array_equal(cf, af)


def test_cast(ctx):                                        # :78-91
    for shp in SHAPES:
        for d1, d2 in itertools.product(DTYPES[:10], repeat=2):
            a, b = gen_gpuarray(shp, d1, False, ctx=ctx)
            ac, bc = a.astype(d2), b.astype(d2)
            assert ac.dtype == bc.dtype and ac.shape == bc.shape
            assert np.array_equal(ac, np.asarray(bc))


@pytest.mark.parametrize("order", ["f", "c"])
@pytest.mark.parametrize("sliced", [1, 2, -1, -2])
def test_ascontiguous_and_asfortran(ctx, sliced, order):   # :139-210
    for shp in SHAPES:
        for dtype in ("float32", "int16", "float64"):
            for off_o, off_i in itertools.product((True, False), repeat=2):
                cpu, gpu = gen_gpuarray(shp, dtype, off_o, off_i, sliced, order, ctx=ctx)
                a, b = np.ascontiguousarray(cpu), ga.ascontiguousarray(gpu)
                if gpu.flags["C_CONTIGUOUS"] and gpu.ndim:
                    assert b is gpu
                else:
                    assert b is not gpu
                assert a.shape == b.shape and a.dtype == b.dtype and b.flags["C_CONTIGUOUS"]
                assert a.strides == b.strides and np.array_equal(np.asarray(b), a)
                a, b = np.asfortranarray(cpu), ga.asfortranarray(gpu)
                if gpu.flags["F_CONTIGUOUS"] and gpu.ndim:
                    assert b is gpu
                else:
                    assert b is not gpu
                assert a.shape == b.shape and a.dtype == b.dtype and b.flags["F_CONTIGUOUS"]
                if not any(s == 1 for s in cpu.shape):
                    assert a.strides == b.strides
                assert np.array_equal(np.asarray(b), a)


@pytest.mark.parametrize("order", ["C", "F"])
def test_zeros_and_empty(ctx, order):                      # :213-270
    for shp in [(), (0,), (5,), (0, 0), (1, 0), (0, 1), (6, 7), (0, 0, 0), (1, 0, 0), (0, 1, 0),
                (0, 0, 1), (4, 8, 9), (1, 8, 9)]:
        for dtype in DTYPES:
            check_all(ga.zeros(shp, dtype, order, context=ctx), np.zeros(shp, dtype, order))
            check_meta(ga.empty(shp, dtype, order, context=ctx), np.empty(shp, dtype, order))
    check_meta(ga.zeros((), context=ctx), np.zeros((), "float32"))
    with pytest.raises(TypeError):
        ga.zeros()
    with pytest.raises(TypeError):
        ga.empty()


def test_getitem_ellipsis_and_none(ctx):                   # :273-308
    rng = np.random.default_rng(3)
    for shp in SHAPES:
        for offseted in (True, False):
            a, g = gen_gpuarray(shp, "float32", offseted, ctx=ctx)
            b = g[...]
            assert b.strides == a.strides and b.shape == a.shape
            assert ga.may_share_memory(b, g) and np.array_equal(np.asarray(b), a)
        a, g = gen_gpuarray(shp, ctx=ctx)
        assert np.array_equal(np.asarray(g[..., None]), a[..., None])
        assert g[..., None].shape == a[..., None].shape
        choices = [0, slice(None), slice(1, None)]
        for _ in range(5):
            idx = tuple(choices[i] for i in rng.integers(0, 3, size=len(shp)))
            idx = idx[:1] + (None,) + idx[1:]
            assert g[idx].shape == a[idx].shape
            assert np.array_equal(np.asarray(g[idx]), a[idx])
        if shp:
            assert np.array_equal(np.asarray(g[1:, None]), a[1:, None])
            assert np.array_equal(np.asarray(g[None]), a[None])


@pytest.mark.parametrize("dtype", ["float32", "int8", "float64", "uint16"])
def test_setitem(ctx, dtype):                              # :311-343
    for shp in [(9,), (8, 9), (4, 8, 9), (1, 8, 9)]:
        for offseted in (True, False):
            a, g = gen_gpuarray(shp, dtype, offseted, ctx=ctx)
            a[...] = 2
            g[...] = 2
            assert np.array_equal(a, np.asarray(g))
            a, g = gen_gpuarray(shp, dtype, offseted, ctx=ctx)
            b, gb = gen_gpuarray(shp[1:], dtype, False, ctx=ctx, rng=np.random.default_rng(1))
            a[:] = b
            g[:] = gb
            assert np.array_equal(a, np.asarray(g))
            a, g = gen_gpuarray(shp, dtype, offseted, ctx=ctx)
            a[0] = b
            g[0] = gb
            assert np.array_equal(a, np.asarray(g))


def test_write_and_read(ctx):                              # :346-398
    cpu, gpu = gen_gpuarray((3, 4, 5), ctx=ctx)
    cpu = cpu.copy()
    cpu[0, 0, 0] = 80
    gpu.write(cpu)
    assert np.array_equal(cpu, np.asarray(gpu))
    cpu[0, 0, 0] = 160
    cpu.setflags(write=False)
    gpu.write(cpu)
    assert np.array_equal(cpu, np.asarray(gpu))
    with pytest.raises(ValueError):
        gpu.write(np.ndarray((2, 4, 5), dtype="float32"))
    with pytest.raises(ValueError):
        gpu.write(np.ndarray((3, 4, 5), dtype="float64"))
    rng = np.random.default_rng(4)
    cpu2 = np.asarray(rng.random((3, 4, 5)), dtype="float32", order="F")
    gpu.write(cpu2)
    assert np.array_equal(cpu2, np.asarray(gpu))
    for order in ("C", "F"):
        cpu2 = np.asarray(rng.random((3, 4, 2, 5)), dtype="float32", order=order)
        gpu.write(cpu2[:, :, 0, :])
        assert np.array_equal(cpu2[:, :, 0, :], np.asarray(gpu))
    out = np.empty((3, 4, 5), dtype="float32")
    gpu.read(out)
    assert np.array_equal(out, np.asarray(gpu))
    ro = np.empty((3, 4, 5), dtype="float32")
    ro.setflags(write=False)
    for bad in (ro, np.empty((2, 4, 5), "float32"), np.empty((3, 4, 5), "float64"),
                np.empty((3, 4, 5), "float32", order="F"),
                np.empty((3, 4, 2, 5), "float32")[:, :, 0, :]):
        with pytest.raises(ValueError):
            gpu.read(bad)


@pytest.mark.parametrize("order1,order2", itertools.product("cf", repeat=2))
def test_copy_view(ctx, order1, order2):                   # :401-457
    for shp in SHAPES[1:]:
        for dtype in ("float32", "int8", "float64"):
            for offseted in (False, True):
                a, b = gen_gpuarray(shp, dtype, offseted, order=order1, ctx=ctx)
                check_flags(b, a)
                for mk_gpu, mk_cpu in ((lambda x: x.copy(order2.upper()), lambda x: x.copy(order2.upper())),
                                       (copy.copy, copy.copy), (lambda x: x.view(), lambda x: x.view()),
                                       (copy.deepcopy, copy.deepcopy),
                                       (lambda x: copy.copy(x.view()), lambda x: copy.copy(x.view()))):
                    c, ac = mk_gpu(b), mk_cpu(a)
                    assert np.array_equal(a, np.asarray(c))
                    check_flags(c, ac)
                    assert np.may_share_memory(a, ac) == ga.may_share_memory(b, c)


SHAPE_PAIRS = [((), (1,)), ((5,), (1, 5)), ((5,), (5, 1)), ((2, 3), (6,)), ((6,), (2, 3)), ((1,), ()),
               ((4,), (-1,)), ((4, 3), (-1,)), ((4, 3), (-1, 3)), ((4, 3), (4, -1)), ((4, 3), (3, -1)),
               ((4, 3), (12, -1)), ((4, 3), (-1, 12)), ((5, 4, 3, 2), (2, -1, 12)), ((4, 2), (2, 2, -1))]


@pytest.mark.parametrize("shps", SHAPE_PAIRS, ids=str)
def test_shape_setter_and_reshape(ctx, shps):              # :460-498
    for offseted in (True, False):
        for order1 in "cf":
            if -1 not in shps[1]:
                ac, ag = gen_gpuarray(shps[0], "float32", offseted, order=order1, ctx=ctx)
                try:
                    ac.shape = shps[1]
                except AttributeError:
                    with pytest.raises(AttributeError):
                        ag.shape = shps[1]
                else:
                    ag.shape = shps[1]
                    assert ac.strides == ag.strides and ac.shape == ag.shape
                    assert np.array_equal(ac, np.asarray(ag))
            for order2 in "acf":
                ac, ag = gen_gpuarray(shps[0], "float32", offseted, order=order1, ctx=ctx)
                outc, outg = ac.reshape(shps[1], order=order2), ag.reshape(shps[1], order=order2)
                assert outc.shape == outg.shape and outc.strides == outg.strides
                assert np.array_equal(outc, np.asarray(outg))


@pytest.mark.parametrize("sliced,newstr", [(1, (4, 4)), (1, (4, 16)), (1, (16, 4)), (1, (16, 8)),
                                           (1, (16, 0)), (-1, (-20, 4)), (-1, (-12, 4))])
def test_strides_setter(ctx, sliced, newstr):              # :501-525
    ac, ag = gen_gpuarray((4, 4), "float32", sliced=sliced, order="c", ctx=ctx)
    try:
        ac.strides = newstr
    except ValueError:
        with pytest.raises(ValueError):
            ag.strides = newstr
        return
    ag.strides = newstr
    check_flags(ag, ac)
    assert np.array_equal(ac, np.asarray(ag))


def test_transpose_interfaces(ctx):                        # :528-589
    for shp in [(2, 3), (4, 8, 9), (1, 2, 3, 4)]:
        for offseted, order, sliced in itertools.product((True, False), "cf", (1, 2, -2, -1)):
            ac, ag = gen_gpuarray(shp, "float32", offseted, sliced=sliced, order=order, ctx=ctx)
            check_all(ag.transpose(), ac.transpose())
            check_all(ag.T, ac.T)
            for perm in itertools.permutations(range(len(shp))):
                check_all(ag.transpose(perm), ac.transpose(perm))
    ac, ag = gen_gpuarray((4, 3, 2), "float32", ctx=ctx)
    check_all(ag.transpose(0, 2, 1), ac.transpose(0, 2, 1))
    with pytest.raises(ValueError):
        ag.transpose(0, 0, 1)


def _cmp(x, y):
    assert isinstance(x, ga.GpuArray)
    check_meta(x, y)
    assert np.array_equal(np.asarray(x), y)


def _cmpf(x, *y):
    with pytest.raises(IndexError):
        x.__getitem__(y)


@pytest.mark.parametrize("dtype", ["float32", "int8", "float64", "uint64"])
@pytest.mark.parametrize("offseted", [True, False])
def test_getitem_w_int(ctx, dtype, offseted):              # :605-672
    a, _a = gen_gpuarray((2,), dtype, offseted, ctx=ctx)
    assert len(_a) == 2
    for k in (Ellipsis, -1, 1, 0, slice(None, None, 1), slice(None, None, -1)):
        _cmp(_a[k], a[k])
    _cmpf(_a, 2)
    a, _a = gen_gpuarray((), dtype, offseted, ctx=ctx)
    _cmp(_a[...], a[...])
    _cmpf(_a, 0)
    _cmpf(_a, slice(1))
    with pytest.raises(TypeError):
        len(_a)
    a, _a = gen_gpuarray((5, 4, 3, 2), dtype, offseted, ctx=ctx)
    _cmpf(_a, slice(-1), slice(-1), 10, -10)
    _cmpf(_a, slice(-1), slice(-1), -10, slice(-1))
    _cmpf(_a, 0, slice(0, -1, -20), -10)
    _cmpf(_a, 10)
    _cmpf(_a, 10, 0, 0, 0)
    _cmpf(_a, -10)
    i64 = np.int64
    for k in (1, -1, i64(1), i64(-1), slice(1, None), slice(1, 2), slice(-1, 1), slice(6, 7),
              (0, 0, slice(None, None, i64(-1)), slice(None, None, -1)),
              (slice(None), slice(None), slice(None, None, i64(-1)), slice(None, None, -1)),
              (slice(None), slice(None), i64(1), -1),
              (slice(None), slice(None), slice(None, None, -10), slice(None, None, -10)),
              (slice(None), slice(None), -1, slice(None)),
              (slice(None), slice(None, None, -2), -1, slice(None)),
              (slice(None), slice(None, None, -20), -1, slice(None)),
              (slice(None), slice(None, None, -2), -1), (0, slice(None, None, -2), -1),
              (-1, -1, -1, -2), Ellipsis):
        _cmp(_a[k], a[k])
    with pytest.raises(NotImplementedError):
        _a[[0, 1]]


def test_flags_object_follows_numpy(ctx):                 # pygpu/gpuarray.pyx:1190-1342
    keys = ["C", "F", "W", "A", "B", "O", "CA", "FA", "FNC", "FORC", "CARRAY", "FARRAY", "FORTRAN",
            "BEHAVED", "OWNDATA", "ALIGNED", "WRITEABLE", "CONTIGUOUS", "C_CONTIGUOUS",
            "F_CONTIGUOUS"]
    base = np.arange(24, dtype="float32").reshape(4, 6)
    for view in (base, base.T, base[::2], base[:, ::2], base[1:2, :], np.asfortranarray(base)):
        g, _ = to_gpu_view(view, ctx)
        own = np.array(view, copy=True, order="K") if False else view
        for k in keys:
            if k in ("O", "OWNDATA"):
                assert g.flags[k] is True          # always, by definition there
                continue
            assert g.flags[k] == own.flags[k], (k, view.strides)
        assert g.flags["U"] is False and g.flags["UPDATEIFCOPY"] is False
        assert g.flags.num == g.ga.flags and g.flags.fortran == g.flags.f_contiguous
        assert g.flags == gpuarray.flags(g.ga.flags) and not (g.flags != gpuarray.flags(g.ga.flags))
        assert g.flags[b"C"] == g.flags.c_contiguous
    with pytest.raises(KeyError):
        g.flags["X"]
    with pytest.raises(KeyError):
        g.flags[3]
    import pickle
    assert pickle.loads(pickle.dumps(g.flags)) == g.flags
    assert "C_CONTIGUOUS" in repr(g.flags) and "UPDATEIFCOPY" in repr(g.flags)


def test_module_interface(ctx):
    assert gpuarray.api_version() == (2, 0) and gpuarray.abi_version() == (3, 0)
    assert gpuarray.count_platforms("hip") == 1 and gpuarray.count_devices("hip", 0) >= 1
    assert gpuarray.dtype_to_ctype(np.dtype("float32")) == "ga_float"
    assert issubclass(gpuarray.UnsupportedException, gpuarray.GpuArrayException)
    # context properties and protocol
    assert ctx.ptr == ctx.ctx.value and len(ctx.unique_id) >= 7 and ":" in ctx.unique_id
    assert ctx.maxlsize1 >= 1 and ctx.maxlsize2 >= 1 and ctx.maxgsize1 >= 1 and ctx.maxgsize2 >= 1
    assert 0 < ctx.largest_memblock <= ctx.total_gmem
    with ctx as c:
        assert c is ctx
    with pytest.raises(RuntimeError):
        ctx.__reduce__()
    # an array over the buffer of another one, by pointer value
    h = np.arange(60, dtype="int32")
    g = gpuarray.array(h, context=ctx)
    v = gpuarray.from_gpudata(g.gpudata, 8, "int32", (4, 5), context=ctx, base=g)
    assert v.base is g and np.array_equal(np.asarray(v), h[2:22].reshape(4, 5))
    v2 = gpuarray.from_gpudata(g.gpudata, 0, "int32", 10, context=ctx, strides=(24,), writable=False,
                               base=g)
    assert np.array_equal(np.asarray(v2), h[::6]) and not v2.flags.writeable
    with pytest.raises(ValueError):
        gpuarray.from_gpudata(g.gpudata, 0, "int32", (2, 2), context=ctx, strides=(4,))
    with pytest.raises(TypeError):
        g.data
    with pytest.raises(TypeError):
        g.base_data


def test_register_dtype_and_use_it(ctx):
    """A caller-defined element type: registered under a C name, usable as the
    element type of arrays and in kernels whose preamble declares it
    (pygpu/gpuarray.pyx:120-158)."""
    pair = np.dtype([("lo", "int32"), ("hi", "int32")])
    tc = gpuarray.register_dtype(pair, "my_pair")
    assert tc >= 512 and gpuarray.dtype_to_typecode(pair) == tc          # user range
    assert gpuarray.typecode_to_dtype(tc) == pair
    h = np.zeros(100, pair)
    h["lo"] = np.arange(100)
    h["hi"] = 7
    g = gpuarray.array(h, context=ctx)
    assert g.dtype == pair and g.itemsize == 8
    back = np.asarray(g.copy())
    assert np.array_equal(back["lo"], h["lo"]) and np.array_equal(back["hi"], h["hi"])
    ew = ga.GpuElemwise(ctx, "o = p.lo + p.hi", [ga.arg("p", pair, read=True),
                                                ga.arg("o", "int32", write=True)],
                        preamble="typedef struct { int lo, hi; } my_pair;")
    out = gpuarray.zeros((100,), "int32", context=ctx)
    ew(g, out)
    assert np.array_equal(np.asarray(out), h["lo"] + 7)


def test_transfer_between_contexts(ctx):
    other = gpuarray.init("hip0")
    h = np.arange(1000, dtype="float32").reshape(10, 100)
    g = gpuarray.array(h, context=ctx)
    t = g.transfer(other)
    assert t.context is other and np.array_equal(np.asarray(t), h)
    f = gpuarray.array(np.asfortranarray(h), context=ctx)
    tf = f.transfer(other)
    assert tf.flags.f_contiguous and np.array_equal(np.asarray(tf), h)
    with pytest.raises(ValueError):
        g[:, ::2].transfer(other)
