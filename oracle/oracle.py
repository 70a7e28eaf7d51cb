"""numpy-facing wrappers over liboracle.so (ga_oracle.c).

TEST INFRASTRUCTURE ONLY: the CPU restatement of what the reference computes
on this path.  Each wrapper names the reference code its C function follows.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")


def build(force=False):
    src = os.path.join(_HERE, "ga_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "liboracle.so"])
    return _SO


def _load():
    if not os.path.exists(_SO):
        build()
    L = C.CDLL(_SO)
    L.orc_pcg_fill_f32.argtypes = [C.c_void_p, C.c_size_t, C.c_uint64]
    L.orc_float2half.restype = C.c_uint16
    L.orc_float2half.argtypes = [C.c_float]
    L.orc_float2half_rte.restype = C.c_uint16
    L.orc_float2half_rte.argtypes = [C.c_float]
    L.orc_half2float.restype = C.c_float
    L.orc_half2float.argtypes = [C.c_uint16]
    L.orc_elemwise_contig_muladd.argtypes = [C.c_size_t, C.c_void_p, C.c_void_p, C.c_void_p]
    L.orc_sched.argtypes = [C.c_size_t, C.c_size_t, C.c_size_t, C.c_uint, C.c_size_t,
                            C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
    PS, PSS = C.POINTER(C.c_size_t), C.POINTER(C.c_ssize_t)
    L.orc_collapse.argtypes = [C.c_uint, C.POINTER(C.c_uint), PS, C.POINTER(PSS)]
    L.orc_check_basic.argtypes = [C.c_uint, C.POINTER(C.c_uint), C.POINTER(PS), C.POINTER(PSS), PS,
                                  C.POINTER(C.c_int), C.c_int, C.c_uint, C.POINTER(C.c_uint), PS,
                                  PSS, PS, C.POINTER(C.c_int)]
    L.orc_elemwise.argtypes = [C.c_int, C.c_size_t, C.c_uint, PS, C.c_uint,
                               C.POINTER(C.c_void_p), PSS, C.c_void_p]
    L.orc_maxandargmax.argtypes = [C.c_void_p, C.c_int, C.c_uint, PS, PSS, C.c_uint,
                                   C.POINTER(C.c_uint), C.c_void_p, PSS, C.c_void_p, PSS]
    L.orc_reduk.argtypes = [C.c_int, C.c_void_p, C.c_int, C.c_uint, PS, PSS, C.POINTER(C.c_int),
                            C.c_void_p, C.c_int, C.c_size_t]
    L.orc_reduk_map2.argtypes = [C.c_int, C.c_int, C.c_int, C.c_uint, PS, C.c_void_p, PSS, C.c_void_p,
                                 PSS, C.c_double, C.POINTER(C.c_int), C.c_void_p, C.c_size_t]
    L.orc_take1.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_uint, PS, PSS, C.c_void_p,
                            C.c_int, C.c_size_t, C.POINTER(C.c_int)]
    return L


_L = _load()

# expression ids of orc_elemwise
MULADD_HALF_F32, A_PLUS_BC_F32, ADD_U32, ADD_F16, AXPB_U32, SAXPY_I32_F32, COPY_F32, \
    COPY_F16_F32, COPY_I32_I64 = range(9)


def pcg_fill_f32(n, seed=1):
    """Test data of tests/check_reduction.c:32-63,103-106 (PCG32, pcgRand01)."""
    out = np.empty(n, dtype=np.float32)
    _L.orc_pcg_fill_f32(out.ctypes.data, n, seed)
    return out


def float2half(f):
    """Host conversion, src/gpuarray/util.h:107-183."""
    return _L.orc_float2half(C.c_float(f))


def float2half_rte(f):
    return _L.orc_float2half_rte(C.c_float(f))


def half2float(h):
    return _L.orc_half2float(h)


def collapse(dims, strs):
    """src/gpuarray_util.c:153-188.  strs: list of stride lists (None = scalar).
    Returns (nd, dims, strs)."""
    nd = C.c_uint(len(dims))
    d = (C.c_size_t * max(len(dims), 1))(*dims)
    rows = []
    ptrs = (C.POINTER(C.c_ssize_t) * max(len(strs), 1))()
    for k, s in enumerate(strs):
        if s is None:
            rows.append(None)
            ptrs[k] = None
        else:
            r = (C.c_ssize_t * max(len(s), 1))(*s)
            rows.append(r)
            ptrs[k] = C.cast(r, C.POINTER(C.c_ssize_t))
    _L.orc_collapse(len(strs), C.byref(nd), d, ptrs)
    n = nd.value
    return n, tuple(d[i] for i in range(n)), tuple(
        None if r is None else tuple(r[i] for i in range(n)) for r in rows)


def check_basic(arrays, is_out, flags):
    """src/gpuarray_elemwise.c:272-383 on numpy views.  Returns
    (err, nd, dims, strs, n, call32)."""
    narr = len(arrays)
    maxnd = max([a.ndim for a in arrays] + [1])
    and_ = (C.c_uint * narr)(*[a.ndim for a in arrays])
    dl = [(C.c_size_t * max(a.ndim, 1))(*a.shape) for a in arrays]
    sl = [(C.c_ssize_t * max(a.ndim, 1))(*a.strides) for a in arrays]
    ad = (C.POINTER(C.c_size_t) * narr)(*[C.cast(x, C.POINTER(C.c_size_t)) for x in dl])
    as_ = (C.POINTER(C.c_ssize_t) * narr)(*[C.cast(x, C.POINTER(C.c_ssize_t)) for x in sl])
    aoff = (C.c_size_t * narr)(*([0] * narr))
    io = (C.c_int * narr)(*[1 if o else 0 for o in is_out])
    nd = C.c_uint(0)
    dims = (C.c_size_t * maxnd)()
    strs = (C.c_ssize_t * (narr * maxnd))()
    n = C.c_size_t(0)
    c32 = C.c_int(0)
    err = _L.orc_check_basic(narr, and_, ad, as_, aoff, io, flags, maxnd, C.byref(nd), dims, strs,
                             C.byref(n), C.byref(c32))
    if err:
        return err, None, None, None, None, None
    k = nd.value
    return (0, k, tuple(dims[i] for i in range(k)),
            tuple(tuple(strs[a * maxnd + i] for i in range(k)) for a in range(narr)), n.value,
            c32.value)


def elemwise(expr, arrays, is_out, flags=0x100 | 0x400, scalar=None):
    """Plan with check_basic, then run the reference's strided kernel body
    (src/gpuarray_elemwise.c:198-238) over numpy views, writing in place.
    Returns the reference's error code (0 or 2)."""
    err, nd, dims, strs, n, _ = check_basic(arrays, is_out, flags)
    if err:
        return err
    if n == 0:
        return 0
    narr = len(arrays)
    base = (C.c_void_p * narr)(*[a.ctypes.data for a in arrays])
    flat = (C.c_ssize_t * (narr * max(nd, 1)))()
    for a in range(narr):
        for i in range(nd):
            flat[a * nd + i] = strs[a][i]
    d = (C.c_size_t * max(nd, 1))(*dims)
    sc = None
    if scalar is not None:
        sc = np.ascontiguousarray(scalar)
    r = _L.orc_elemwise(expr, n, nd, d, narr, base, flat,
                        None if sc is None else C.c_void_p(sc.ctypes.data))
    return r


def elemwise_contig_muladd(a, b, c):
    """Flat kernel for c = a*b + 0.5f (src/gpuarray_elemwise.c:472-532)."""
    _L.orc_elemwise_contig_muladd(a.size, a.ctypes.data, b.ctypes.data, c.ctypes.data)


def sched(n, max_l=1024, min_l=64, numprocs=256, max_g=2147483647, gs=0, ls=0):
    """GpuKernel_sched, src/gpuarray_kernel.c:38-89."""
    g, l = C.c_size_t(gs), C.c_size_t(ls)
    _L.orc_sched(n, max_l, min_l, numprocs, max_g, C.byref(g), C.byref(l))
    return g.value, l.value


_ET = {np.dtype("float32"): 0, np.dtype("float64"): 1, np.dtype("int32"): 2,
       np.dtype("float16"): 3, np.dtype("int64"): 4, np.dtype("uint8"): 5,
       np.dtype("bool"): 5}


def maxandargmax(src, redux):
    """src/gpuarray_reduction.c:545-607 on a numpy view (float32/float64/int32/
    float16).  Returns (max, argmax) as dense arrays; argmax is int64."""
    redux = list(redux)
    et = _ET[src.dtype]
    if et > 3:
        raise ValueError("unsupported dtype for the maxandargmax checker")
    oshape = tuple(d for i, d in enumerate(src.shape) if i not in redux)
    dmax = np.empty(oshape, dtype=src.dtype)
    darg = np.empty(oshape, dtype=np.int64)
    nd = src.ndim
    dims = (C.c_size_t * nd)(*src.shape)
    strs = (C.c_ssize_t * nd)(*src.strides)
    rl = (C.c_uint * len(redux))(*redux)
    ms = (C.c_ssize_t * max(len(oshape), 1))(*dmax.strides)
    as_ = (C.c_ssize_t * max(len(oshape), 1))(*darg.strides)
    err = _L.orc_maxandargmax(C.c_void_p(src.ctypes.data), et, nd, dims, strs, len(redux), rl,
                              C.c_void_p(dmax.ctypes.data), ms, C.c_void_p(darg.ctypes.data), as_)
    if err:
        raise ValueError("orc_maxandargmax: error %d" % err)
    return dmax, darg


def reduk(op, src, axes, out_dtype, ls=256):
    """pygpu/reduction.py:33-134 with a work-group of `ls` lanes.
    op in {"sum","prod","all","any"}."""
    opid = {"sum": 0, "prod": 1, "all": 2, "any": 3}[op]
    out_dtype = np.dtype(out_dtype)
    nd = src.ndim
    axes = [a % nd for a in axes]
    redux = (C.c_int * nd)(*[1 if i in axes else 0 for i in range(nd)])
    oshape = tuple(d for i, d in enumerate(src.shape) if i not in axes)
    out = np.empty(oshape, dtype=out_dtype)
    dims = (C.c_size_t * nd)(*src.shape)
    strs = (C.c_ssize_t * nd)(*src.strides)
    err = _L.orc_reduk(opid, C.c_void_p(src.ctypes.data), _ET[src.dtype], nd, dims, strs, redux,
                       C.c_void_p(out.ctypes.data), _ET[out_dtype], ls)
    if err:
        raise ValueError("orc_reduk: error %d" % err)
    return out


def check_args(shapes, strides, collapse=False, broadcast=False):
    """The Python-level argument check, pygpu/tools.py:68-168, on plain
    shape/stride tuples (None = scalar).  Returns (n, nd, dims, strs).
    Differences from the C check (src/gpuarray_elemwise.c:272-383): there is no
    output, so with `broadcast` the iteration space is the union shape; and a
    size-1 dim keeps its stride unless it is actually stretched."""
    strs, dims, n, nd = [], None, None, None
    for shp, st in zip(shapes, strides):
        if shp is None:
            strs.append(None)
            continue
        strs.append(list(st))
        if dims is None:
            nd, dims = len(shp), list(shp)
            n = 1
            for d in shp:
                n *= d
        else:
            if len(shp) != nd:
                raise ValueError("Array order differs")
            if not broadcast and list(shp) != dims:
                raise ValueError("Array shape differs")
    if dims is None:
        raise TypeError("No arrays in kernel arguments, something is wrong")
    if broadcast:
        if 1 in dims:
            for shp in shapes:
                if shp is None:
                    continue
                for i, d in enumerate(shp):
                    if dims[i] != d and dims[i] == 1:
                        dims[i] = d
                        n *= d
        for k, shp in enumerate(shapes):
            if shp is None or list(shp) == dims:
                continue
            for j, d in enumerate(shp):
                if dims[j] != d:
                    if d == 1:
                        strs[k][j] = 0
                    else:
                        raise ValueError("Array shape differs")
    if collapse and nd > 1:
        for i in range(nd - 1, -1, -1):
            if nd > 1 and dims[i] == 1:
                del dims[i]
                for st in strs:
                    if st is not None:
                        del st[i]
                nd -= 1
        for i in range(nd - 1, 0, -1):
            if all(st is None or st[i] * dims[i] == st[i - 1] for st in strs):
                dims[i - 1] *= dims[i]
                del dims[i]
                for st in strs:
                    if st is not None:
                        st[i - 1] = st[i]
                        del st[i]
                nd -= 1
    return n, nd, tuple(dims), tuple(None if st is None else tuple(st) for st in strs)


def take1(v, ind, out=None):
    """GpuArray_take1 (src/gpuarray_array.c:325-548) on host arrays: returns
    (rows, err) where err is -1 when some index was out of range (those rows
    keep the content of `out`, or zeros)."""
    ind = np.ascontiguousarray(ind)
    n0 = ind.shape[0]
    if out is None:
        out = np.zeros((n0,) + v.shape[1:], dtype=v.dtype)
    assert out.flags.c_contiguous and out.dtype == v.dtype
    nd = v.ndim
    dims = (C.c_size_t * nd)(*v.shape)
    strs = (C.c_ssize_t * nd)(*v.strides)
    kind = ind.dtype.itemsize * (-1 if ind.dtype.kind == "i" else 1)
    err = C.c_int(0)
    rc = _L.orc_take1(C.c_void_p(out.ctypes.data), C.c_void_p(v.ctypes.data), v.dtype.itemsize, nd,
                      dims, strs, C.c_void_p(ind.ctypes.data), kind, n0, C.byref(err))
    if rc:
        raise ValueError("orc_take1: error %d" % rc)
    return out, err.value


MAP_MUL, MAP_ABSDIFF, MAP_SAXPY, MAP_SQUARE = range(4)
RED_ADD, RED_MAX = range(2)


def reduk_map2(map_id, red_id, a, b, s, axes, ls=256):
    """pygpu/reduction.py:33-134 with map_expr over arrays a, b (broadcast
    against each other, pygpu/tools.py check_args) and scalar s; float32 or
    float64 throughout."""
    assert a.dtype == b.dtype and a.dtype in (np.float32, np.float64) and a.ndim == b.ndim
    nd = a.ndim
    shape = tuple(max(x, y) for x, y in zip(a.shape, b.shape))
    astr = [st if d == full else 0 for st, d, full in zip(a.strides, a.shape, shape)]
    bstr = [st if d == full else 0 for st, d, full in zip(b.strides, b.shape, shape)]
    axes = [x % nd for x in axes]
    redux = (C.c_int * nd)(*[1 if i in axes else 0 for i in range(nd)])
    oshape = tuple(d for i, d in enumerate(shape) if i not in axes)
    out = np.empty(oshape, dtype=a.dtype)
    rc = _L.orc_reduk_map2(map_id, red_id, 0 if a.dtype == np.float32 else 1, nd,
                           (C.c_size_t * nd)(*shape), C.c_void_p(a.ctypes.data),
                           (C.c_ssize_t * nd)(*astr), C.c_void_p(b.ctypes.data),
                           (C.c_ssize_t * nd)(*bstr), float(s), redux,
                           C.c_void_p(out.ctypes.data), ls)
    if rc:
        raise ValueError("orc_reduk_map2: error %d" % rc)
    return out
