"""Reductions over the C ABI with the reference's Python-level rules.

`reduce1` / `sum` / `prod` / `all` / `any` follow pygpu/_array.py:238-294 and
pygpu/reduction.py:294-319: axis may be None, an int or a tuple (negative
values count from the end, out of range raises ValueError); sum/prod keep the
input dtype except that integers narrower than the platform int are widened
to it; all/any give bool; `out` must have exactly the result's shape and
dtype (TypeError otherwise); a 0-d array is returned as a copy.

The reference refuses float16 here (pygpu/reduction.py:156-160); this engine
accepts it and accumulates in float32.  min/max/argmin/argmax/maxandargmax
exist in the reference only as GpuArray_maxandargmax
(src/gpuarray_reduction.c:100-124); their index convention is the same.
"""
import builtins as _b
import ctypes as C

import numpy as np

from . import _lib
from ._lib import lib, check
from . import gpuarray
from .gpuarray import GpuArray, dtype_to_typecode

_OPS = {
    "sum": _lib.GA_REDUCE_SUM, "prod": _lib.GA_REDUCE_PROD, "prodnz": _lib.GA_REDUCE_PRODNZ,
    "min": _lib.GA_REDUCE_MIN, "max": _lib.GA_REDUCE_MAX,
    "argmin": _lib.GA_REDUCE_ARGMIN, "argmax": _lib.GA_REDUCE_ARGMAX,
    "minandargmin": _lib.GA_REDUCE_MINANDARGMIN, "maxandargmax": _lib.GA_REDUCE_MAXANDARGMAX,
    "and": _lib.GA_REDUCE_AND, "or": _lib.GA_REDUCE_OR, "xor": _lib.GA_REDUCE_XOR,
    "all": _lib.GA_REDUCE_ALL, "any": _lib.GA_REDUCE_ANY,
}


class GpuReduction(object):
    """One reduction operator for one source dtype (GpuReduction_new/_call/_free)."""

    def __init__(self, context, op, dtype, ndf=0, ndr=0):
        self.context = context
        self.op = op
        self.dtype = np.dtype(dtype)
        self.gr = C.c_void_p()
        check(lib.GpuReduction_new(C.byref(self.gr), context.ctx, _OPS[op], ndf, ndr,
                                   dtype_to_typecode(dtype), 0), context.ctx)

    def __del__(self):
        gr = getattr(self, "gr", None)
        if gr:
            lib.GpuReduction_free(gr)
            self.gr = None

    def __call__(self, src, axes, d0=None, d1=None):
        axes = list(axes)
        arr = (C.c_int * _b.max(len(axes), 1))(*axes)
        check(lib.GpuReduction_call(self.gr, d0._ptr() if d0 is not None else None,
                                    d1._ptr() if d1 is not None else None, src._ptr(),
                                    len(axes), arr, 0), self.context.ctx)


_cache = {}


def _operator(context, op, dtype):
    key = (id(context), op, np.dtype(dtype).str)
    r = _cache.get(key)
    if r is None or r.context is not context:
        r = _cache[key] = GpuReduction(context, op, dtype)
    return r


def _normalize_axes(ndim, axis):
    """reference pygpu/reduction.py:294-309"""
    if axis is None:
        return list(range(ndim))
    if not isinstance(axis, (list, tuple)):
        axis = (axis,)
    axes = []
    for ax in axis:
        ax = int(ax)
        if ax < 0:
            ax += ndim
        if ax < 0 or ax >= ndim:
            raise ValueError("axis out of bounds")
        if ax not in axes:
            axes.append(ax)
    return axes


def _out_shape(shape, axes):
    return tuple(d for i, d in enumerate(shape) if i not in axes)


def _upcast(dtype):
    """sum/prod result type (reference pygpu/_array.py:250-262,282-293)."""
    dtype = np.dtype(dtype)
    if dtype.kind == "i" and np.dtype("int").itemsize > dtype.itemsize:
        return np.dtype("int")
    if dtype.kind == "u" and np.dtype("uint").itemsize > dtype.itemsize:
        return np.dtype("uint")
    if dtype.kind == "b":
        return np.dtype("int")   # numpy sums booleans as platform ints
    return dtype


def reduce1(ary, op, out_type, axis=None, out=None):
    """Value reduction `op` of `ary` over `axis` into dtype `out_type`."""
    out_type = np.dtype(out_type)
    if ary.ndim == 0:
        res = ary.astype(out_type) if out_type != ary.dtype else ary.copy()
        return res
    axes = _normalize_axes(ary.ndim, axis)
    oshape = _out_shape(ary.shape, axes)
    if out is None:
        out = gpuarray.empty(oshape, dtype=out_type, context=ary.context, cls=type(ary))
    elif out.shape != oshape or out.dtype != out_type:
        raise TypeError("Out array is not of expected type (expected %s %s, got %s %s)" % (
            oshape, out_type, out.shape, out.dtype))
    _operator(ary.context, op, ary.dtype)(ary, axes, d0=out)
    return out


def sum(ary, axis=None, dtype=None, out=None):
    return reduce1(ary, "sum", _upcast(ary.dtype) if dtype is None else dtype, axis, out)


def prod(ary, axis=None, dtype=None, out=None):
    return reduce1(ary, "prod", _upcast(ary.dtype) if dtype is None else dtype, axis, out)


def all(ary, axis=None, out=None):
    return reduce1(ary, "all", np.dtype("bool"), axis, out)


def any(ary, axis=None, out=None):
    return reduce1(ary, "any", np.dtype("bool"), axis, out)


def max(ary, axis=None, out=None):
    return reduce1(ary, "max", ary.dtype, axis, out)


def min(ary, axis=None, out=None):
    return reduce1(ary, "min", ary.dtype, axis, out)


def _arg_reduce(ary, op, axis, want_value):
    axes = _normalize_axes(ary.ndim, axis)
    oshape = _out_shape(ary.shape, axes)
    idx = gpuarray.empty(oshape, dtype="int64", context=ary.context, cls=type(ary))
    val = gpuarray.empty(oshape, dtype=ary.dtype, context=ary.context, cls=type(ary)) \
        if want_value else None
    _operator(ary.context, op, ary.dtype)(ary, axes, d0=val, d1=idx)
    return (val, idx) if want_value else idx


def argmax(ary, axis=None):
    return _arg_reduce(ary, "argmax", axis, False)


def argmin(ary, axis=None):
    return _arg_reduce(ary, "argmin", axis, False)


def maxandargmax(ary, axis=None):
    return _arg_reduce(ary, "maxandargmax", axis, True)


def minandargmin(ary, axis=None):
    return _arg_reduce(ary, "minandargmin", axis, True)


def maxandargmax_c(src, axes, dst_max=None, dst_argmax=None):
    """Straight call of the reference's C entry point GpuArray_maxandargmax."""
    axes = list(axes)
    oshape = _out_shape(src.shape, axes)
    if dst_max is None:
        dst_max = gpuarray.empty(oshape, dtype=src.dtype, context=src.context)
    if dst_argmax is None:
        dst_argmax = gpuarray.empty(oshape, dtype="uint64", context=src.context)
    arr = (C.c_uint * len(axes))(*axes)
    check(lib.GpuArray_maxandargmax(dst_max._ptr(), dst_argmax._ptr(), src._ptr(), len(axes), arr),
          src.context.ctx)
    return dst_max, dst_argmax
