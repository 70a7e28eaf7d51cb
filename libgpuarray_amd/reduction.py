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
import re

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
        self._axes = {}
        check(lib.GpuReduction_new(C.byref(self.gr), context.ctx, _OPS[op], ndf, ndr,
                                   dtype_to_typecode(dtype), 0), context.ctx)

    def __del__(self):
        gr = getattr(self, "gr", None)
        if gr:
            lib.GpuReduction_free(gr)
            self.gr = None

    def __call__(self, src, axes, d0=None, d1=None, noalloc=False):
        """noalloc=True goes through GpuReduction_call_noalloc: partials in the
        library's static device array, no allocation on the way."""
        key = tuple(axes)
        arr = self._axes.get(key)
        if arr is None:            # the C array of an axis list, built once
            arr = self._axes[key] = (C.c_int * _b.max(len(key), 1))(*key)
        fn = lib.GpuReduction_call_noalloc if noalloc else lib.GpuReduction_call
        err = fn(self.gr, d0._ref if d0 is not None else None,
                 d1._ref if d1 is not None else None, src._ref, len(key), arr, 0)
        if err:
            check(err, self.context.ctx)


from .tools import Argument, ArrayArg, ScalarArg, as_argument  # noqa: E402,F401
from .dtypes import parse_c_arg_backend  # noqa: E402


_INDEX_RE = re.compile(r"([a-zA-Z_][a-zA-Z0-9_]*)\[i\]")


def parse_c_args(arguments):
    """"float *a, float *b, float s" -> (ArrayArg, ArrayArg, ScalarArg)
    (reference pygpu/reduction.py:13-15)."""
    return tuple(parse_c_arg_backend(c_arg.replace("GLOBAL_MEM", ""), ScalarArg, ArrayArg)
                 for c_arg in arguments.split(","))


def massage_op(operation):
    """`a[i]` -> `a[0]` for every indexed name (reference pygpu/reduction.py:21-22)."""
    return _INDEX_RE.sub(r"\g<1>[0]", operation)


def _ceil_log2(x):
    """Exponent of the nearest power of two at or above x (reference pygpu/reduction.py:25-30)."""
    return int(x - 1).bit_length() if x > 0 else 0


class ReductionKernel(object):
    """reference pygpu/reduction.py:137-291: `reduce_expr` (in a and b) folds
    the values of `map_expr` (arrays written `name[i]`) over the axes flagged
    in `redux`, starting from `neutral`, accumulating in `dtype_out`.  One
    pass over the inputs: the expression is evaluated inside the reduction
    kernel.  Differences: float16 is accepted (accumulated in float32; the
    reference raises NotImplementedError, :156-160) and nothing limits the
    number of outputs (:256-258)."""

    def __init__(self, context, dtype_out, neutral, reduce_expr, redux, map_expr=None,
                 arguments=None, preamble="", init_nd=None):
        self.context = context
        self.neutral = neutral
        self.redux = tuple(redux)
        if not _b.any(self.redux):
            raise ValueError("Reduction is along no axes")
        self.dtype_out = np.dtype(dtype_out)
        if isinstance(arguments, str):
            self.arguments = parse_c_args(arguments)
        elif arguments is None:
            self.arguments = [ArrayArg(self.dtype_out, "_reduce_input")]
        else:
            self.arguments = list(arguments)
        self.reduce_expr = reduce_expr
        if map_expr is None:
            if len(self.arguments) != 1:
                raise ValueError("Don't know what to do with more than one argument. "
                                 "Specify map_expr to explicitly state what you want.")
            self.operation = "%s[i]" % (self.arguments[0].name,)
        else:
            self.operation = map_expr
        if not _b.any(a.isarray() for a in self.arguments):
            raise ValueError("ReductionKernel can only be used with functions that have at "
                             "least one vector argument.")
        self.preamble = preamble
        # arrays are named by their element in the C interface
        expr = _INDEX_RE.sub(r"\g<1>", self.operation)
        self._op = MapReduction(context, "custom", self.dtype_out, expr, self.arguments,
                                preamble=preamble, reduce_expr=str(reduce_expr),
                                neutral=str(neutral))

    def __call__(self, *args, **kwargs):
        broadcast = kwargs.pop("broadcast", None)
        out = kwargs.pop("out", None)
        if len(kwargs) != 0:
            raise TypeError("Unexpected keyword argument: %s" % list(kwargs.keys())[0])
        if len(args) != len(self.arguments):
            raise TypeError("Expected %d arguments, got %d" % (len(self.arguments), len(args)))
        arrays = [a for a, d in zip(args, self.arguments) if d.isarray()]
        for a in arrays:
            if not isinstance(a, GpuArray):
                raise TypeError("array argument expected, got %r" % (type(a),))
            if a.ndim != len(self.redux):
                raise ValueError("Array has %d dimensions, the kernel reduces over %d" % (
                    a.ndim, len(self.redux)))
        dims = _common_shape(arrays, broadcast)
        out_shape = tuple(d for i, d in enumerate(dims) if not self.redux[i])
        if out is None:
            out = gpuarray.empty(out_shape, dtype=self.dtype_out, context=self.context)
        elif out.shape != out_shape or out.dtype != self.dtype_out:
            raise TypeError("Out array is not of expected type (expected %s %s, got %s %s)" % (
                out_shape, self.dtype_out, out.shape, out.dtype))
        axes = [i for i, r in enumerate(self.redux) if r]
        self._op(args, axes, d0=out, broadcast=bool(broadcast))
        return out


def _common_shape(arrays, broadcast):
    """reference pygpu/tools.py check_args with collapse=False"""
    dims = list(arrays[0].shape)
    for a in arrays[1:]:
        if a.ndim != len(dims):
            raise ValueError("Arrays have %d and %d dimensions" % (len(dims), a.ndim))
        for i, d in enumerate(a.shape):
            if d != dims[i]:
                if broadcast and dims[i] == 1:
                    dims[i] = d
                elif not (broadcast and d == 1):
                    raise ValueError("Array shape mismatch on dimension %d: %d vs %d" % (
                        i, d, dims[i]))
    return dims


class MapReduction(object):
    """GpuReduction_new_map / GpuReduction_call_map: operation `op` (a name of
    the table above, or "custom" with `reduce_expr` in a and b and its
    `neutral`) over the values of `map_expr`, an expression in the names of
    `arguments` (ArrayArg / ScalarArg), evaluated in the reduction kernel and
    accumulated in `acc_dtype`."""

    def __init__(self, context, op, acc_dtype, map_expr, arguments, preamble="",
                 reduce_expr=None, neutral=None):
        self.context = context
        self.arguments = list(arguments)
        self.acc_dtype = np.dtype(acc_dtype)
        n = len(self.arguments)
        self._names = [a.name.encode() for a in self.arguments]
        self._descr = (_lib.ElemwiseArg * _b.max(n, 1))()
        for i, a in enumerate(self.arguments):
            self._descr[i].name = self._names[i]
            self._descr[i].typecode = dtype_to_typecode(a.dtype)
            self._descr[i].flags = _lib.GE_READ | (0 if a.isarray() else _lib.GE_SCALAR)
        opid = _lib.GA_REDUCE_CUSTOM if op == "custom" else _OPS[op]
        self.gr = C.c_void_p()
        check(lib.GpuReduction_new_map(
            C.byref(self.gr), context.ctx, opid,
            reduce_expr.encode() if reduce_expr is not None else None,
            neutral.encode() if neutral is not None else None,
            dtype_to_typecode(self.acc_dtype), preamble.encode(), map_expr.encode(), n,
            C.cast(self._descr, C.c_void_p), 0), context.ctx)

    def __del__(self):
        gr = getattr(self, "gr", None)
        if gr:
            lib.GpuReduction_free(gr)
            self.gr = None

    def __call__(self, args, axes, d0=None, d1=None, broadcast=False):
        keep = []
        ptrs = (C.c_void_p * _b.max(len(args), 1))()
        for i, (a, d) in enumerate(zip(args, self.arguments)):
            if d.isarray():
                ptrs[i] = C.cast(a._ptr(), C.c_void_p)
            else:
                v = np.asarray(a, dtype=d.dtype).reshape(1).copy()
                keep.append(v)
                ptrs[i] = v.ctypes.data
        axes = list(axes)
        arr = (C.c_int * _b.max(len(axes), 1))(*axes)
        check(lib.GpuReduction_call_map(self.gr, d0._ptr() if d0 is not None else None,
                                        d1._ptr() if d1 is not None else None, ptrs, len(axes),
                                        arr, _lib.GE_BROADCAST if broadcast else 0),
              self.context.ctx)


def _operator(context, op, dtype):
    """The GpuReduction for (op, dtype), kept on the context object itself (as
    the elementwise helpers keep theirs), so that dropping the context frees
    the operators and, with them, the context's device memory."""
    cache = context.__dict__.setdefault("_reduction_cache", {})
    key = (op, np.dtype(dtype).str)
    r = cache.get(key)
    if r is None:
        r = cache[key] = GpuReduction(context, op, dtype)
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


# (C operator, neutral) pairs of the reference's reduce1 callers
# (pygpu/_array.py:238-294) and the built-in operation each one is
_BUILTIN = {("+", "0"): "sum", ("*", "1"): "prod", ("&&", "1"): "all", ("||", "0"): "any",
            ("&", "-1"): "and", ("|", "0"): "or", ("^", "0"): "xor"}


def reduce1(ary, op, neutral, out_type, axis=None, out=None, oper=None):
    """reference pygpu/reduction.py:294-319: reduce `ary` over `axis` with the
    C binary operator `op` (or the expression `oper` in a and b) from
    `neutral`, accumulating in `out_type`.  The operator/neutral pairs the
    reference's own callers use run the built-in operations; anything else
    goes through ReductionKernel."""
    name = _BUILTIN.get((op, str(neutral).strip())) if oper is None else None
    if name in ("all", "any") and np.dtype(out_type) != np.dtype("bool"):
        name = None
    if name is not None:
        return _reduce_named(ary, name, out_type, axis, out)
    if ary.ndim == 0:
        return ary.astype(out_type) if np.dtype(out_type) != ary.dtype else ary.copy()
    axes = _normalize_axes(ary.ndim, axis)
    redux = [i in axes for i in range(ary.ndim)]
    r = ReductionKernel(ary.context, dtype_out=out_type, neutral=neutral,
                        reduce_expr=oper if oper is not None else "a %s b" % (op,), redux=redux,
                        arguments=[ArrayArg(ary.dtype, "a")])
    return r(ary, out=out)


def _reduce_named(ary, op, out_type, axis=None, out=None):
    """Built-in value reduction `op` of `ary` over `axis` into dtype `out_type`."""
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
    return _reduce_named(ary, "sum", _upcast(ary.dtype) if dtype is None else dtype, axis, out)


def prod(ary, axis=None, dtype=None, out=None):
    return _reduce_named(ary, "prod", _upcast(ary.dtype) if dtype is None else dtype, axis, out)


def all(ary, axis=None, out=None):
    return _reduce_named(ary, "all", np.dtype("bool"), axis, out)


def any(ary, axis=None, out=None):
    return _reduce_named(ary, "any", np.dtype("bool"), axis, out)


def max(ary, axis=None, out=None):
    return _reduce_named(ary, "max", ary.dtype, axis, out)


def min(ary, axis=None, out=None):
    return _reduce_named(ary, "min", ary.dtype, axis, out)


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
