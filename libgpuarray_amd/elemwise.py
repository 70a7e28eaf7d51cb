"""GpuElemwise over the C ABI, shaped like the reference's Python binding
(pygpu/_elemwise.pyx:51-221: `arg`, `GpuElemwise.__call__` with
broadcast=True / padshape=True defaults) and its helpers
(pygpu/elemwise.py:24-102: elemwise1 / elemwise2 / compare).
"""
import ctypes as C

import numpy as np

from . import _lib
from ._lib import lib, check, ElemwiseArg
from . import gpuarray
from .gpuarray import GpuArray, dtype_to_typecode
from .dtypes import dtype_to_ctype, get_common_dtype


class arg(object):
    """Argument descriptor (reference pygpu/_elemwise.pyx:51-94)."""

    def __init__(self, name, type, read=False, write=False, scalar=False):
        self.name = name
        self.dtype = np.dtype(type)
        self.read, self.write, self.scalar = bool(read), bool(write), bool(scalar)
        if scalar:
            self.read, self.write = True, False
        if not (self.read or self.write):
            raise ValueError("no flags specified for arg %s" % (name,))

    @property
    def flags(self):
        fl = 0
        if self.scalar:
            fl |= _lib.GE_SCALAR
        if self.read:
            fl |= _lib.GE_READ
        if self.write:
            fl |= _lib.GE_WRITE
        return fl


class GpuElemwise(object):
    """expr applied elementwise (reference pygpu/_elemwise.pyx:97-221)."""

    def __init__(self, context, expr, args, nd=0, preamble="", convert_f16=False):
        self.context = context
        self.args = list(args)
        self._names = [a.name.encode() for a in self.args]
        n = len(self.args)
        arr = (ElemwiseArg * max(n, 1))()
        for i, a in enumerate(self.args):
            arr[i].name = self._names[i]
            arr[i].typecode = dtype_to_typecode(a.dtype)
            arr[i].flags = a.flags
        flags = _lib.GE_CONVERT_F16 if convert_f16 else 0
        self.ge = lib.GpuElemwise_new(context.ctx, preamble.encode(), expr.encode(), n, arr, nd,
                                      flags)
        # argument table of a call, reused: array slots take the address of the
        # caller's GpuArray struct, scalar slots point at a value held here
        self._ptrs = (C.c_void_p * max(n, 1))()
        self._scalars = {}
        for i, a in enumerate(self.args):
            if a.scalar:
                buf = np.zeros((), dtype=a.dtype)
                self._scalars[i] = buf
                self._ptrs[i] = buf.ctypes.data
        self._slots = [(i, a.scalar, a.name) for i, a in enumerate(self.args)]
        if not self.ge:
            # the code is in the context's record; surface it like any other failure
            msg = context.error()
            raise _lib.GpuArrayException("Could not initialize C GpuElemwise instance: " + msg,
                                         _lib.GA_IMPL_ERROR)

    def __del__(self):
        ge = getattr(self, "ge", None)
        if ge:
            lib.GpuElemwise_free(ge)
            self.ge = None

    def __call__(self, *values, **kwargs):
        flags = _lib.GE_BROADCAST | _lib.GE_PADSHAPE
        if kwargs:
            if not kwargs.pop("broadcast", True):
                flags &= ~_lib.GE_BROADCAST
            if not kwargs.pop("padshape", True):
                flags &= ~_lib.GE_PADSHAPE
            if not kwargs.pop("collapse", True):
                flags |= _lib.GE_NOCOLLAPSE
            if kwargs:
                raise TypeError("unexpected keyword arguments: %s" % (sorted(kwargs),))
        if len(values) != len(self._slots):
            raise TypeError("expected %d arguments, got %d" % (len(self._slots), len(values)))
        ptrs = self._ptrs
        for i, scalar, name in self._slots:
            v = values[i]
            if scalar:
                self._scalars[i][...] = v
            else:
                try:
                    ptrs[i] = v._addr
                except AttributeError:
                    raise TypeError("argument %d (%s) must be a GpuArray" % (i, name))
        err = lib.GpuElemwise_call(self.ge, ptrs, flags)
        if err:
            check(err, self.context.ctx)


def _dtype(o):
    if hasattr(o, "dtype"):
        return o.dtype
    return np.asarray(o).dtype


def as_argument(o, name, read=False, write=False):
    """reference pygpu/elemwise.py:17-21"""
    if (not read) and (not write):
        raise ValueError("argument is neither read not write")
    return arg(name, _dtype(o), scalar=not isinstance(o, GpuArray), read=read, write=write)


def _kernel(context, oper, args, convert_f16):
    """The GpuElemwise for an expression and argument signature, built once per
    context: the helpers below are called per operation (every `a + b` of an
    ndgpuarray), and building the C object costs several times a launch."""
    cache = context.__dict__.setdefault("_elemwise_cache", {})
    key = (oper, convert_f16, tuple((x.name, x.dtype.str, x.flags) for x in args))
    k = cache.get(key)
    if k is None:
        if len(cache) >= 512:
            cache.clear()
        k = cache[key] = GpuElemwise(context, oper, args, convert_f16=convert_f16)
    return k


_common = {}


def _common_dtype(a, b):
    """get_common_dtype(a, b, True), remembered per pair of (dtype | Python scalar type)."""
    ka = a.dtype if hasattr(a, "dtype") else type(a)
    kb = b.dtype if hasattr(b, "dtype") else type(b)
    try:
        return _common[(ka, kb)]
    except KeyError:
        res = get_common_dtype(a, b, True)
        if ka in (int, float, bool, complex) or hasattr(a, "dtype"):
            if kb in (int, float, bool, complex) or hasattr(b, "dtype"):
                _common[(ka, kb)] = res
        return res


def elemwise1(a, op, oper=None, op_tmpl="res = %(op)sa", out=None, convert_f16=True):
    """Unary op into a new (or given) array (reference pygpu/elemwise.py:24-39)."""
    args = (as_argument(a, "res", write=True), as_argument(a, "a", read=True))
    res = a._empty_like_me() if out is None else out
    if oper is None:
        oper = op_tmpl % {"op": op}
    k = _kernel(a.context, oper, args, convert_f16)
    k(res, a)
    return res


def elemwise2(a, op, b, ary, odtype=None, oper=None,
              op_tmpl="res = (%(out_t)s)a %(op)s (%(out_t)s)b", broadcast=False,
              convert_f16=True):
    """Binary op with NumPy's result type (reference pygpu/elemwise.py:42-80)."""
    ndim_extend = True
    if not isinstance(a, GpuArray):
        a_np, ndim_extend = a, False
        a = np.asarray(a)
    else:
        a_np = a
    if not isinstance(b, GpuArray):
        b_np, ndim_extend = b, False
        b = np.asarray(b)
    else:
        b_np = b
    if odtype is None:
        odtype = _common_dtype(a_np, b_np)
    odtype = np.dtype(odtype)
    args = [arg("res", odtype, write=True), as_argument(a, "a", read=True),
            as_argument(b, "b", read=True)]
    if ndim_extend:
        if a.ndim != b.ndim:
            nd = max(a.ndim, b.ndim)
            if a.ndim < nd:
                a = a.reshape(((1,) * (nd - a.ndim)) + a.shape)
            if b.ndim < nd:
                b = b.reshape(((1,) * (nd - b.ndim)) + b.shape)
        out_shape = tuple(max(sa, sb) for sa, sb in zip(a.shape, b.shape))
        res = gpuarray.empty(out_shape, dtype=odtype, context=ary.context, cls=ary.__class__)
    else:
        res = ary._empty_like_me(dtype=odtype)
    if oper is None:
        ot = odtype
        if convert_f16 and ot == np.dtype("float16"):
            ot = np.dtype("float32")
        oper = op_tmpl % {"op": op, "out_t": dtype_to_ctype(ot)}
    k = _kernel(ary.context, oper, args, convert_f16)
    k(res, a, b, broadcast=broadcast)
    return res


def ielemwise2(a, op, b, oper=None, op_tmpl="a = a %(op)s b", broadcast=False, convert_f16=True):
    """In-place binary op (reference pygpu/elemwise.py:83-97)."""
    if not isinstance(b, GpuArray):
        b = np.asarray(b)
    args = [as_argument(a, "a", read=True, write=True), as_argument(b, "b", read=True)]
    if oper is None:
        oper = op_tmpl % {"op": op}
    k = _kernel(a.context, oper, args, convert_f16)
    k(a, b, broadcast=broadcast)
    return a


def compare(a, op, b, broadcast=False, convert_f16=True):
    """reference pygpu/elemwise.py:99-102"""
    return elemwise2(a, op, b, a, odtype=np.dtype("bool"), op_tmpl="res = (a %(op)s b)",
                     broadcast=broadcast, convert_f16=convert_f16)
