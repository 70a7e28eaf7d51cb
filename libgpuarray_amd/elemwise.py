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
        broadcast = kwargs.pop("broadcast", True)
        padshape = kwargs.pop("padshape", True)
        collapse = kwargs.pop("collapse", True)
        if kwargs:
            raise TypeError("unexpected keyword arguments: %s" % (sorted(kwargs),))
        if len(values) != len(self.args):
            raise TypeError("expected %d arguments, got %d" % (len(self.args), len(values)))
        keep = []
        ptrs = (C.c_void_p * max(len(values), 1))()
        for i, (a, v) in enumerate(zip(self.args, values)):
            if a.scalar:
                s = np.asarray(v, dtype=a.dtype).reshape(())
                buf = np.ascontiguousarray(s)
                keep.append(buf)
                ptrs[i] = buf.ctypes.data
            else:
                if not isinstance(v, GpuArray):
                    raise TypeError("argument %d (%s) must be a GpuArray" % (i, a.name))
                ptrs[i] = C.addressof(v.ga)
        flags = 0
        if broadcast:
            flags |= _lib.GE_BROADCAST
        if padshape:
            flags |= _lib.GE_PADSHAPE
        if not collapse:
            flags |= _lib.GE_NOCOLLAPSE
        check(lib.GpuElemwise_call(self.ge, ptrs, flags), self.context.ctx)


def _broadcast_shape(*shapes):
    return np.broadcast_shapes(*shapes)


def elemwise1(a, op, oper=None, op_tmpl="res = %(op)sa", out=None, convert_f16=True):
    """Unary op into a new (or given) array (reference pygpu/elemwise.py:24-39)."""
    args = (arg("res", a.dtype if out is None else out.dtype, write=True),
            arg("a", a.dtype, read=True))
    if out is None:
        out = gpuarray.empty(a.shape, dtype=a.dtype, context=a.context, cls=type(a))
    if oper is None:
        oper = op_tmpl % {"op": op}
    k = GpuElemwise(a.context, oper, args, convert_f16=convert_f16)
    k(out, a)
    return out


def elemwise2(a, op, b, ary, odtype=None, oper=None, op_tmpl="res = (%(out_t)s)a %(op)s (%(out_t)s)b",
              broadcast=False, convert_f16=True):
    """Binary op with numpy result-type rules (reference pygpu/elemwise.py:42-88)."""
    ctx = ary.context
    if not isinstance(a, GpuArray):
        a = np.asarray(a)
    if not isinstance(b, GpuArray):
        b = np.asarray(b)
    if odtype is None:
        odtype = np.result_type(a.dtype, b.dtype)
    a_scalar = not isinstance(a, GpuArray)
    b_scalar = not isinstance(b, GpuArray)
    shapes = [x.shape for x in (a, b) if isinstance(x, GpuArray)]
    oshape = _broadcast_shape(*shapes) if broadcast else shapes[0]
    out = gpuarray.empty(oshape, dtype=odtype, context=ctx, cls=type(ary))
    ctypes_names = {"float16": "ga_float", "float32": "ga_float", "float64": "ga_double",
                    "bool": "ga_bool", "int8": "ga_byte", "uint8": "ga_ubyte",
                    "int16": "ga_short", "uint16": "ga_ushort", "int32": "ga_int",
                    "uint32": "ga_uint", "int64": "ga_long", "uint64": "ga_ulong"}
    if oper is None:
        oper = op_tmpl % {"op": op, "out_t": ctypes_names[np.dtype(odtype).name]}
    args = (arg("res", out.dtype, write=True),
            arg("a", a.dtype, read=True, scalar=a_scalar),
            arg("b", b.dtype, read=True, scalar=b_scalar))
    k = GpuElemwise(ctx, oper, args, convert_f16=convert_f16)
    k(out, a, b, broadcast=broadcast)
    return out
