"""`ndgpuarray`: GpuArray with NumPy's arithmetic, comparison and reduction
methods, every one a GpuElemwise or reduction call on the device (reference
pygpu/_array.py:10-294).  Result types are what NumPy gives for the same
operands; integer `/`, `//` and `%` are C's (truncating) as in the reference,
which agrees with NumPy for non-negative operands.

Beyond the reference: min and max (commented out there, :264-280) are
provided on top of the C reductions.
"""
import numpy as np

from . import gpuarray
from .dtypes import dtype_to_ctype, get_common_dtype, get_np_obj
from .elemwise import GpuElemwise, arg, as_argument, compare, elemwise1, elemwise2, ielemwise2
from . import reduction as _red


def _div_result(a, b):
    return np.asarray(get_np_obj(a) / get_np_obj(b)).dtype


class ndgpuarray(gpuarray.GpuArray):
    # add
    def __add__(self, other):
        return elemwise2(self, "+", other, self, broadcast=True)

    def __radd__(self, other):
        return elemwise2(other, "+", self, self, broadcast=True)

    def __iadd__(self, other):
        return ielemwise2(self, "+", other, broadcast=True)

    # sub
    def __sub__(self, other):
        return elemwise2(self, "-", other, self, broadcast=True)

    def __rsub__(self, other):
        return elemwise2(other, "-", self, self, broadcast=True)

    def __isub__(self, other):
        return ielemwise2(self, "-", other, broadcast=True)

    # mul
    def __mul__(self, other):
        return elemwise2(self, "*", other, self, broadcast=True)

    def __rmul__(self, other):
        return elemwise2(other, "*", self, self, broadcast=True)

    def __imul__(self, other):
        return ielemwise2(self, "*", other, broadcast=True)

    # truediv
    def __truediv__(self, other):
        return elemwise2(self, "/", other, self, odtype=_div_result(self, other), broadcast=True)

    def __rtruediv__(self, other):
        return elemwise2(other, "/", self, self, odtype=_div_result(other, self), broadcast=True)

    def __itruediv__(self, other):
        np2 = np.asarray(get_np_obj(other))
        kw = {"broadcast": True}
        if self.dtype == np.float32 or np2.dtype == np.float32:
            kw["op_tmpl"] = "a = (float)a / (float)b"
        if self.dtype == np.float64 or np2.dtype == np.float64:
            kw["op_tmpl"] = "a = (double)a / (double)b"
        return ielemwise2(self, "/", other, **kw)

    # floordiv
    def __floordiv__(self, other):
        out_dtype = get_common_dtype(self, other, True)
        kw = {"broadcast": True}
        if out_dtype.kind == "f":
            kw["op_tmpl"] = "res = floor((%(out_t)s)a / (%(out_t)s)b)"
        return elemwise2(self, "/", other, self, odtype=out_dtype, **kw)

    def __rfloordiv__(self, other):
        out_dtype = get_common_dtype(other, self, True)
        kw = {"broadcast": True}
        if out_dtype.kind == "f":
            kw["op_tmpl"] = "res = floor((%(out_t)s)a / (%(out_t)s)b)"
        return elemwise2(other, "/", self, self, odtype=out_dtype, **kw)

    def __ifloordiv__(self, other):
        kw = {"broadcast": True}
        if self.dtype == np.float32:
            kw["op_tmpl"] = "a = floor((float)a / (float)b)"
        if self.dtype == np.float64:
            kw["op_tmpl"] = "a = floor((double)a / (double)b)"
        return ielemwise2(self, "/", other, **kw)

    # mod
    def __mod__(self, other):
        out_dtype = get_common_dtype(self, other, True)
        kw = {"broadcast": True}
        if out_dtype.kind == "f":
            kw["op_tmpl"] = "res = fmod((%(out_t)s)a, (%(out_t)s)b)"
        return elemwise2(self, "%", other, self, odtype=out_dtype, **kw)

    def __rmod__(self, other):
        out_dtype = get_common_dtype(other, self, True)
        kw = {"broadcast": True}
        if out_dtype.kind == "f":
            kw["op_tmpl"] = "res = fmod((%(out_t)s)a, (%(out_t)s)b)"
        return elemwise2(other, "%", self, self, odtype=out_dtype, **kw)

    def __imod__(self, other):
        out_dtype = get_common_dtype(self, other, self.dtype == np.float64)
        kw = {"broadcast": True}
        if out_dtype == np.float32:
            kw["op_tmpl"] = "a = fmod((float)a, (float)b)"
        if out_dtype == np.float64:
            kw["op_tmpl"] = "a = fmod((double)a, (double)b)"
        return ielemwise2(self, "%", other, **kw)

    # divmod
    def _divmod(self, a, b):
        a_np, b_np = a, b
        if not isinstance(a, gpuarray.GpuArray):
            a = np.asarray(a)
        if not isinstance(b, gpuarray.GpuArray):
            b = np.asarray(b)
        odtype = get_common_dtype(a_np, b_np, True)
        args = [arg("div", odtype, write=True), arg("mod", odtype, write=True),
                as_argument(a, "a", read=True), as_argument(b, "b", read=True)]
        div = self._empty_like_me(dtype=odtype)
        mod = self._empty_like_me(dtype=odtype)
        if odtype.kind == "f":
            tmpl = ("div = floor((%(out_t)s)a / (%(out_t)s)b),"
                    "mod = fmod((%(out_t)s)a, (%(out_t)s)b)")
        else:
            tmpl = "div = (%(out_t)s)a / (%(out_t)s)b,mod = a %% b"
        k = GpuElemwise(self.context, tmpl % {"out_t": dtype_to_ctype(odtype)}, args)
        k(div, mod, a, b, broadcast=True)
        return (div, mod)

    def __divmod__(self, other):
        return self._divmod(self, other)

    def __rdivmod__(self, other):
        return self._divmod(other, self)

    def __neg__(self):
        return elemwise1(self, "-")

    def __pos__(self):
        return elemwise1(self, "+")

    def __abs__(self):
        if self.dtype.kind == "u":
            return self.copy()
        if self.dtype.kind == "f":
            oper = "res = fabs(a)"
        elif self.dtype.itemsize < 4:
            oper = "res = abs((int)a)"
        elif self.dtype.itemsize == 8:
            oper = "res = a < 0 ? -a : a"
        else:
            oper = "res = abs(a)"
        return elemwise1(self, None, oper=oper)

    # richcmp
    def __lt__(self, other):
        return compare(self, "<", other, broadcast=True)

    def __le__(self, other):
        return compare(self, "<=", other, broadcast=True)

    def __eq__(self, other):
        return compare(self, "==", other, broadcast=True)

    def __ne__(self, other):
        return compare(self, "!=", other, broadcast=True)

    def __ge__(self, other):
        return compare(self, ">=", other, broadcast=True)

    def __gt__(self, other):
        return compare(self, ">", other, broadcast=True)

    __hash__ = None

    @property
    def T(self):
        if self.ndim < 2:
            return self
        return self.transpose()

    # reductions
    def all(self, axis=None, out=None):
        if self.ndim == 0:
            return self.copy()
        return _red.reduce1(self, "&&", "1", np.dtype("bool"), axis=axis, out=out)

    def any(self, axis=None, out=None):
        if self.ndim == 0:
            return self.copy()
        return _red.reduce1(self, "||", "0", np.dtype("bool"), axis=axis, out=out)

    def prod(self, axis=None, dtype=None, out=None):
        if dtype is None:
            dtype = _red._upcast(self.dtype)
        return _red.reduce1(self, "*", "1", dtype, axis=axis, out=out)

    def sum(self, axis=None, dtype=None, out=None):
        if dtype is None:
            dtype = _red._upcast(self.dtype)
        return _red.reduce1(self, "+", "0", dtype, axis=axis, out=out)

    def max(self, axis=None, out=None):
        return _red.max(self, axis=axis, out=out)

    def min(self, axis=None, out=None):
        return _red.min(self, axis=axis, out=out)

    def argmax(self, axis=None):
        return _red.argmax(self, axis=axis)

    def argmin(self, axis=None):
        return _red.argmin(self, axis=axis)
