"""`ndgpuarray`: a GpuArray that behaves like a NumPy array under Python's
operators and the sum/prod/any/all/min/max methods.  Every operation is one
GpuElemwise or GpuReduction call on the device.

The rules are those of the reference's class of the same name
(pygpu/_array.py:10-294), stated here as a table instead of one method per
operator:

  result type      what NumPy gives for the same operands (dtypes.get_common_dtype),
                   for `/` the type of NumPy's true division
  + - *            computed in the result type
  / // %           on integers C's truncating division and remainder (equal to
                   NumPy's for operands of one sign); `//` on floating results is
                   floor(a / b), `%` is fmod(a, b)
  op=              computed in C's own promotion of the two operand types and
                   stored back into the left array's type; floating forms as above
  comparisons      element-wise, bool result
  sum, prod        accumulate in the result type, small integers widened to the
                   platform integer (reference :250-262, :282-294)
  any, all         truth values, bool result (reference :238-248)
  min, max, argmin, argmax   not in the reference (commented out, :264-280)
"""
import numpy as np

from . import gpuarray
from . import reduction as _red
from .dtypes import dtype_to_ctype, get_common_dtype, get_np_obj
from .elemwise import GpuElemwise, arg, as_argument, compare, elemwise1, elemwise2, ielemwise2

_F16, _F32, _F64 = np.dtype("float16"), np.dtype("float32"), np.dtype("float64")

# operator -> (C symbol, form used when the computation is floating, else None)
_BINARY = {
    "add": ("+", None),
    "sub": ("-", None),
    "mul": ("*", None),
    "truediv": ("/", None),
    "floordiv": ("/", "floor({x} / {y})"),
    "mod": ("%", "fmod({x}, {y})"),
}
_COMPARE = {"lt": "<", "le": "<=", "eq": "==", "ne": "!=", "ge": ">=", "gt": ">"}


def _compute_ctype(dt):
    """C type a result of dtype `dt` is computed in (halves are computed as floats)."""
    return dtype_to_ctype(_F32 if dt == _F16 else dt)


def _statement(dst, sym, float_form, ctype, x="a", y="b"):
    """`dst = x <op> y`; with a C type, both operands are converted to it first."""
    if ctype is not None:
        x, y = "(%s)%s" % (ctype, x), "(%s)%s" % (ctype, y)
    if float_form is not None and ctype in ("ga_float", "ga_double", "float", "double"):
        return "%s = %s" % (dst, float_form.format(x=x, y=y))
    return "%s = %s %s %s" % (dst, x, sym, y)


def _result_dtype(name, x, y):
    if name == "truediv":
        return np.asarray(get_np_obj(x) / get_np_obj(y)).dtype
    return get_common_dtype(x, y, True)


def _inplace_ctype(name, self, other):
    """Type an `op=` is computed in: C's promotion of the operands, except that
    the floating forms of `/`, `//` and `%` are spelled with explicit casts
    (reference pygpu/_array.py:59-68, :89-96, :121-131):
      /=   double if either side is float64, else float if either is float32
      //=  by the left array's type alone
      %=   by the common type, double only when the left array is float64 (so
           that a float32 array and a Python float meet in float32, as in NumPy)."""
    if name not in ("truediv", "floordiv", "mod"):
        return None
    mine, theirs = self.dtype, np.asarray(get_np_obj(other)).dtype
    if name == "mod":
        kinds = (np.dtype(get_common_dtype(self, other, mine == _F64)),)
    elif name == "floordiv":
        kinds = (mine,)
    else:
        kinds = (mine, theirs)
    if _F64 in kinds:
        return "double"
    if _F32 in kinds or _F16 in kinds:
        return "float"
    return None


def _make_binary(name):
    sym, float_form = _BINARY[name]

    def apply(x, y, like):
        dt = np.dtype(_result_dtype(name, x, y))
        oper = _statement("res", sym, float_form, _compute_ctype(dt))
        return elemwise2(x, sym, y, like, odtype=dt, oper=oper, broadcast=True)

    def forward(self, other):
        return apply(self, other, self)

    def reflected(self, other):
        return apply(other, self, self)

    def inplace(self, other):
        oper = _statement("a", sym, float_form, _inplace_ctype(name, self, other))
        return ielemwise2(self, sym, other, oper=oper, broadcast=True)
    return forward, reflected, inplace


def _make_compare(sym):
    def method(self, other):
        return compare(self, sym, other, broadcast=True)
    return method


class ndgpuarray(gpuarray.GpuArray):
    __hash__ = None      # == compares element-wise, so instances cannot be dictionary keys

    def _divmod(self, x, y):
        """(x // y, x % y) from one kernel with two outputs."""
        dt = np.dtype(get_common_dtype(x, y, True))
        ct = _compute_ctype(dt)
        xs = x if isinstance(x, gpuarray.GpuArray) else np.asarray(x)
        ys = y if isinstance(y, gpuarray.GpuArray) else np.asarray(y)
        quot, rem = self._empty_like_me(dtype=dt), self._empty_like_me(dtype=dt)
        oper = "%s; %s" % (_statement("quot", "/", _BINARY["floordiv"][1], ct),
                           _statement("rem", "%", _BINARY["mod"][1], ct))
        k = GpuElemwise(self.context, oper,
                        [arg("quot", dt, write=True), arg("rem", dt, write=True),
                         as_argument(xs, "a", read=True), as_argument(ys, "b", read=True)])
        k(quot, rem, xs, ys, broadcast=True)
        return quot, rem

    def __divmod__(self, other):
        return self._divmod(self, other)

    def __rdivmod__(self, other):
        return self._divmod(other, self)

    def __neg__(self):
        return elemwise1(self, "-")

    def __pos__(self):
        return elemwise1(self, "+")

    def __abs__(self):
        kind, size = self.dtype.kind, self.dtype.itemsize
        if kind in "ub":
            return self.copy()
        if kind == "f":
            oper = "res = fabs(a)"
        elif size == 8:
            oper = "res = a < 0 ? -a : a"       # no 64-bit abs() in the device dialect
        else:
            oper = "res = abs((int)a)" if size < 4 else "res = abs(a)"
        return elemwise1(self, None, oper=oper)

    @property
    def T(self):
        return self.transpose() if self.ndim >= 2 else self

    # -- reductions ---------------------------------------------------------------
    def _logical(self, c_op, neutral, axis, out):
        if self.ndim == 0:
            return self.copy()
        return _red.reduce1(self, c_op, neutral, np.dtype("bool"), axis=axis, out=out)

    def all(self, axis=None, out=None):
        return self._logical("&&", "1", axis, out)

    def any(self, axis=None, out=None):
        return self._logical("||", "0", axis, out)

    def _arith(self, c_op, neutral, axis, dtype, out):
        return _red.reduce1(self, c_op, neutral, _red._upcast(self.dtype) if dtype is None else dtype,
                            axis=axis, out=out)

    def sum(self, axis=None, dtype=None, out=None):
        return self._arith("+", "0", axis, dtype, out)

    def prod(self, axis=None, dtype=None, out=None):
        return self._arith("*", "1", axis, dtype, out)

    def max(self, axis=None, out=None):
        return _red.max(self, axis=axis, out=out)

    def min(self, axis=None, out=None):
        return _red.min(self, axis=axis, out=out)

    def argmax(self, axis=None):
        return _red.argmax(self, axis=axis)

    def argmin(self, axis=None):
        return _red.argmin(self, axis=axis)


for _name in _BINARY:
    _f, _r, _i = _make_binary(_name)
    for _prefix, _fn in (("", _f), ("r", _r), ("i", _i)):
        _fn.__name__ = "__%s%s__" % (_prefix, _name)
        setattr(ndgpuarray, _fn.__name__, _fn)
for _name, _sym in _COMPARE.items():
    _m = _make_compare(_sym)
    _m.__name__ = "__%s__" % _name
    setattr(ndgpuarray, _m.__name__, _m)
del _name, _sym, _f, _r, _i, _m, _prefix, _fn
