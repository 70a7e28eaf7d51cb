"""Contexts and arrays over the C ABI, with the names and behaviour of the
reference's Python layer for this path (pygpu/gpuarray.pyx: GpuContext :1027,
GpuArray :1482, `array`/`empty`/`zeros` :700-930) and its numpy-like array
class (pygpu/_array.py: ndgpuarray).

All device work happens inside libgpuarray.so; this file only marshals
shapes, strides and pointers.
"""
import ctypes as C
import os

import numpy as np

from . import _lib
from ._lib import lib, check, GpuArrayException, UnsupportedException, GpuArrayStruct, c_ssize_t
from .dtypes import dtype_to_ctype  # noqa: F401  (part of this module's interface, as in the reference)

# numpy dtype.num equals the typecode on LP64 Linux
# (reference pygpu/gpuarray.pyx:101-116).
_TYPECODES = {
    np.dtype("bool"): _lib.GA_BOOL, np.dtype("int8"): _lib.GA_BYTE,
    np.dtype("uint8"): _lib.GA_UBYTE, np.dtype("int16"): _lib.GA_SHORT,
    np.dtype("uint16"): _lib.GA_USHORT, np.dtype("int32"): _lib.GA_INT,
    np.dtype("uint32"): _lib.GA_UINT, np.dtype("int64"): _lib.GA_LONG,
    np.dtype("uint64"): _lib.GA_ULONG, np.dtype("float32"): _lib.GA_FLOAT,
    np.dtype("float64"): _lib.GA_DOUBLE, np.dtype("float16"): _lib.GA_HALF,
    np.dtype("complex64"): _lib.GA_CFLOAT, np.dtype("complex128"): _lib.GA_CDOUBLE,
}
_DTYPES = {v: k for k, v in _TYPECODES.items()}


def dtype_to_typecode(dtype):
    try:
        return _TYPECODES[dtype]          # a dtype object: the common case
    except (KeyError, TypeError):
        pass
    try:
        return _TYPECODES[np.dtype(dtype)]
    except KeyError:
        raise ValueError("don't know how to convert to dtype: %s" % (dtype,))


def typecode_to_dtype(typecode):
    try:
        return _DTYPES[typecode]
    except KeyError:
        raise NotImplementedError("TODO: support for typecode %d" % typecode)


def count_devices(kind="hip", platform=0):
    n = C.c_uint(0)
    check(lib.gpu_get_device_count(kind.encode(), platform, C.byref(n)))
    return n.value


def count_platforms(kind="hip"):
    """reference pygpu/gpuarray.pyx:534-545"""
    n = C.c_uint(0)
    check(lib.gpu_get_platform_count(kind.encode(), C.byref(n)))
    return n.value


def api_version():
    """(library API version, module version); reference pygpu/gpuarray.pyx:14-18"""
    return (_lib.GPUARRAY_API_VERSION, 0)


def abi_version():
    """(major, minor) of the library ABI; reference pygpu/gpuarray.pyx:20-25"""
    return (_lib.GPUARRAY_ABI_VERSION // 1000, _lib.GPUARRAY_ABI_VERSION % 1000)


_registered = []   # the type records handed to the C table must stay alive


def register_dtype(dtype, cname):
    """Make a new element type known to the kernel generators under the C name
    `cname`; returns its typecode (reference pygpu/gpuarray.pyx:120-158)."""
    dtype = np.dtype(dtype)
    name = cname.encode() if isinstance(cname, str) else bytes(cname)
    rec = _lib.GpuArrayType(name, dtype.itemsize, dtype.alignment, 0)
    typecode = lib.gpuarray_register_type(C.byref(rec), None)
    if typecode == -1:
        raise RuntimeError("Could not register type")
    _registered.append((rec, name))
    from . import dtypes
    dtypes._REGISTERED[dtype] = name.decode()
    _TYPECODES[dtype] = typecode
    _DTYPES[typecode] = dtype
    return typecode


class GpuContext(object):
    """One device, one stream (reference pygpu/gpuarray.pyx:1027-1168)."""

    def __init__(self, kind="hip", devno=0, single_stream=True, initial_cache_size=None,
                 max_cache_size=None, kernel_cache_path=None):
        props = C.c_void_p()
        check(lib.gpucontext_props_new(C.byref(props)))
        lib.gpucontext_props_hip_dev(props, devno)
        if single_stream:
            lib.gpucontext_props_set_single_stream(props)
        if kernel_cache_path is not None:
            # the props object keeps the pointer, not a copy: hold the bytes
            self._kcache = os.fsencode(kernel_cache_path)
            lib.gpucontext_props_kernel_cache(props, self._kcache)
        if initial_cache_size is not None or max_cache_size is not None:
            # max_cache_size == 0 turns the device memory cache off
            err = lib.gpucontext_props_alloc_cache(
                props, initial_cache_size or 0,
                (1 << 64) - 1 if max_cache_size is None else max_cache_size)
            if err:
                lib.gpucontext_props_del(props)
                check(err)
        self.ctx = C.c_void_p()
        self.kind = kind
        # init consumes props
        check(lib.gpucontext_init(C.byref(self.ctx), kind.encode(), props))

    def __del__(self):
        ctx = getattr(self, "ctx", None)
        if ctx:
            lib.gpucontext_deref(ctx)
            self.ctx = None

    def _prop(self, prop_id, ctype):
        v = ctype()
        check(lib.gpucontext_property(self.ctx, prop_id, C.byref(v)), self.ctx)
        return v.value

    @property
    def devname(self):
        buf = C.create_string_buffer(256)
        check(lib.gpucontext_property(self.ctx, _lib.GA_CTX_PROP_DEVNAME, buf), self.ctx)
        return buf.value.decode()

    @property
    def bin_id(self):
        return self._prop(_lib.GA_CTX_PROP_BIN_ID, C.c_char_p).decode()

    @property
    def unique_id(self):
        """PCI bus id of the device"""
        buf = C.create_string_buffer(16)
        check(lib.gpucontext_property(self.ctx, _lib.GA_CTX_PROP_UNIQUE_ID, buf), self.ctx)
        return buf.value.decode()

    @property
    def ptr(self):
        """the gpucontext pointer as an integer"""
        return self.ctx.value

    def __enter__(self):
        # the reference makes a CUDA context current here (cuda_enter); every
        # call of this backend selects its device itself
        return self

    def __exit__(self, t, v, tb):
        return False

    def __reduce__(self):
        raise RuntimeError("Cannot pickle GpuContext object")

    numprocs = property(lambda s: s._prop(_lib.GA_CTX_PROP_NUMPROCS, C.c_uint))
    maxlsize1 = property(lambda s: s._prop(_lib.GA_CTX_PROP_MAXLSIZE1, C.c_size_t))
    maxlsize2 = property(lambda s: s._prop(_lib.GA_CTX_PROP_MAXLSIZE2, C.c_size_t))
    maxgsize1 = property(lambda s: s._prop(_lib.GA_CTX_PROP_MAXGSIZE1, C.c_size_t))
    maxgsize2 = property(lambda s: s._prop(_lib.GA_CTX_PROP_MAXGSIZE2, C.c_size_t))
    largest_memblock = property(lambda s: s._prop(_lib.GA_CTX_PROP_LARGEST_MEMBLOCK, C.c_size_t))
    lmemsize = property(lambda s: s._prop(_lib.GA_CTX_PROP_LMEMSIZE, C.c_size_t))
    maxlsize0 = property(lambda s: s._prop(_lib.GA_CTX_PROP_MAXLSIZE0, C.c_size_t))
    maxgsize0 = property(lambda s: s._prop(_lib.GA_CTX_PROP_MAXGSIZE0, C.c_size_t))
    total_gmem = property(lambda s: s._prop(_lib.GA_CTX_PROP_TOTAL_GMEM, C.c_size_t))
    free_gmem = property(lambda s: s._prop(_lib.GA_CTX_PROP_FREE_GMEM, C.c_size_t))

    def error(self):
        return lib.gpucontext_error(self.ctx, 0).decode(errors="replace")

    # timing on the context's own stream (HIP events), in milliseconds
    def time_begin(self):
        fn = _lib.extension("hip_time_begin", C.c_int, [C.c_void_p])
        check(fn(self.ctx), self.ctx)

    def time_end(self):
        fn = _lib.extension("hip_time_end", C.c_float, [C.c_void_p])
        ms = fn(self.ctx)
        if ms < 0:
            raise GpuArrayException("event timing failed: " + self.error(), _lib.GA_IMPL_ERROR)
        return ms

    def mark(self, slot):
        """Timing mark `slot` on the stream (no wait)."""
        fn = _lib.extension("hip_event_record", C.c_int, [C.c_void_p, C.c_uint])
        check(fn(self.ctx, slot), self.ctx)

    def elapsed(self, a, b):
        """Milliseconds between marks a and b (waits for b)."""
        fn = _lib.extension("hip_event_elapsed", C.c_float, [C.c_void_p, C.c_uint, C.c_uint])
        ms = fn(self.ctx, a, b)
        if ms < 0:
            raise GpuArrayException("event timing failed: " + self.error(), _lib.GA_IMPL_ERROR)
        return ms

    def last_launch_hash(self):
        """Hash (hex) of the text and entry point of the kernel launched last."""
        fn = _lib.extension("hip_last_launch_hash", C.c_ulonglong, [C.c_void_p])
        return "%016x" % fn(self.ctx)

    def kernel_timing(self, on=True):
        """Give every launch from now on its own start and stop event."""
        fn = _lib.extension("hip_kernel_timing", C.c_int, [C.c_void_p, C.c_int])
        check(fn(self.ctx, 1 if on else 0), self.ctx)

    def kernel_times(self, limit=65536):
        """Milliseconds of each launch recorded since kernel_timing(True)."""
        fn = _lib.extension("hip_kernel_times", C.c_int, [C.c_void_p, C.POINTER(C.c_float), C.c_uint])
        buf = (C.c_float * limit)()
        n = fn(self.ctx, buf, limit)
        if n < 0:
            raise GpuArrayException("kernel timing failed: " + self.error(), _lib.GA_IMPL_ERROR)
        return list(buf[:min(n, limit)])

    def kernel_hashes(self, limit=65536):
        """Text hash (hex) of each launch recorded since kernel_timing(True)."""
        fn = _lib.extension("hip_kernel_hashes", C.c_int, [C.c_void_p, C.POINTER(C.c_ulonglong), C.c_uint])
        buf = (C.c_ulonglong * limit)()
        n = fn(self.ctx, buf, limit)
        return ["%016x" % v for v in buf[:min(n, limit)]]

    def reload_tuning(self):
        """Read the GPUARRAY_* tuning knobs from the environment again (a
        context reads them once, when it is made)."""
        fn = _lib.extension("hip_reload_tuning", C.c_int, [C.c_void_p])
        check(fn(self.ctx), self.ctx)

    def sync(self):
        # any buffer of the context syncs the one stream; use the error buffer
        eb = C.c_void_p()
        check(lib.gpucontext_property(self.ctx, _lib.GA_CTX_PROP_ERRBUF, C.byref(eb)), self.ctx)
        check(lib.gpudata_sync(eb), self.ctx)


_default_context = None


def set_default_context(ctx):
    global _default_context
    _default_context = ctx


def get_default_context():
    return _default_context


def init(dev="hip0"):
    """`init("hipN")`: reference pygpu.gpuarray.init("cudaN"/"openclP:D")."""
    if not dev.startswith("hip"):
        raise ValueError("only \"hipN\" devices exist on this backend, got %r" % (dev,))
    devno = int(dev[3:] or 0)
    return GpuContext("hip", devno)


def _ensure_context(context):
    ctx = context if context is not None else _default_context
    if ctx is None:
        raise TypeError("No context specified.")
    return ctx


class flags(object):
    """NumPy-style view of an array's flag word, by attribute or by NumPy's
    flag names and one- or two-letter short forms (reference
    pygpu/gpuarray.pyx:1190-1342)."""

    _KEYS = {"C": "c_contiguous", "F": "f_contiguous", "W": "writeable", "B": "behaved",
             "O": "owndata", "A": "aligned", "U": "updateifcopy", "CA": "carray", "FA": "farray",
             "FNC": "fnc", "FORC": "forc", "CARRAY": "carray", "FARRAY": "farray",
             "FORTRAN": "fortran", "BEHAVED": "behaved", "OWNDATA": "owndata",
             "ALIGNED": "aligned", "WRITEABLE": "writeable", "CONTIGUOUS": "c_contiguous",
             "UPDATEIFCOPY": "updateifcopy", "C_CONTIGUOUS": "c_contiguous",
             "F_CONTIGUOUS": "f_contiguous"}
    _BEHAVED = _lib.GA_ALIGNED | _lib.GA_WRITEABLE

    def __init__(self, fl):
        self.fl = int(fl)

    def __reduce__(self):
        return (flags, (self.fl,))

    c_contiguous = property(lambda s: bool(s.fl & _lib.GA_C_CONTIGUOUS))
    f_contiguous = property(lambda s: bool(s.fl & _lib.GA_F_CONTIGUOUS))
    contiguous = c_contiguous
    fortran = f_contiguous
    aligned = property(lambda s: bool(s.fl & _lib.GA_ALIGNED))
    writeable = property(lambda s: bool(s.fl & _lib.GA_WRITEABLE))
    updateifcopy = property(lambda s: False)     # not supported
    owndata = property(lambda s: True)           # no equivalent for device arrays
    behaved = property(lambda s: (s.fl & s._BEHAVED) == s._BEHAVED)
    carray = property(lambda s: s.behaved and s.c_contiguous)
    forc = property(lambda s: s.c_contiguous or s.f_contiguous)
    fnc = property(lambda s: s.f_contiguous and not s.c_contiguous)
    # any of F_CONTIGUOUS / ALIGNED / WRITEABLE set and not C-contiguous: NumPy's own definition
    farray = property(lambda s: bool(s.fl & (_lib.GA_F_CONTIGUOUS | s._BEHAVED)) and not s.c_contiguous)
    num = property(lambda s: s.fl)

    def __getitem__(self, key):
        if isinstance(key, bytes):
            key = key.decode()
        if not isinstance(key, str) or key not in self._KEYS:
            raise KeyError("Unknown flag")
        return getattr(self, self._KEYS[key])

    def __eq__(self, other):
        if not isinstance(other, flags):
            return NotImplemented
        return self.fl == other.fl

    def __ne__(self, other):
        if not isinstance(other, flags):
            return NotImplemented
        return self.fl != other.fl

    __hash__ = None

    def __repr__(self):
        return "\n".join(" %s : %s" % (n.upper(), getattr(self, n)) for n in
                         ("c_contiguous", "f_contiguous", "owndata", "writeable", "aligned",
                          "updateifcopy"))


class GpuArray(object):
    """A strided view over a device buffer (reference pygpu/gpuarray.pyx:1482-2160
    and pygpu/_array.py)."""

    def __init__(self, context):
        self.context = context
        self.ga = GpuArrayStruct()
        self._addr = C.addressof(self.ga)   # of the C struct; fixed for the object's life
        self._ref = C.byref(self.ga)
        self.base = None

    def __del__(self):
        ga = getattr(self, "ga", None)
        if ga is not None and ga.data:
            lib.GpuArray_clear(C.byref(ga))

    # -- metadata ---------------------------------------------------------------
    def _get_shape(self):
        return tuple(self.ga.dimensions[i] for i in range(self.ga.nd))

    def _set_shape(self, newshape):
        """In-place reshape; refuses what would need a copy
        (reference pygpu/gpuarray.pyx:2136-2166)."""
        if isinstance(newshape, (int, np.integer)):
            newshape = (newshape,)
        newshape = self._fill_unknown(list(newshape))
        dims = (C.c_size_t * max(len(newshape), 1))(*newshape)
        err = lib.GpuArray_reshape_inplace(self._ptr(), len(newshape), dims, _lib.GA_C_ORDER)
        if err == _lib.GA_COPY_ERROR:
            raise AttributeError("Incompatible shape for in-place modification")
        self._check(err)

    shape = property(_get_shape, _set_shape)

    def _get_strides(self):
        return tuple(self.ga.strides[i] for i in range(self.ga.nd))

    def _set_strides(self, newstrides):
        """reference pygpu/gpuarray.pyx:241-267,2177-2185: the new strides must
        keep every element inside the buffer."""
        newstrides = tuple(int(v) for v in newstrides)
        if len(newstrides) != self.ga.nd:
            raise ValueError("new strides are the wrong length")
        size = C.c_size_t()
        self._check(lib.gpudata_property(self.ga.data, _lib.GA_BUFFER_PROP_SIZE, C.byref(size)))
        lower = upper = self.ga.offset
        ok = True
        for i in range(self.ga.nd):
            if self.ga.dimensions[i] == 0:
                break
            off = newstrides[i] * (self.ga.dimensions[i] - 1)
            if off > 0:
                if upper + off > size.value:
                    ok = False
                    break
                upper += off
            else:
                if lower < -off:
                    ok = False
                    break
                lower += off
        else:
            ok = upper + self.itemsize <= size.value
        if not ok:
            raise ValueError("new strides go outside of allocated memory")
        for i in range(self.ga.nd):
            self.ga.strides[i] = newstrides[i]
        lib.GpuArray_fix_flags(self._ptr())

    strides = property(_get_strides, _set_strides)

    def _fill_unknown(self, shape):
        shape = [int(d) for d in shape]
        if shape.count(-1) > 1:
            raise ValueError("can only specify one unknown dimension")
        if shape.count(-1) == 1:
            known = 1
            for d in shape:
                if d != -1:
                    known *= d
            if known == 0 or self.size % known:
                raise ValueError("total size of new array must be unchanged")
            shape[shape.index(-1)] = self.size // known
        return shape

    gpudata = property(lambda s: s.ga.data)
    ndim = property(lambda s: s.ga.nd)
    offset = property(lambda s: s.ga.offset)
    typecode = property(lambda s: s.ga.typecode)
    dtype = property(lambda s: typecode_to_dtype(s.ga.typecode))
    itemsize = property(lambda s: s.dtype.itemsize)
    flags = property(lambda s: flags(s.ga.flags))

    @property
    def size(self):
        n = 1
        for d in self.shape:
            n *= d
        return n

    def __len__(self):
        if self.ga.nd == 0:
            raise TypeError("len() of unsized object")
        return self.ga.dimensions[0]

    def __bool__(self):
        """reference pygpu/gpuarray.pyx:2118-2125"""
        if self.size == 0:
            return False
        if self.size == 1:
            return bool(np.asarray(self))
        raise ValueError("Truth value of array with more than one element is ambiguous")

    __hash__ = None

    def _empty_like_me(self, dtype=None, order="C"):
        """A new array of this one's shape, class and context
        (reference pygpu/gpuarray.pyx:1714-1735)."""
        if order.upper() == "A":
            order = "F" if (self.flags.f_contiguous and not self.flags.c_contiguous) else "C"
        return empty(self.shape, self.dtype if dtype is None else dtype, order, self.context,
                     cls=type(self))

    def _ptr(self):
        return self._ref

    def _check(self, err):
        check(err, self.context.ctx)

    def _new(self):
        return type(self)(self.context)

    # -- data movement ------------------------------------------------------------
    def sync(self):
        self._check(lib.GpuArray_sync(self._ptr()))

    def write(self, src):
        """Copy a numpy array of the same shape and dtype in (one-segment arrays)."""
        src = np.asarray(src)
        if src.dtype != self.dtype or src.shape != self.shape:
            raise ValueError("shape or dtype mismatch")
        if self.flags.c_contiguous:
            src = np.ascontiguousarray(src)
        elif self.flags.f_contiguous:
            src = np.asfortranarray(src)
        self._check(lib.GpuArray_write(self._ptr(), src.ctypes.data_as(C.c_void_p), src.nbytes))

    def read(self, dst):
        """Copy into a writeable NumPy array of the same shape, dtype and
        contiguity (reference pygpu/gpuarray.pyx:1756-1786)."""
        if not isinstance(dst, np.ndarray) or not dst.flags.writeable:
            raise ValueError("Destination is not a writeable ndarray")
        if dst.dtype != self.dtype or dst.shape != self.shape:
            raise ValueError("shape or dtype mismatch")
        if self.flags.c_contiguous and dst.flags.c_contiguous:
            pass
        elif self.flags.f_contiguous and dst.flags.f_contiguous:
            pass
        else:
            raise ValueError("source and destination must be contiguous in the same order")
        self._check(lib.GpuArray_read(dst.ctypes.data_as(C.c_void_p), dst.nbytes, self._ptr()))

    def __copy__(self):
        return self.copy("C")          # reference pygpu/gpuarray.pyx:1793-1800

    def __deepcopy__(self, memo):
        if id(self) in memo:
            return memo[id(self)]
        return self.copy("C")

    def __array__(self, dtype=None, copy=None):
        a = self
        if not (self.flags.c_contiguous or self.flags.f_contiguous):
            a = self.copy("C")
        order = "C" if a.flags.c_contiguous else "F"
        out = np.empty(a.shape, dtype=a.dtype, order=order)
        if out.nbytes:
            a._check(lib.GpuArray_read(out.ctypes.data_as(C.c_void_p), out.nbytes, a._ptr()))
        if dtype is not None and np.dtype(dtype) != out.dtype:
            out = out.astype(dtype)
        return out

    def copy(self, order="C"):
        res = self._new()
        o = {"C": _lib.GA_C_ORDER, "F": _lib.GA_F_ORDER, "A": _lib.GA_ANY_ORDER}[order.upper()]
        if o == _lib.GA_ANY_ORDER:
            o = _lib.GA_F_ORDER if (self.flags.f_contiguous and not self.flags.c_contiguous) \
                else _lib.GA_C_ORDER
        self._check(lib.GpuArray_copy(res._ptr(), self._ptr(), o))
        return res

    def transfer(self, new_ctx):
        """A copy of this array in another context
        (reference pygpu/gpuarray.pyx:1779-1791)."""
        if not (self.flags.c_contiguous or self.flags.f_contiguous):
            raise ValueError("transfer() only works for contigous source")
        res = empty(self.shape, self.dtype, "C" if self.flags.c_contiguous else "F", context=new_ctx)
        check(lib.GpuArray_transfer(res._ptr(), self._ptr()), new_ctx.ctx)
        return res

    @property
    def data(self):
        """The raw OpenCL buffer object in the reference
        (pygpu/gpuarray.pyx:2223-2236): there is no such object here."""
        raise TypeError("This is for OpenCL arrays.")

    base_data = data

    def take1(self, idx, check=True):
        """Rows of `self` picked by the 1-D integer array `idx`
        (reference pygpu/gpuarray.pyx:2098-2113): negative entries count from
        the end, an entry out of range raises IndexError.  check=False is
        GpuArray_take1's check_error = 0: the call does not wait for the
        kernel to read the bounds flag back, a row whose index is out of range
        keeps what the result's memory held, and the flag stays set for the
        next checked call (reference src/gpuarray_array.c:534-543)."""
        if idx.ndim != 1:
            raise ValueError("Expected index with nd=1")
        if self.ndim == 0:
            raise _lib.GpuArrayException("take1 of a 0-d array", _lib.GA_INVALID_ERROR)
        res = empty((idx.shape[0],) + self.shape[1:], self.dtype, context=self.context)
        err = lib.GpuArray_take1(res._ptr(), self._ptr(), idx._ptr(), 1 if check else 0)
        if err == _lib.GA_VALUE_ERROR:
            msg = lib.gpucontext_error(self.context.ctx, err)
            raise IndexError(msg.decode(errors="replace") if msg else "Index out of bounds")
        self._check(err)
        return res

    def astype(self, dtype, order="A"):
        res = empty(self.shape, dtype=dtype, order="C" if order in "AC" else "F",
                    context=self.context, cls=type(self))
        self._check(lib.GpuArray_move(res._ptr(), self._ptr()))
        return res

    def view(self):
        res = self._new()
        self._check(lib.GpuArray_view(res._ptr(), self._ptr()))
        res.base = self
        return res

    def memset(self, byte):
        self._check(lib.GpuArray_memset(self._ptr(), byte))

    # -- shape manipulation ---------------------------------------------------------
    def transpose(self, *axes):
        if len(axes) == 1 and isinstance(axes[0], (tuple, list)):
            axes = tuple(axes[0])
        res = self._new()
        if len(axes) == 0 or axes == (None,):
            arg = None
        else:
            if len(axes) != self.ndim:
                raise ValueError("axes don't match array")
            arg = (C.c_uint * len(axes))(*[a % self.ndim if self.ndim else a for a in axes])
        self._check(lib.GpuArray_transpose(res._ptr(), self._ptr(), arg))
        res.base = self
        return res

    T = property(lambda s: s.transpose())

    def reshape(self, shape, order="C"):
        if isinstance(shape, int):
            shape = (shape,)
        shape = self._fill_unknown(list(shape))
        dims = (C.c_size_t * max(len(shape), 1))(*shape)
        o = {"C": _lib.GA_C_ORDER, "F": _lib.GA_F_ORDER, "A": _lib.GA_ANY_ORDER}[order.upper()]
        res = self._new()
        self._check(lib.GpuArray_reshape(res._ptr(), self._ptr(), len(shape), dims, o, 0))
        return res

    def __getitem__(self, key):
        """Basic indexing only: ints, slices, Ellipsis (reference
        pygpu/gpuarray.pyx:1928-2069 lowers these to start/stop/step triples)."""
        if isinstance(key, list):
            if any(isinstance(k, slice) or k is Ellipsis for k in key):
                key = tuple(key)
            else:
                raise NotImplementedError("fancy indexing not supported")
        if not isinstance(key, tuple):
            key = (key,)
        if any(isinstance(k, (list, np.ndarray, GpuArray)) and getattr(k, "ndim", 1) > 0 for k in key):
            raise NotImplementedError("fancy indexing not supported")
        if any(k is None for k in key):
            # index without the None entries, then put the unit dims back
            # (reference pygpu/gpuarray.pyx:1974-2008)
            sliced = self.__getitem__(tuple(k for k in key if k is not None))
            n_real = len([k for k in key if k is not None and k is not Ellipsis])
            expanded = []
            for k in key:
                if k is Ellipsis:
                    expanded.extend([slice(None)] * (self.ndim - n_real))
                else:
                    expanded.append(k)
            if Ellipsis not in key:
                expanded.extend([slice(None)] * (self.ndim - n_real))
            new_shape, new_strides, i = [], [], 0
            for k in expanded:
                if k is None:
                    new_shape.append(1)
                    new_strides.append(0)
                elif isinstance(k, slice):
                    new_shape.append(sliced.shape[i])
                    new_strides.append(sliced.strides[i])
                    i += 1
            res = from_strided(sliced, sliced.offset, new_shape, new_strides,
                               writeable=sliced.flags.writeable)
            res.base = self
            return res
        nd = self.ndim
        if len([k for k in key if k is Ellipsis]) > 1:
            raise IndexError("an index can only have a single ellipsis")
        n_explicit = len([k for k in key if k is not Ellipsis])
        if n_explicit > nd:
            raise IndexError("too many indices for array")
        full = []
        for k in key:
            if k is Ellipsis:
                full.extend([slice(None)] * (nd - n_explicit))
            else:
                full.append(k)
        full.extend([slice(None)] * (nd - len(full)))
        starts = (c_ssize_t * max(nd, 1))()
        stops = (c_ssize_t * max(nd, 1))()
        steps = (c_ssize_t * max(nd, 1))()
        for i, k in enumerate(full):
            dim = self.shape[i]
            if isinstance(k, slice):
                st, sp, stp = k.indices(dim)
                if stp < 0 and sp < 0:
                    sp = -1
                if (stp > 0 and sp < st) or (stp < 0 and sp > st):
                    sp = st
                starts[i], stops[i], steps[i] = st, sp, stp
            else:
                if not isinstance(k, (int, np.integer)) and not (
                        isinstance(k, np.ndarray) and k.ndim == 0 and k.dtype.kind in "iu"):
                    raise IndexError("only integers, slices, None and Ellipsis are valid indices")
                k = int(k)
                if k < 0:
                    k += dim
                if k < 0 or k >= dim:
                    raise IndexError("index %d out of bounds" % k)
                starts[i], stops[i], steps[i] = k, k + 1, 0
        res = self._new()
        self._check(lib.GpuArray_index(res._ptr(), self._ptr(), starts, stops, steps))
        res.base = self
        return res

    def __setitem__(self, key, value):
        """a[key] = value through GpuArray_setarray (reference gpuarray.pyx:2071-2096)."""
        target = self if key is Ellipsis or key == slice(None) else self.__getitem__(key)
        if not isinstance(value, GpuArray):
            value = array(np.asarray(value, dtype=self.dtype), context=self.context)
        target._check(lib.GpuArray_setarray(target._ptr(), value._ptr()))

    def __repr__(self):
        return "gpuarray." + repr(np.asarray(self))


_DIM_ARRAYS = {}     # rank -> ctypes array type of that many extents
_ORDERS = {"C": _lib.GA_C_ORDER, "F": _lib.GA_F_ORDER, "A": _lib.GA_ANY_ORDER,
           "c": _lib.GA_C_ORDER, "f": _lib.GA_F_ORDER, "a": _lib.GA_ANY_ORDER}


def _make(cls, context):
    return (cls or GpuArray)(context)


def empty(shape, dtype="float32", order="C", context=None, cls=None):
    ctx = _ensure_context(context)
    if isinstance(shape, (int, np.integer)):
        shape = (int(shape),)
    res = _make(cls, ctx)
    nd = len(shape)
    dims = _DIM_ARRAYS.get(nd)
    if dims is None:
        dims = _DIM_ARRAYS[nd] = C.c_size_t * max(nd, 1)
    err = lib.GpuArray_empty(res._ref, ctx.ctx, dtype_to_typecode(dtype), nd, dims(*shape),
                             _ORDERS[order])
    if err:
        check(err, ctx.ctx)
    return res


def zeros(shape, dtype="float32", order="C", context=None, cls=None):
    res = empty(shape, dtype, order, context, cls)
    res.memset(0)
    return res


def array(obj, dtype=None, order="A", context=None, cls=None):
    """Device copy of anything numpy can turn into an array."""
    if isinstance(obj, GpuArray):
        return obj.copy("C" if order == "A" else order)
    a = np.array(obj, dtype=dtype, copy=True)
    # (np.ascontiguousarray would turn a 0-d array into a 1-d one)
    if order.upper() == "F" or (order.upper() == "A" and a.flags.f_contiguous
                                and not a.flags.c_contiguous):
        a = np.array(a, order="F", copy=None)
        o = "F"
    else:
        a = np.array(a, order="C", copy=None)
        o = "C"
    res = empty(a.shape, a.dtype, o, context, cls)
    if a.nbytes:
        check(lib.GpuArray_write(res._ptr(), a.ctypes.data_as(C.c_void_p), a.nbytes),
              res.context.ctx)
    return res


def asarray(obj, dtype=None, order="A", context=None, cls=None):
    if isinstance(obj, GpuArray) and (dtype is None or np.dtype(dtype) == obj.dtype):
        return obj
    return array(obj, dtype, order, context, cls)


def from_strided(base, offset, shape, strides, dtype=None, writeable=True, cls=None):
    """View `base`'s buffer with explicit byte offset and strides
    (GpuArray_fromdata; reference gpuarray.pyx `from_gpudata` :760-815)."""
    res = (cls or type(base))(base.context)
    nd = len(shape)
    dims = (C.c_size_t * max(nd, 1))(*shape)
    strs = (c_ssize_t * max(nd, 1))(*strides)
    tc = base.typecode if dtype is None else dtype_to_typecode(dtype)
    check(lib.GpuArray_fromdata(res._ptr(), base.ga.data, offset, tc, nd, dims, strs,
                                1 if writeable else 0), base.context.ctx)
    res.base = base
    return res


class _gpudata_owner(object):
    """Stands for a buffer known only by its gpudata pointer."""

    def __init__(self, context, data):
        self.context = context
        self.ga = GpuArrayStruct()
        self.ga.data = data


def from_gpudata(data, offset, dtype, shape, context=None, strides=None, writable=True, base=None,
                 cls=None):
    """An array over an existing buffer given as the integer value of its
    gpudata pointer (the `gpudata` attribute of an array); C-contiguous
    unless `strides` are given.  `base` is kept alive with the result
    (reference pygpu/gpuarray.pyx:849-939).  As there, a wrong pointer takes
    the interpreter down."""
    context = _ensure_context(context)
    try:
        shape = tuple(shape)
    except TypeError:
        shape = (shape,)
    if strides is not None and len(strides) != len(shape):
        raise ValueError("strides must be the same length as shape")
    dtype = np.dtype(dtype)
    if not strides:
        strides, step = [], dtype.itemsize
        for d in reversed(shape):
            strides.insert(0, step)
            step *= d
    res = from_strided(_gpudata_owner(context, data), offset, shape, strides, dtype=dtype,
                       writeable=writable, cls=cls or GpuArray)
    res.base = base
    return res


def zeros_like(a, dtype=None, order="C"):
    return zeros(a.shape, a.dtype if dtype is None else dtype, order, a.context, cls=type(a))


def empty_like(a, dtype=None, order="C"):
    return a._empty_like_me(dtype=dtype, order=order)


def ascontiguousarray(a, dtype=None, context=None):
    """C-ordered device array; `a` itself when it already is one of the right
    type (reference pygpu/gpuarray.pyx:797-817; 0-d input gives a 1-d result,
    as NumPy's function does)."""
    if isinstance(a, GpuArray):
        if (dtype is None or np.dtype(dtype) == a.dtype) and a.flags.c_contiguous and a.ndim >= 1:
            return a
        res = a.astype(a.dtype if dtype is None else dtype, order="C") \
            if (dtype is not None and np.dtype(dtype) != a.dtype) else a.copy("C")
        return res.reshape((1,)) if res.ndim == 0 else res
    res = array(a, dtype=dtype, order="C", context=context)
    return res.reshape((1,)) if res.ndim == 0 else res


def asfortranarray(a, dtype=None, context=None):
    """Fortran-ordered device array (reference pygpu/gpuarray.pyx:819-839)."""
    if isinstance(a, GpuArray):
        if (dtype is None or np.dtype(dtype) == a.dtype) and a.flags.f_contiguous and a.ndim >= 1:
            return a
        if dtype is not None and np.dtype(dtype) != a.dtype:
            a = a.astype(dtype)
        res = a.copy("F")
        return res.reshape((1,)) if res.ndim == 0 else res
    res = array(a, dtype=dtype, order="F", context=context)
    return res.reshape((1,)) if res.ndim == 0 else res


def may_share_memory(a, b):
    """reference pygpu/gpuarray.pyx:841-847 (GpuArray_share)"""
    return bool(lib.GpuArray_share(a._ptr(), b._ptr()))


class GpuKernel(object):
    """A kernel from source text (reference pygpu/gpuarray.pyx:2269-2500):
    `types` lists the argument types, GpuArray for buffers and dtypes for
    by-value arguments; the call takes `n` (a problem size the library turns
    into a launch shape) or explicit `gs`/`ls` of up to three dims."""

    def __init__(self, source, name, types, context=None, have_double=False, have_small=False,
                 have_complex=False, have_half=False, cuda=False, opencl=False):
        self.context = _ensure_context(context)
        flags = 0
        if have_double:
            flags |= _lib.GA_USE_DOUBLE
        if have_small:
            flags |= _lib.GA_USE_SMALL
        if have_complex:
            flags |= _lib.GA_USE_COMPLEX
        if have_half:
            flags |= _lib.GA_USE_HALF
        if cuda:
            flags |= _lib.GA_USE_CUDA
        if opencl:
            flags |= _lib.GA_USE_OPENCL
        self._types = [_lib.GA_BUFFER if t is GpuArray else dtype_to_typecode(t) for t in types]
        self._dtypes = [None if t is GpuArray else np.dtype(t) for t in types]
        src = source.encode() if isinstance(source, str) else source
        srcs = (C.c_char_p * 1)(src)
        lens = (C.c_size_t * 1)(len(src))
        tarr = (C.c_int * max(len(self._types), 1))(*self._types)
        self.k = _lib.GpuKernelStruct()
        err_str = C.c_char_p()
        err = lib.GpuKernel_init(C.byref(self.k), self.context.ctx, 1, srcs, lens,
                                 name.encode() if isinstance(name, str) else name,
                                 len(self._types), tarr, flags, C.byref(err_str))
        if err != _lib.GA_NO_ERROR:
            self.k = None
            log = err_str.value.decode(errors="replace") if err_str.value else ""
            try:
                check(err, self.context.ctx)
            except GpuArrayException as e:
                raise type(e)("%s\n%s" % (e.args[0], log), err)

    def __del__(self):
        k = getattr(self, "k", None)
        if k is not None:
            lib.GpuKernel_clear(C.byref(k))
            self.k = None

    def __reduce__(self):
        raise RuntimeError("Cannot pickle GpuKernel object")

    def _prop(self, prop_id, ctype):
        v = ctype()
        check(lib.gpukernel_property(self.k.k, prop_id, C.byref(v)), self.context.ctx)
        return v.value

    maxlsize = property(lambda s: s._prop(_lib.GA_KERNEL_PROP_MAXLSIZE, C.c_size_t))
    preflsize = property(lambda s: s._prop(_lib.GA_KERNEL_PROP_PREFLSIZE, C.c_size_t))
    numargs = property(lambda s: s._prop(_lib.GA_KERNEL_PROP_NUMARGS, C.c_uint))

    def __call__(self, *args, **kwargs):
        n, gs, ls = kwargs.pop("n", None), kwargs.pop("gs", None), kwargs.pop("ls", None)
        shared = kwargs.pop("shared", 0)
        if kwargs:
            raise TypeError("unexpected keyword arguments: %s" % (sorted(kwargs),))
        if n is None and (ls is None or gs is None):
            raise ValueError("Must specify size (n) or both gs and ls")
        lsz, gsz = (C.c_size_t * 3)(0, 1, 1), (C.c_size_t * 3)(0, 1, 1)
        if ls is None:
            nd = 1
        elif isinstance(ls, (int, np.integer)):
            lsz[0], nd = int(ls), 1
        elif isinstance(ls, (list, tuple)):
            if len(ls) > 3:
                raise ValueError("ls is not of length 3 or less")
            nd = len(ls)
            for i in range(nd):
                lsz[i] = int(ls[i])
        else:
            raise TypeError("ls is not int or list")
        if gs is None:
            if nd != 1:
                raise ValueError("nd mismatch for gs (None)")
        elif isinstance(gs, (int, np.integer)):
            if nd != 1:
                raise ValueError("nd mismatch for gs (int)")
            gsz[0] = int(gs)
        elif isinstance(gs, (list, tuple)):
            if len(gs) > 3:
                raise ValueError("gs is not of length 3 or less")
            if len(gs) != nd:
                raise ValueError("nd mismatch for gs (tuple)")
            for i in range(nd):
                gsz[i] = int(gs[i])
        else:
            raise TypeError("gs is not int or list")
        if len(args) != len(self._types):
            raise TypeError("Expected %d arguments, got %d," % (len(self._types), len(args)))
        keep = []
        ptrs = (C.c_void_p * max(len(args), 1))()
        for i, (t, dt, a) in enumerate(zip(self._types, self._dtypes, args)):
            if t == _lib.GA_BUFFER:
                if not isinstance(a, GpuArray):
                    raise TypeError("expected a GpuArray")
                ptrs[i] = a.ga.data
            else:
                v = np.asarray(a, dtype=dt).reshape(1).copy()
                keep.append(v)
                ptrs[i] = v.ctypes.data
        if n is not None:
            if nd != 1:
                raise ValueError("n is specified and nd != 1")
            check(lib.GpuKernel_sched(C.byref(self.k), int(n), gsz, lsz), self.context.ctx)
        check(lib.GpuKernel_call(C.byref(self.k), nd, gsz, lsz, int(shared), ptrs), self.context.ctx)


def _split(a, ind, axis):
    """reference pygpu/gpuarray.pyx:1467-1496: views of `a` cut along `axis`
    at the positions `ind` (capped at the extent)."""
    if not 0 <= axis < a.ndim:
        raise ValueError("split on non-existant axis")
    m = a.shape[axis]
    cuts = [min(int(v), m) for v in ind]
    res = [type(a)(a.context) for _ in range(len(cuts) + 1)]
    ptrs = (_lib.PA * len(res))(*[C.pointer(r.ga) for r in res])
    p = (C.c_size_t * max(len(cuts), 1))(*cuts)
    check(lib.GpuArray_split(ptrs, a._ptr(), len(cuts), p, axis), a.context.ctx)
    for r in res:
        r.base = a
    return res


def _concatenate(al, axis, restype, cls, context):
    """reference pygpu/gpuarray.pyx:1505-1522"""
    context = _ensure_context(context)
    for a in al:
        if not isinstance(a, GpuArray):
            raise TypeError("expected GpuArrays to concatenate")
    res = _make(cls, context)
    ptrs = (_lib.PA * len(al))(*[C.pointer(a.ga) for a in al])
    check(lib.GpuArray_concatenate(res._ptr(), ptrs, len(al), axis, restype), context.ctx)
    return res
