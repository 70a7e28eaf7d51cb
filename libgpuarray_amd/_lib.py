"""ctypes view of libgpuarray.so: the C ABI declared in include/gpuarray/*.h.

Nothing here computes anything.  If the shared object is missing the import
fails loudly: there is no fallback path.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# GPUARRAY_LIBRARY names another build of the same library (the DEBUG and
# sanitizer variants of csrc/Makefile); there is no other implementation.
LIB_PATH = os.environ.get("GPUARRAY_LIBRARY") or os.path.join(_HERE, "libgpuarray.so")

if not os.path.exists(LIB_PATH):
    raise ImportError(
        "%s is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
        "or `make -C libgpuarray_amd/csrc`" % LIB_PATH)

lib = C.CDLL(LIB_PATH)

c_ssize_t = C.c_ssize_t

# ---- constants (include/gpuarray/*.h) -------------------------------------
GA_NO_ERROR = 0
GA_MEMORY_ERROR = 1
GA_VALUE_ERROR = 2
GA_IMPL_ERROR = 3
GA_INVALID_ERROR = 4
GA_UNSUPPORTED_ERROR = 5
GA_SYS_ERROR = 6
GA_DEVSUP_ERROR = 8
GA_UNALIGNED_ERROR = 12
GA_COPY_ERROR = 13
GA_NODEV_ERROR = 14
GA_XLARGE_ERROR = 17

GA_BUFFER = -1
GA_BOOL, GA_BYTE, GA_UBYTE, GA_SHORT, GA_USHORT = 0, 1, 2, 3, 4
GA_INT, GA_UINT, GA_LONG, GA_ULONG = 5, 6, 7, 8
GA_FLOAT, GA_DOUBLE, GA_CFLOAT, GA_CDOUBLE = 11, 12, 14, 15
GA_HALF, GA_SIZE, GA_SSIZE = 23, 24, 25

GA_C_CONTIGUOUS = 0x0001
GA_F_CONTIGUOUS = 0x0002
GA_ALIGNED = 0x0100
GA_WRITEABLE = 0x0400

GA_ANY_ORDER, GA_C_ORDER, GA_F_ORDER = -1, 0, 1

GE_SCALAR, GE_READ, GE_WRITE = 0x0001, 0x0002, 0x0004
GE_NOADDR64, GE_CONVERT_F16 = 0x0001, 0x0002
GE_BROADCAST, GE_NOCOLLAPSE, GE_PADSHAPE = 0x0100, 0x0200, 0x0400

GA_USE_SMALL, GA_USE_DOUBLE, GA_USE_COMPLEX, GA_USE_HALF = 0x02, 0x04, 0x08, 0x10
GA_USE_CUDA, GA_USE_OPENCL = 0x2000, 0x4000

GA_BUFFER_INIT = 0x04

GA_CTX_PROP_DEVNAME = 1
GA_CTX_PROP_LMEMSIZE = 3
GA_CTX_PROP_NUMPROCS = 4
GA_CTX_PROP_BIN_ID = 7
GA_CTX_PROP_ERRBUF = 8
GA_CTX_PROP_TOTAL_GMEM = 9
GA_CTX_PROP_FREE_GMEM = 10
GA_CTX_PROP_MAXGSIZE0 = 12
GA_CTX_PROP_MAXLSIZE0 = 15
GA_CTX_PROP_MAXGSIZE1 = 13
GA_CTX_PROP_MAXGSIZE2 = 14
GA_CTX_PROP_MAXLSIZE1 = 16
GA_CTX_PROP_MAXLSIZE2 = 17
GA_CTX_PROP_UNIQUE_ID = 19
GA_CTX_PROP_LARGEST_MEMBLOCK = 20
GPUARRAY_API_VERSION = 2       # include/gpuarray/config.h
GPUARRAY_ABI_VERSION = 3000    # include/gpuarray/abi_version.h
GA_BUFFER_PROP_REFCNT = 513
GA_BUFFER_PROP_SIZE = 514
GA_KERNEL_PROP_MAXLSIZE = 1025
GA_KERNEL_PROP_PREFLSIZE = 1026
GA_KERNEL_PROP_NUMARGS = 1027

(GA_REDUCE_SUM, GA_REDUCE_PROD, GA_REDUCE_PRODNZ, GA_REDUCE_MIN, GA_REDUCE_MAX,
 GA_REDUCE_ARGMIN, GA_REDUCE_ARGMAX, GA_REDUCE_MINANDARGMIN, GA_REDUCE_MAXANDARGMAX,
 GA_REDUCE_AND, GA_REDUCE_OR, GA_REDUCE_XOR, GA_REDUCE_ALL, GA_REDUCE_ANY,
 GA_REDUCE_CUSTOM) = range(15)


# ---- structs -----------------------------------------------------------------
class GpuArrayStruct(C.Structure):
    _fields_ = [("data", C.c_void_p),
                ("dimensions", C.POINTER(C.c_size_t)),
                ("strides", C.POINTER(c_ssize_t)),
                ("offset", C.c_size_t),
                ("nd", C.c_uint),
                ("flags", C.c_int),
                ("typecode", C.c_int)]


class GpuKernelStruct(C.Structure):
    _fields_ = [("k", C.c_void_p), ("args", C.POINTER(C.c_void_p))]


class ElemwiseArg(C.Structure):
    _fields_ = [("name", C.c_char_p), ("typecode", C.c_int), ("flags", C.c_int)]


class GpuArrayType(C.Structure):
    _fields_ = [("cluda_name", C.c_char_p), ("size", C.c_size_t),
                ("align", C.c_size_t), ("typecode", C.c_int)]


class HalfT(C.Structure):
    _fields_ = [("h", C.c_uint16)]


PA = C.POINTER(GpuArrayStruct)
P_SIZE = C.POINTER(C.c_size_t)
P_SSIZE = C.POINTER(c_ssize_t)

# Every public symbol with its signature; the load test walks this table.
SIGNATURES = {
    # error.h
    "gpuarray_error_str": (C.c_char_p, [C.c_int]),
    # util.h
    "gpuarray_register_type": (C.c_int, [C.POINTER(GpuArrayType), C.POINTER(C.c_int)]),
    "gpuarray_get_type": (C.POINTER(GpuArrayType), [C.c_int]),
    "gpuarray_get_elsize": (C.c_size_t, [C.c_int]),
    "gpuarray_type_flags": (C.c_int, None),  # variadic
    "gpuarray_type_flagsa": (C.c_int, [C.c_uint, C.POINTER(ElemwiseArg)]),
    "gpuarray_elemwise_collapse": (None, [C.c_uint, C.POINTER(C.c_uint), P_SIZE,
                                          C.POINTER(P_SSIZE)]),
    "gpuarray_float2half": (HalfT, [C.c_float]),
    "gpuarray_half2float": (C.c_float, [HalfT]),
    # extension.h
    "gpuarray_get_extension": (C.c_void_p, [C.c_char_p]),
    # buffer.h
    "gpu_get_platform_count": (C.c_int, [C.c_char_p, C.POINTER(C.c_uint)]),
    "gpu_get_device_count": (C.c_int, [C.c_char_p, C.c_uint, C.POINTER(C.c_uint)]),
    "gpucontext_props_new": (C.c_int, [C.POINTER(C.c_void_p)]),
    "gpucontext_props_hip_dev": (C.c_int, [C.c_void_p, C.c_int]),
    "gpucontext_props_cuda_dev": (C.c_int, [C.c_void_p, C.c_int]),
    "gpucontext_props_opencl_dev": (C.c_int, [C.c_void_p, C.c_int, C.c_int]),
    "gpucontext_props_sched": (C.c_int, [C.c_void_p, C.c_int]),
    "gpucontext_props_set_single_stream": (C.c_int, [C.c_void_p]),
    "gpucontext_props_kernel_cache": (C.c_int, [C.c_void_p, C.c_char_p]),
    "gpucontext_props_alloc_cache": (C.c_int, [C.c_void_p, C.c_size_t, C.c_size_t]),
    "gpucontext_props_del": (None, [C.c_void_p]),
    "gpucontext_init": (C.c_int, [C.POINTER(C.c_void_p), C.c_char_p, C.c_void_p]),
    "gpucontext_deref": (None, [C.c_void_p]),
    "gpucontext_property": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p]),
    "gpucontext_error": (C.c_char_p, [C.c_void_p, C.c_int]),
    "gpudata_alloc": (C.c_void_p, [C.c_void_p, C.c_size_t, C.c_void_p, C.c_int,
                                   C.POINTER(C.c_int)]),
    "gpudata_retain": (None, [C.c_void_p]),
    "gpudata_release": (None, [C.c_void_p]),
    "gpudata_share": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(C.c_int)]),
    "gpudata_move": (C.c_int, [C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t]),
    "gpudata_transfer": (C.c_int, [C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t]),
    "gpudata_read": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t]),
    "gpudata_write": (C.c_int, [C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t]),
    "gpudata_memset": (C.c_int, [C.c_void_p, C.c_size_t, C.c_int]),
    "gpudata_sync": (C.c_int, [C.c_void_p]),
    "gpudata_property": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p]),
    "gpudata_context": (C.c_void_p, [C.c_void_p]),
    "gpukernel_init": (C.c_void_p, [C.c_void_p, C.c_uint, C.POINTER(C.c_char_p), P_SIZE,
                                    C.c_char_p, C.c_uint, C.POINTER(C.c_int), C.c_int,
                                    C.POINTER(C.c_int), C.POINTER(C.c_char_p)]),
    "gpukernel_retain": (None, [C.c_void_p]),
    "gpukernel_release": (None, [C.c_void_p]),
    "gpukernel_setarg": (C.c_int, [C.c_void_p, C.c_uint, C.c_void_p]),
    "gpukernel_call": (C.c_int, [C.c_void_p, C.c_uint, P_SIZE, P_SIZE, C.c_size_t,
                                 C.POINTER(C.c_void_p)]),
    "gpukernel_property": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p]),
    "gpukernel_context": (C.c_void_p, [C.c_void_p]),
    # kernel.h
    "GpuKernel_init": (C.c_int, [C.POINTER(GpuKernelStruct), C.c_void_p, C.c_uint,
                                 C.POINTER(C.c_char_p), P_SIZE, C.c_char_p, C.c_uint,
                                 C.POINTER(C.c_int), C.c_int, C.POINTER(C.c_char_p)]),
    "GpuKernel_clear": (None, [C.POINTER(GpuKernelStruct)]),
    "GpuKernel_context": (C.c_void_p, [C.POINTER(GpuKernelStruct)]),
    "GpuKernel_setarg": (C.c_int, [C.POINTER(GpuKernelStruct), C.c_uint, C.c_void_p]),
    "GpuKernel_sched": (C.c_int, [C.POINTER(GpuKernelStruct), C.c_size_t, P_SIZE, P_SIZE]),
    "GpuKernel_call": (C.c_int, [C.POINTER(GpuKernelStruct), C.c_uint, P_SIZE, P_SIZE,
                                 C.c_size_t, C.POINTER(C.c_void_p)]),
    "GpuKernel_error": (C.c_char_p, [C.POINTER(GpuKernelStruct), C.c_int]),
    # array.h
    "GpuArray_fix_flags": (None, [PA]),
    "GpuArray_empty": (C.c_int, [PA, C.c_void_p, C.c_int, C.c_uint, P_SIZE, C.c_int]),
    "GpuArray_zeros": (C.c_int, [PA, C.c_void_p, C.c_int, C.c_uint, P_SIZE, C.c_int]),
    "GpuArray_fromdata": (C.c_int, [PA, C.c_void_p, C.c_size_t, C.c_int, C.c_uint, P_SIZE,
                                    P_SSIZE, C.c_int]),
    "GpuArray_view": (C.c_int, [PA, PA]),
    "GpuArray_sync": (C.c_int, [PA]),
    "GpuArray_index": (C.c_int, [PA, PA, P_SSIZE, P_SSIZE, P_SSIZE]),
    "GpuArray_index_inplace": (C.c_int, [PA, P_SSIZE, P_SSIZE, P_SSIZE]),
    "GpuArray_take1": (C.c_int, [PA, PA, PA, C.c_int]),
    "GpuArray_setarray": (C.c_int, [PA, PA]),
    "GpuArray_reshape": (C.c_int, [PA, PA, C.c_uint, P_SIZE, C.c_int, C.c_int]),
    "GpuArray_reshape_inplace": (C.c_int, [PA, C.c_uint, P_SIZE, C.c_int]),
    "GpuArray_transpose": (C.c_int, [PA, PA, C.POINTER(C.c_uint)]),
    "GpuArray_transpose_inplace": (C.c_int, [PA, C.POINTER(C.c_uint)]),
    "GpuArray_clear": (None, [PA]),
    "GpuArray_share": (C.c_int, [PA, PA]),
    "GpuArray_context": (C.c_void_p, [PA]),
    "GpuArray_move": (C.c_int, [PA, PA]),
    "GpuArray_write": (C.c_int, [PA, C.c_void_p, C.c_size_t]),
    "GpuArray_read": (C.c_int, [C.c_void_p, C.c_size_t, PA]),
    "GpuArray_memset": (C.c_int, [PA, C.c_int]),
    "GpuArray_copy": (C.c_int, [PA, PA, C.c_int]),
    "GpuArray_transfer": (C.c_int, [PA, PA]),
    "GpuArray_split": (C.c_int, [C.POINTER(PA), PA, C.c_size_t, P_SIZE, C.c_uint]),
    "GpuArray_concatenate": (C.c_int, [PA, C.POINTER(PA), C.c_size_t, C.c_uint, C.c_int]),
    "GpuArray_error": (C.c_char_p, [PA, C.c_int]),
    "GpuArray_fprintf": (None, [C.c_void_p, PA]),
    "GpuArray_fdump": (C.c_int, [C.c_void_p, PA]),
    "GpuArray_maxandargmax": (C.c_int, [PA, PA, PA, C.c_uint, C.POINTER(C.c_uint)]),
    # elemwise.h
    "GpuElemwise_new": (C.c_void_p, [C.c_void_p, C.c_char_p, C.c_char_p, C.c_uint,
                                     C.POINTER(ElemwiseArg), C.c_uint, C.c_int]),
    "GpuElemwise_free": (None, [C.c_void_p]),
    "GpuElemwise_call": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p), C.c_int]),
    # reduction.h
    "GpuReduction_new": (C.c_int, [C.POINTER(C.c_void_p), C.c_void_p, C.c_int, C.c_uint,
                                   C.c_uint, C.c_int, C.c_int]),
    "GpuReduction_new_map": (C.c_int, [C.POINTER(C.c_void_p), C.c_void_p, C.c_int, C.c_char_p,
                                       C.c_char_p, C.c_int, C.c_char_p, C.c_char_p, C.c_uint,
                                       C.c_void_p, C.c_int]),
    "GpuReduction_call_map": (C.c_int, [C.c_void_p, PA, PA, C.POINTER(C.c_void_p), C.c_uint,
                                        C.POINTER(C.c_int), C.c_int]),
    "GpuReduction_free": (None, [C.c_void_p]),
    "GpuReduction_call": (C.c_int, [C.c_void_p, PA, PA, PA, C.c_uint, C.POINTER(C.c_int),
                                    C.c_int]),
    "GpuReduction_call_noalloc": (C.c_int, [C.c_void_p, PA, PA, PA, C.c_uint, C.POINTER(C.c_int),
                                            C.c_int]),
}

for _name, (_res, _args) in SIGNATURES.items():
    _fn = getattr(lib, _name)   # AttributeError here = symbol missing from the .so
    _fn.restype = _res
    if _args is not None:
        _fn.argtypes = _args


class GpuArrayException(Exception):
    """An entry point returned an error code (reference: pygpu.gpuarray.GpuArrayException)."""

    def __init__(self, msg, code):
        Exception.__init__(self, msg)
        self.code = code


class UnsupportedException(GpuArrayException):
    pass


def check(err, ctx=None):
    """Raise for a non-zero return code, with the context's message."""
    if err == GA_NO_ERROR:
        return
    msg = lib.gpucontext_error(ctx, err)
    base = lib.gpuarray_error_str(err).decode()
    text = "%s: %s" % (base, msg.decode(errors="replace") if msg else "")
    if err in (GA_UNSUPPORTED_ERROR, GA_DEVSUP_ERROR):
        raise UnsupportedException(text, err)
    if err == GA_VALUE_ERROR:
        raise ValueErrorGA(text, err)
    raise GpuArrayException(text, err)


class ValueErrorGA(GpuArrayException, ValueError):
    """GA_VALUE_ERROR; also a ValueError, as pygpu raises for shape mismatches."""


def extension(name, restype, argtypes):
    """Typed function pointer for a backend hook (include/gpuarray/ext_hip.h)."""
    addr = lib.gpuarray_get_extension(name.encode())
    if not addr:
        raise GpuArrayException("extension %s not available" % name, GA_INVALID_ERROR)
    return C.CFUNCTYPE(restype, *argtypes)(addr)
