"""dtype helpers of the reference's Python layer (pygpu/dtypes.py:17-202):
C spellings of NumPy dtypes and NumPy's own promotion as the result-type rule."""
import numpy as np

_CTYPES = {"bool": "ga_bool", "int8": "ga_byte", "uint8": "ga_ubyte", "int16": "ga_short",
           "uint16": "ga_ushort", "int32": "ga_int", "uint32": "ga_uint", "int64": "ga_long",
           "uint64": "ga_ulong", "float16": "ga_half", "float32": "ga_float",
           "float64": "ga_double", "complex64": "ga_cfloat", "complex128": "ga_cdouble"}


def dtype_to_ctype(dtype):
    """reference pygpu/dtypes.py:78-93 (the cluda spelling of a dtype)"""
    dtype = np.dtype(dtype)
    try:
        return _CTYPES[dtype.name]
    except KeyError:
        raise ValueError("unable to map dtype: %s" % (dtype,))


def get_np_obj(obj):
    """A NumPy stand-in with the dtype and scalar-ness of `obj`, for asking
    NumPy what an operation's result type is (reference pygpu/dtypes.py:152-166).
    Python scalars are returned as they are so that NumPy applies its own rule
    for them."""
    if isinstance(obj, np.ndarray) and obj.shape == ():
        return obj
    if hasattr(obj, "dtype"):
        return np.ones(1, dtype=obj.dtype)
    return obj


def get_common_dtype(obj1, obj2, allow_double):
    """reference pygpu/dtypes.py:169-192"""
    result = np.asarray(get_np_obj(obj1) + get_np_obj(obj2)).dtype
    if not allow_double:
        if result == np.float64:
            result = np.dtype(np.float32)
        elif result == np.complex128:
            result = np.dtype(np.complex64)
    return result


def upcast(*args):
    """reference pygpu/dtypes.py:195-199"""
    a = np.array([0], dtype=args[0])
    for t in args[1:]:
        a = a + np.array([0], dtype=t)
    return a.dtype
