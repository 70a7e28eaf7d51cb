"""dtype helpers of the reference's Python layer (pygpu/dtypes.py:17-202):
C spellings of NumPy dtypes and NumPy's own promotion as the result-type rule."""
import numpy as np

_CTYPES = {"bool": "ga_bool", "int8": "ga_byte", "uint8": "ga_ubyte", "int16": "ga_short",
           "uint16": "ga_ushort", "int32": "ga_int", "uint32": "ga_uint", "int64": "ga_long",
           "uint64": "ga_ulong", "float16": "ga_half", "float32": "ga_float",
           "float64": "ga_double", "complex64": "ga_cfloat", "complex128": "ga_cdouble"}


_REGISTERED = {}     # dtype -> C name, for element types added with register_dtype
_BY_DTYPE = {}       # dtype object -> C name of a built-in type (dtype.name is slow to form)
NAME_TO_DTYPE = {}   # C spelling -> dtype, for parsing C argument lists


def dtype_to_ctype(dtype):
    """reference pygpu/dtypes.py:78-93 (the cluda spelling of a dtype)"""
    if dtype is None:
        raise ValueError("dtype may not be None")
    try:
        return _BY_DTYPE[dtype]        # the common case: a dtype object seen before
    except (KeyError, TypeError):
        pass
    dtype = np.dtype(dtype)
    if dtype in _REGISTERED:
        return _REGISTERED[dtype]
    try:
        res = _BY_DTYPE[dtype] = _CTYPES[dtype.name]
        return res
    except KeyError:
        raise ValueError("unable to map dtype: %s" % (dtype,))


def register_dtype(dtype, c_names):
    """Associate a dtype with its C spellings: the first one is what generated
    code uses, all of them map back to the dtype when a C argument list is
    parsed.  A dtype the library does not know yet is registered with it
    (reference pygpu/dtypes.py:38-70)."""
    if isinstance(c_names, str):
        c_names = [c_names]
    dtype = np.dtype(dtype)
    try:
        dtype_to_ctype(dtype)
    except ValueError:
        from . import gpuarray     # not at import time: that module imports this one
        gpuarray.register_dtype(dtype, c_names[0])
    for nm in c_names:
        if nm in NAME_TO_DTYPE and NAME_TO_DTYPE[nm] != dtype:
            raise RuntimeError("name '%s' already registered" % nm)
        NAME_TO_DTYPE[nm] = dtype


def _fill_dtype_registry():
    """The built-in spellings (reference pygpu/dtypes.py:73-97, plus half)."""
    for dt, names in (
            (np.bool_, ["ga_bool", "bool"]),
            (np.int8, ["ga_byte", "char", "signed char"]),
            (np.uint8, ["ga_ubyte", "unsigned char"]),
            (np.int16, ["ga_short", "short", "signed short", "signed short int", "short signed int"]),
            (np.uint16, ["ga_ushort", "unsigned short", "unsigned short int", "short unsigned int"]),
            (np.int32, ["ga_int", "int", "signed int"]),
            (np.uint32, ["ga_uint", "unsigned", "unsigned int"]),
            (np.int64, ["ga_long", "long", "long int", "signed long int", "long signed int",
                        "long long", "ga_ssize", "ssize_t"]),
            (np.uint64, ["ga_ulong", "unsigned long", "unsigned long int", "long unsigned int",
                         "unsigned long long", "ga_size", "size_t"]),
            (np.float16, ["ga_half", "half"]),
            (np.float32, ["ga_float", "float"]),
            (np.float64, ["ga_double", "double"])):
        register_dtype(dt, names)


def parse_c_arg_backend(c_arg, scalar_arg_class, vec_arg_class):
    """One C parameter declaration -> scalar_arg_class(dtype, name), or
    vec_arg_class(dtype, name) for a pointer or array declarator
    (reference pygpu/dtypes.py:120-147)."""
    import re
    c_arg = c_arg.replace("const", "").replace("volatile", "")
    m = re.search(r"(\**)\s*([_a-zA-Z0-9]+)(\s*\[[ 0-9]*\])*\s*$", c_arg)
    if m is None:
        raise ValueError("couldn't parse C declarator '%s'" % c_arg)
    tp = " ".join(c_arg[:m.start()].split())
    try:
        dtype = NAME_TO_DTYPE[tp]
    except KeyError:
        raise ValueError("unknown type '%s'" % tp)
    cls = vec_arg_class if (m.group(1) or m.group(3) is not None) else scalar_arg_class
    return cls(dtype, m.group(2))


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


_fill_dtype_registry()
