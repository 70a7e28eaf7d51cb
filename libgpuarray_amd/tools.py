"""Helpers for code that writes kernels over GpuArrays (reference pygpu/tools.py):
argument descriptors, the argument check with dimension collapsing and
broadcasting, a small least-recently-used cache decorator, and prod()."""
import functools

import numpy as np

from .dtypes import dtype_to_ctype
from .gpuarray import GpuArray


class Argument(object):
    """A named kernel argument of a dtype (reference pygpu/tools.py:22-37)."""

    def __init__(self, dtype, name):
        self.dtype = np.dtype(dtype)
        self.name = name

    def ctype(self):
        return dtype_to_ctype(self.dtype)

    def __hash__(self):
        return hash(type(self)) ^ hash(self.dtype) ^ hash(self.name)

    def __eq__(self, other):
        return type(self) == type(other) and self.dtype == other.dtype and self.name == other.name

    def __ne__(self, other):
        return not self == other

    def __repr__(self):
        return "%s(%s, %r)" % (type(self).__name__, self.dtype, self.name)


class ArrayArg(Argument):
    """reference pygpu/tools.py:40-51"""

    def decltype(self):
        return "GLOBAL_MEM %s *" % (self.ctype(),)

    def expr(self):
        return "%s[i]" % (self.name,)

    def isarray(self):
        return True

    def spec(self):
        return GpuArray


class ScalarArg(Argument):
    """reference pygpu/tools.py:54-65"""

    def decltype(self):
        return self.ctype()

    def expr(self):
        return self.name

    def isarray(self):
        return False

    def spec(self):
        return self.dtype


def as_argument(obj, name):
    """reference pygpu/tools.py:15-19"""
    if isinstance(obj, GpuArray):
        return ArrayArg(obj.dtype, name)
    return ScalarArg(np.asarray(obj).dtype, name)


def check_args(args, collapse=False, broadcast=False):
    """(n, nd, dims, strides per argument, offsets per argument) of a kernel's
    arguments; None stands in the last two for an argument that is no array
    (reference pygpu/tools.py:68-168).

    All arrays must have one rank, and one shape unless `broadcast`, which
    gives an extent of 1 a stride of 0 against a larger extent of another
    array.  `collapse` (None counts as True) drops extents of 1 and merges a
    dimension into the one before it wherever every array steps through both
    as through one; at least one dimension is kept."""
    if collapse is None:
        collapse = True
    arrays = [a for a in args if isinstance(a, GpuArray)]
    if not arrays:
        raise TypeError("No arrays in kernel arguments, something is wrong")
    nd = arrays[0].ndim
    dims = list(arrays[0].shape)
    for a in arrays[1:]:
        if a.ndim != nd:
            raise ValueError("Array order differs")
        if not broadcast and a.shape != arrays[0].shape:
            raise ValueError("Array shape differs")
    if broadcast:
        for a in arrays:
            for k, d in enumerate(a.shape):
                if dims[k] == 1:
                    dims[k] = d
    strs = []
    for a in args:
        if not isinstance(a, GpuArray):
            strs.append(None)
            continue
        st = list(a.strides)
        for k, d in enumerate(a.shape):
            if d != dims[k]:
                if d != 1:      # only reachable with broadcast
                    raise ValueError("Array shape differs")
                st[k] = 0
        strs.append(st)
    offsets = tuple(a.offset if isinstance(a, GpuArray) else None for a in args)
    n = 1
    for d in dims:
        n *= d

    if collapse and nd > 1:
        keep = [k for k in range(nd) if dims[k] != 1]
        if not keep:
            keep = [0]      # all ones: the first dimension stays
        dims = [dims[k] for k in keep]
        strs = [None if st is None else [st[k] for k in keep] for st in strs]
        live = [st for st in strs if st is not None]
        k = len(dims) - 1
        while k > 0:
            if all(st[k] * dims[k] == st[k - 1] for st in live):
                dims[k - 1] *= dims[k]
                del dims[k]
                for st in live:
                    st[k - 1] = st[k]
                    del st[k]
            k -= 1
        nd = len(dims)

    return (n, nd, tuple(dims),
            tuple(None if st is None else tuple(st) for st in strs), offsets)


def lru_cache(maxsize=20):
    """Decorator: remember results per positional-argument tuple; once more
    than `maxsize` are held, the least recently used tenth goes.  The wrapper
    carries hits, misses, maxsize, clear() and get(*key) (KeyError when the
    key is not held), as the reference's (pygpu/tools.py:171-218)."""
    def decorate(fn):
        held = {}       # key -> result; insertion order = recency (oldest first)

        def touch(key):
            held[key] = held.pop(key)

        @functools.wraps(fn)
        def wrapper(*key):
            if key in held:
                wrapper.hits += 1
                touch(key)
                return held[key]
            res = fn(*key)
            wrapper.misses += 1
            held[key] = res
            if len(held) > wrapper.maxsize:
                for old in list(held)[:wrapper.maxsize // 10]:
                    del held[old]
            return res

        @functools.wraps(fn)
        def get(*key):
            res = held[key]
            touch(key)
            wrapper.hits += 1
            return res

        def clear():
            held.clear()
            wrapper.hits = wrapper.misses = 0

        wrapper.hits = wrapper.misses = 0
        wrapper.maxsize = maxsize
        wrapper.clear = clear
        wrapper.get = get
        return wrapper
    return decorate


def prod(iterable):
    """Product of the items, 1 for none (reference pygpu/tools.py:221-222)."""
    res = 1
    for v in iterable:
        res *= v
    return res
