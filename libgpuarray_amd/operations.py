"""NumPy's split/stack family over GpuArray_split and GpuArray_concatenate
(reference pygpu/operations.py:8-142).  Splits are views; concatenation
allocates the result in the promoted type of its inputs."""
from .gpuarray import _split, _concatenate, dtype_to_typecode, asarray
from .dtypes import upcast


def _atleast(nd, arys):
    res = []
    for ary in arys:
        ary = asarray(ary)
        if nd >= 1 and ary.ndim == 0:
            ary = ary.reshape((1,) * nd)
        elif nd >= 2 and ary.ndim == 1:
            ary = ary.reshape((1, ary.shape[0]) + (1,) * (nd - 2))
        elif nd == 3 and ary.ndim == 2:
            ary = ary.reshape(ary.shape + (1,))
        res.append(ary)
    return res[0] if len(res) == 1 else res


def atleast_1d(*arys):
    return _atleast(1, arys)


def atleast_2d(*arys):
    return _atleast(2, arys)


def atleast_3d(*arys):
    return _atleast(3, arys)


def split(ary, indices_or_sections, axis=0):
    try:
        len(indices_or_sections)
    except TypeError:
        if ary.shape[axis] % indices_or_sections != 0:
            raise ValueError("array split does not result in an equal division")
    return array_split(ary, indices_or_sections, axis)


def array_split(ary, indices_or_sections, axis=0):
    if axis < 0:
        axis += ary.ndim
    if axis < 0:
        raise ValueError("axis out of bounds")
    try:
        indices = list(indices_or_sections)
    except TypeError:
        nsec = int(indices_or_sections)
        if nsec <= 0:
            raise ValueError("number of sections must be larger than 0.")
        neach, extra = divmod(ary.shape[axis], nsec)
        # the first `extra` sections get one element more, as NumPy does
        indices = (list(range(neach + 1, (neach + 1) * extra + 1, neach + 1)) +
                   list(range((neach + 1) * extra + neach, ary.shape[axis], neach)))
    return _split(ary, indices, axis)


def hsplit(ary, indices_or_sections):
    if ary.ndim == 0:
        raise ValueError("hsplit only works on arrays of 1 or more dimensions")
    return split(ary, indices_or_sections, axis=1 if ary.ndim > 1 else 0)


def vsplit(ary, indices_or_sections):
    if ary.ndim < 2:
        raise ValueError("vsplit only works on arrays of 2 or more dimensions")
    return split(ary, indices_or_sections, axis=0)


def dsplit(ary, indices_or_sections):
    if ary.ndim < 3:
        raise ValueError("dsplit only works on arrays of 3 or more dimensions")
    return split(ary, indices_or_sections, axis=2)


def concatenate(arys, axis=0, context=None):
    if len(arys) == 0:
        raise ValueError("concatenation of zero-length sequences is impossible")
    al = [asarray(a, context=context) for a in arys]
    if axis < 0:
        axis += al[0].ndim
    if axis < 0:
        raise ValueError("axis out of bounds")
    if context is None:
        context = al[0].context
    outtype = upcast(*[a.dtype for a in al])
    return _concatenate(al, axis, dtype_to_typecode(outtype), type(al[0]), context)


def vstack(tup, context=None):
    return concatenate([atleast_2d(a) for a in tup], 0, context)


def hstack(tup, context=None):
    tup = [atleast_1d(a) for a in tup]
    return concatenate(tup, 0 if tup[0].ndim == 1 else 1, context)


def dstack(tup, context=None):
    return concatenate([atleast_3d(a) for a in tup], 2, context)
