"""MI355X-native elementwise and reduction engine behind the libgpuarray C API.

`libgpuarray.so` (built from csrc/) is the product; the modules here mirror
the part of the reference's Python layer that drives this path:

  gpuarray   contexts and strided arrays   (pygpu/gpuarray.pyx, pygpu/_array.py)
  elemwise   GpuElemwise and helpers       (pygpu/_elemwise.pyx, pygpu/elemwise.py)
  reduction  sum/prod/all/any/min/max/arg* (pygpu/reduction.py, pygpu/_array.py)
"""
from . import _lib
from ._lib import GpuArrayException, UnsupportedException, LIB_PATH
from . import gpuarray, elemwise, reduction
from .gpuarray import (GpuContext, GpuArray, init, array, asarray, empty, zeros,
                       set_default_context, get_default_context, count_devices)
from .elemwise import GpuElemwise, arg, elemwise1, elemwise2
from .reduction import GpuReduction

__all__ = ["GpuContext", "GpuArray", "GpuElemwise", "GpuReduction", "arg", "init", "array",
           "asarray", "empty", "zeros", "gpuarray", "elemwise", "reduction",
           "GpuArrayException", "UnsupportedException"]
