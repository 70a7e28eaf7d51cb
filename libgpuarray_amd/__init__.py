"""MI355X-native elementwise and reduction engine behind the libgpuarray C API.

`libgpuarray.so` (built from csrc/) is the product; the modules here mirror
the part of the reference's Python layer that drives this path:

  gpuarray   contexts and strided arrays   (pygpu/gpuarray.pyx, pygpu/_array.py)
  elemwise   GpuElemwise and helpers       (pygpu/_elemwise.pyx, pygpu/elemwise.py)
  reduction  sum/prod/all/any/min/max/arg* (pygpu/reduction.py, pygpu/_array.py)
  _array     ndgpuarray: NumPy operators   (pygpu/_array.py)
  dtypes     C spellings, promotion        (pygpu/dtypes.py)
  operations split / stack family          (pygpu/operations.py)
  basic      triu / tril via GpuKernel     (pygpu/basic.py)
  tools      argument descriptors, check_args, lru_cache (pygpu/tools.py)
"""
from . import _lib
from ._lib import GpuArrayException, UnsupportedException, LIB_PATH
from . import gpuarray, elemwise, reduction, operations, basic, tools
from .gpuarray import (GpuContext, GpuArray, GpuKernel, init, array, asarray, empty, zeros, zeros_like,
                       empty_like, ascontiguousarray, asfortranarray, may_share_memory,
                       set_default_context, get_default_context, count_devices, count_platforms,
                       from_gpudata, register_dtype, api_version, abi_version)
from .elemwise import GpuElemwise, arg, as_argument, elemwise1, elemwise2, ielemwise2, compare
from .reduction import GpuReduction, ReductionKernel
from ._array import ndgpuarray

__all__ = ["GpuContext", "GpuArray", "ndgpuarray", "GpuElemwise", "GpuReduction", "ReductionKernel",
           "arg", "as_argument", "elemwise1", "elemwise2", "ielemwise2", "compare", "init", "array",
           "asarray", "empty", "zeros", "gpuarray", "elemwise", "reduction",
           "GpuArrayException", "UnsupportedException"]
