"""triu / tril on contiguous 2-D arrays with a hand-passed kernel text, the
reference's example of the raw GpuKernel interface (pygpu/basic.py:5-77)."""
import numpy as np

from .gpuarray import GpuArray, GpuKernel
from .dtypes import dtype_to_ctype

_TMPL = """
#include "cluda.h"
KERNEL void extract_tri(GLOBAL_MEM %(ctype)s *a, ga_size a_off, ga_uint N) {
  a = (GLOBAL_MEM %(ctype)s *)(((GLOBAL_MEM char *)a) + a_off);
  unsigned int idx = GID_1 * LDIM_0 * GDIM_0 + GID_0 * LDIM_0 + LID_0;
  unsigned int ix = idx / %(cols)d;
  unsigned int iy = idx %% %(cols)d;
  if (idx < N) {
    if (ix %(le)s iy) a[idx] = 0;
  }
}
"""


def _generate_kernel(ctx, cols, dtype, upper=True):
    dtype = np.dtype(dtype)
    ctype = "ga_ushort" if dtype == np.float16 else dtype_to_ctype(dtype)   # zero has all bits clear
    src = _TMPL % {"cols": cols, "ctype": ctype, "le": ">" if upper else "<"}
    return GpuKernel(src, "extract_tri", [GpuArray, "uint64", "uint32"], context=ctx,
                     have_double=dtype in (np.float64, np.complex128),
                     have_small=dtype.itemsize < 4,
                     have_complex=dtype in (np.complex64, np.complex128))


def _tri(A, inplace, want_upper):
    if A.ndim != 2:
        raise ValueError("%s only works for 2d arrays" % ("triu" if want_upper else "tril"))
    if not (A.flags.c_contiguous or A.flags.f_contiguous):
        raise ValueError("%s only works for contiguous arrays" % ("triu" if want_upper else "tril"))
    if not inplace:
        A = A.copy("C" if A.flags.c_contiguous else "F")
    if A.flags.c_contiguous:
        upper, cols = want_upper, A.shape[1]
    else:
        upper, cols = not want_upper, A.shape[0]
    n = A.shape[0] * A.shape[1]
    if n:
        _generate_kernel(A.context, cols, A.dtype, upper)(A, A.offset, n, n=n)
    return A


def triu(A, inplace=True):
    return _tri(A, inplace, True)


def tril(A, inplace=True):
    return _tri(A, inplace, False)
