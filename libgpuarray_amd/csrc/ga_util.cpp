// Feature flags, dimension collapsing, host half conversion.
#include "private.hpp"

// Which GA_USE_* a typecode needs (reference src/gpuarray_util.c:111-122):
// double/cdouble -> DOUBLE, half -> HALF, cfloat/cdouble -> COMPLEX, and any
// type narrower than 4 bytes -> SMALL.
static int flags_of(int typecode) {
  int fl = 0;
  if (typecode == GA_DOUBLE || typecode == GA_CDOUBLE) fl |= GA_USE_DOUBLE;
  if (typecode == GA_HALF) fl |= GA_USE_HALF;
  if (typecode == GA_CFLOAT || typecode == GA_CDOUBLE) fl |= GA_USE_COMPLEX;
  if (gpuarray_get_elsize(typecode) < 4) fl |= GA_USE_SMALL;
  return fl;
}

extern "C" int gpuarray_type_flags(int init, ...) {
  va_list ap;
  int fl = 0;
  va_start(ap, init);
  for (int tc = init; tc != -1; tc = va_arg(ap, int)) fl |= flags_of(tc);
  va_end(ap);
  return fl;
}

extern "C" int gpuarray_type_flagsa(unsigned int n, gpuelemwise_arg *args) {
  int fl = 0;
  for (unsigned int i = 0; i < n; i++) fl |= flags_of(args[i].typecode);
  return fl;
}

// Remove entry i from a row of length nd.
template <typename T> static void drop(T *row, unsigned int i, unsigned int nd) {
  if (row) memmove(row + i, row + i + 1, (nd - i - 1) * sizeof(T));
}

// Reference src/gpuarray_util.c:153-188: first delete size-1 dims (walking
// from the last dim, never going below one dim), then, from the last pair
// to the first, fuse dim i into dim i-1 when every array steps over dim i-1
// exactly dims[i] times its step over dim i.  NULL stride rows are skipped.
extern "C" void gpuarray_elemwise_collapse(unsigned int n, unsigned int *_nd,
                                           size_t *dims, ssize_t **strs) {
  unsigned int nd = *_nd;
  for (unsigned int i = nd; i > 0; i--) {
    if (nd > 1 && dims[i - 1] == 1) {
      drop(dims, i - 1, nd);
      for (unsigned int k = 0; k < n; k++) drop(strs[k], i - 1, nd);
      nd--;
    }
  }
  for (unsigned int i = nd ? nd - 1 : 0; i > 0; i--) {
    bool fuse = true;
    for (unsigned int k = 0; k < n && fuse; k++)
      fuse = strs[k] == nullptr ||
             strs[k][i - 1] == (ssize_t)dims[i] * strs[k][i];
    if (!fuse) continue;
    dims[i - 1] *= dims[i];
    drop(dims, i, nd);
    for (unsigned int k = 0; k < n; k++) {
      if (strs[k] == nullptr) continue;
      strs[k][i - 1] = strs[k][i];
      drop(strs[k], i, nd);
    }
    nd--;
  }
  *_nd = nd;
}

// Reference src/gpuarray/util.h:107-183.  Three ranges by the float's biased
// exponent field E (bits 30..23 kept in place):
//   E >= 0x47800000 (|f| >= 65536, inf, nan): inf, or a NaN that keeps the
//       top payload bits and is forced non-zero;
//   E <= 0x38000000 (|f| < 2^-14): subnormal half; below 2^-25 it is zero;
//       the implicit bit is restored, the value shifted into place and the
//       bit under the kept mantissa added before truncation;
//   otherwise: rebias, add the bit under the kept mantissa, truncate; a carry
//       out of the mantissa correctly bumps the exponent (and can reach inf).
extern "C" ga_half_t gpuarray_float2half(float f) {
  uint32_t bits;
  memcpy(&bits, &f, 4);
  ga_half_t out;
  const uint16_t sign = (uint16_t)((bits & 0x80000000u) >> 16);
  const uint32_t e = bits & 0x7f800000u;
  uint32_t m = bits & 0x007fffffu;

  if (e >= 0x47800000u) {
    if (e == 0x7f800000u && m != 0) {
      uint16_t r = (uint16_t)(0x7c00u + (m >> 13));
      if (r == 0x7c00u) r++;
      out.h = (uint16_t)(r + sign);
    } else {
      out.h = (uint16_t)(sign + 0x7c00u);
    }
    return out;
  }
  if (e <= 0x38000000u) {
    if (e < 0x33000000u) {
      out.h = sign;
      return out;
    }
    uint32_t sig = (0x00800000u + m) >> (113 - (e >> 23));
    sig += 0x00001000u;
    out.h = (uint16_t)(sign + (uint16_t)(sig >> 13));
    return out;
  }
  const uint16_t he = (uint16_t)((e - 0x38000000u) >> 13);
  m += 0x00001000u;
  out.h = (uint16_t)(sign + he + (uint16_t)(m >> 13));
  return out;
}

extern "C" float gpuarray_half2float(ga_half_t h) {
  const uint32_t sign = (uint32_t)(h.h & 0x8000u) << 16;
  uint32_t e = (h.h >> 10) & 0x1f;
  uint32_t m = h.h & 0x3ffu;
  uint32_t bits;
  if (e == 0x1f) {
    bits = sign | 0x7f800000u | (m << 13);
  } else if (e == 0) {
    if (m == 0) {
      bits = sign;
    } else {
      // normalise the subnormal
      int shift = 0;
      while (!(m & 0x400u)) { m <<= 1; shift++; }
      m &= 0x3ffu;
      bits = sign | ((uint32_t)(113 - shift) << 23) | (m << 13);
    }
  } else {
    bits = sign | ((e + 112) << 23) | (m << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}
