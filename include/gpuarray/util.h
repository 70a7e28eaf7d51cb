/* Type table access, feature flags, dimension collapsing, float->half.
 * Same entry points as the reference's src/gpuarray/util.h:35-183
 * (impl src/gpuarray_util.c:24-188). */
#ifndef GPUARRAY_UTIL
#define GPUARRAY_UTIL

#include <gpuarray/config.h>
#include <gpuarray/elemwise.h>
#include <gpuarray/types.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Register a user type; returns its new typecode (>= 512) or -1. */
GPUARRAY_PUBLIC int gpuarray_register_type(gpuarray_type *t, int *ret);
/* Never NULL: unknown codes give a row with typecode -1 and size 0. */
GPUARRAY_PUBLIC const gpuarray_type *gpuarray_get_type(int typecode);
GPUARRAY_PUBLIC size_t gpuarray_get_elsize(int typecode);

/* OR of GA_USE_* needed by the listed typecodes; the list ends with -1. */
GPUARRAY_PUBLIC int gpuarray_type_flags(int init, ...);
GPUARRAY_PUBLIC int gpuarray_type_flagsa(unsigned int n, gpuelemwise_arg *arg);

/* Drop size-1 dims, then merge neighbouring dims that every array walks as
 * one run (ref util.h:75-99).  n arrays; strs[k] may be NULL (scalar).
 * *nd, dims and strs are updated in place; strides are in bytes. */
GPUARRAY_PUBLIC void gpuarray_elemwise_collapse(unsigned int n,
                                                unsigned int *nd, size_t *dim,
                                                ssize_t **strs);

typedef struct _ga_half_t { uint16_t h; } ga_half_t;

/* Host float -> IEEE binary16 with the reference's rounding
 * (ref util.h:107-183): the bit below the kept mantissa is added, i.e. ties
 * round away from zero in magnitude; overflow gives infinity; values below
 * the smallest subnormal flush to signed zero. */
GPUARRAY_PUBLIC ga_half_t gpuarray_float2half(float f);
static inline ga_half_t ga_float2half(float f) { return gpuarray_float2half(f); }
/* Host binary16 -> float (exact). */
GPUARRAY_PUBLIC float gpuarray_half2float(ga_half_t h);

#ifdef __cplusplus
}
#endif
#endif
