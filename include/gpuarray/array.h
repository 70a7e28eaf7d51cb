/* GpuArray: a strided view over a device buffer, plus the operations on it.
 * Layout, flag values and entry points follow the reference's
 * src/gpuarray/array.h:21-644 (impl src/gpuarray_array.c).
 * Strides and offset are in BYTES everywhere. */
#ifndef GPUARRAY_ARRAY_H
#define GPUARRAY_ARRAY_H

#include <gpuarray/buffer.h>
#include <gpuarray/util.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct _GpuArray {
  gpudata *data;        /* retained buffer */
  size_t *dimensions;   /* nd extents, owned */
  ssize_t *strides;     /* nd byte strides, owned */
  size_t offset;        /* byte offset of element (0,..,0) in data */
  unsigned int nd;
  int flags;            /* GA_* below */
  int typecode;
#define GA_C_CONTIGUOUS 0x0001
#define GA_F_CONTIGUOUS 0x0002
#define GA_ALIGNED      0x0100
#define GA_WRITEABLE    0x0400
#define GA_BEHAVED      (GA_ALIGNED | GA_WRITEABLE)
#define GA_CARRAY       (GA_C_CONTIGUOUS | GA_BEHAVED)
#define GA_FARRAY       (GA_F_CONTIGUOUS | GA_BEHAVED)
} GpuArray;

typedef enum _ga_order { GA_ANY_ORDER = -1, GA_C_ORDER = 0, GA_F_ORDER = 1 } ga_order;

static inline int GpuArray_CHKFLAGS(const GpuArray *a, int flags) {
  return (a->flags & flags) == flags;
}
#define GpuArray_ISWRITEABLE(a)     GpuArray_CHKFLAGS(a, GA_WRITEABLE)
#define GpuArray_ISALIGNED(a)       GpuArray_CHKFLAGS(a, GA_ALIGNED)
#define GpuArray_ISONESEGMENT(a)    ((a)->flags & (GA_C_CONTIGUOUS | GA_F_CONTIGUOUS))
#define GpuArray_IS_C_CONTIGUOUS(a) ((a)->flags & GA_C_CONTIGUOUS)
#define GpuArray_IS_F_CONTIGUOUS(a) ((a)->flags & GA_F_CONTIGUOUS)
#define GpuArray_ISFORTRAN(a)       (GpuArray_CHKFLAGS(a, GA_F_CONTIGUOUS))
#define GpuArray_ITEMSIZE(a)        gpuarray_get_elsize((a)->typecode)

/* Recompute contiguity/alignment flags from dims and strides, keeping only
 * GA_WRITEABLE (ref array.h:194-204, src/gpuarray_array.c:91-98).
 * Size-1 dims never break contiguity. */
GPUARRAY_PUBLIC void GpuArray_fix_flags(GpuArray *a);

/* Allocation and wrapping (ref array.h:206-296). */
GPUARRAY_PUBLIC int GpuArray_empty(GpuArray *a, gpucontext *ctx, int typecode,
                                   unsigned int nd, const size_t *dims,
                                   ga_order ord);
GPUARRAY_PUBLIC int GpuArray_zeros(GpuArray *a, gpucontext *ctx, int typecode,
                                   unsigned int nd, const size_t *dims,
                                   ga_order ord);
GPUARRAY_PUBLIC int GpuArray_fromdata(GpuArray *a, gpudata *data,
                                      size_t offset, int typecode,
                                      unsigned int nd, const size_t *dims,
                                      const ssize_t *strides, int writeable);
GPUARRAY_PUBLIC int GpuArray_view(GpuArray *v, const GpuArray *a);
GPUARRAY_PUBLIC int GpuArray_sync(GpuArray *a);

/* Basic slicing (ref array.h:298-346): per dim start/stop/step; step 0
 * selects index `start` and drops the dim; a full reversal is
 * start = len-1, stop = -1, step = -1. */
GPUARRAY_PUBLIC int GpuArray_index(GpuArray *r, const GpuArray *a,
                                   const ssize_t *starts, const ssize_t *stops,
                                   const ssize_t *steps);
GPUARRAY_PUBLIC int GpuArray_index_inplace(GpuArray *a, const ssize_t *starts,
                                           const ssize_t *stops,
                                           const ssize_t *steps);

/* a[i[k], ...] = v gather along the first axis (ref array.h:348-366). */
GPUARRAY_PUBLIC int GpuArray_take1(GpuArray *a, const GpuArray *v,
                                   const GpuArray *i, int check_error);
/* a[...] = v with broadcasting of v (ref array.h:368-378). */
GPUARRAY_PUBLIC int GpuArray_setarray(GpuArray *a, const GpuArray *v);

/* Shape changes (ref array.h:380-458).  reshape copies only when the
 * strides cannot express the new shape and nocopy == 0; otherwise
 * GA_COPY_ERROR.  transpose: new_axes == NULL reverses the axes. */
GPUARRAY_PUBLIC int GpuArray_reshape(GpuArray *res, const GpuArray *a,
                                     unsigned int nd, const size_t *newdims,
                                     ga_order ord, int nocopy);
GPUARRAY_PUBLIC int GpuArray_reshape_inplace(GpuArray *a, unsigned int nd,
                                             const size_t *newdims,
                                             ga_order ord);
GPUARRAY_PUBLIC int GpuArray_transpose(GpuArray *res, const GpuArray *a,
                                       const unsigned int *new_axes);
GPUARRAY_PUBLIC int GpuArray_transpose_inplace(GpuArray *a,
                                               const unsigned int *new_axes);

/* Release the buffer reference and the dims/strides, zero the struct. */
GPUARRAY_PUBLIC void GpuArray_clear(GpuArray *a);
GPUARRAY_PUBLIC int GpuArray_share(const GpuArray *a, const GpuArray *b);
GPUARRAY_PUBLIC gpucontext *GpuArray_context(const GpuArray *a);

/* Data movement (ref array.h:488-572).  move copies src into dst (same
 * shape), converting types and handling any strides; read/write/memset need
 * a one-segment array. */
GPUARRAY_PUBLIC int GpuArray_move(GpuArray *dst, const GpuArray *src);
GPUARRAY_PUBLIC int GpuArray_write(GpuArray *dst, const void *src,
                                   size_t src_sz);
GPUARRAY_PUBLIC int GpuArray_read(void *dst, size_t dst_sz,
                                  const GpuArray *src);
GPUARRAY_PUBLIC int GpuArray_memset(GpuArray *a, int data);
GPUARRAY_PUBLIC int GpuArray_copy(GpuArray *res, const GpuArray *a,
                                  ga_order order);
GPUARRAY_PUBLIC int GpuArray_transfer(GpuArray *res, const GpuArray *a);
GPUARRAY_PUBLIC int GpuArray_split(GpuArray **rs, const GpuArray *a, size_t n,
                                   size_t *p, unsigned int axis);
GPUARRAY_PUBLIC int GpuArray_concatenate(GpuArray *r, const GpuArray **as,
                                         size_t n, unsigned int axis,
                                         int restype);

GPUARRAY_PUBLIC const char *GpuArray_error(const GpuArray *a, int err);
GPUARRAY_PUBLIC void GpuArray_fprintf(FILE *fd, const GpuArray *a);
GPUARRAY_PUBLIC int GpuArray_fdump(FILE *fd, const GpuArray *a);

/* Maximum and flattened index of the maximum over the axes in reduxList
 * (ref array.h:607-644, impl src/gpuarray_reduction.c:100-847).
 * dstMax has the source's element type, dstArgmax a 64-bit integer type;
 * both have the source's shape minus the reduced axes and are addressed
 * through their own strides.  The index of a coordinate (i_r0, i_r1, ...)
 * of the reduced axes r = reduxList, in the caller's order, is
 *     sum_k i_rk * prod_{j>k} src.shape[r_j].
 * Comparison is a strict '>' scan in that order: ties keep the lowest
 * index, and a NaN only survives when it is the first element scanned. */
GPUARRAY_PUBLIC int GpuArray_maxandargmax(GpuArray *dstMax,
                                          GpuArray *dstArgmax,
                                          const GpuArray *src,
                                          unsigned reduxLen,
                                          const unsigned *reduxList);

#ifdef __cplusplus
}
#endif
#endif
