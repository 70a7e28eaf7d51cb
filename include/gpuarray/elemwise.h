/* GpuElemwise: one C-like expression applied over broadcastable strided
 * arrays.  Drop-in for the reference's src/gpuarray/elemwise.h:28-162
 * (impl src/gpuarray_elemwise.c:604-787): same descriptor, flags and calls.
 */
#ifndef GPUARRAY_ELEMWISE_H
#define GPUARRAY_ELEMWISE_H

#include <gpuarray/buffer.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct _GpuElemwise GpuElemwise;

/* One argument of the expression (ref elemwise.h:28-68).  `name` is the
 * identifier used inside `expr`; scalars are passed by value, arrays are
 * read into / written from a local of that name. */
typedef struct _gpuelemwise_arg {
  const char *name;
  int typecode;
  int flags;
#define GE_SCALAR 0x0001
#define GE_READ   0x0002
#define GE_WRITE  0x0004
} gpuelemwise_arg;

/* Build the operation (ref elemwise.h:70-104).  `preamble` (may be NULL) is
 * pasted before the kernel, `expr` is one or more C statements without the
 * final semicolon.  `nd` only pre-builds strided kernels up to that rank;
 * any rank works later.  Returns NULL with the message in the context. */
GPUARRAY_PUBLIC GpuElemwise *GpuElemwise_new(gpucontext *ctx,
                                             const char *preamble,
                                             const char *expr, unsigned int n,
                                             gpuelemwise_arg *args,
                                             unsigned int nd, int flags);
#define GE_NOADDR64    0x0001  /* do not pre-build 64-bit index kernels */
#define GE_CONVERT_F16 0x0002  /* half arrays are seen as float in expr */

GPUARRAY_PUBLIC void GpuElemwise_free(GpuElemwise *ge);

/* Run it (ref elemwise.h:114-140).  args[i] is a GpuArray* for arrays and a
 * pointer to a host value of the declared type for scalars.  The first
 * GE_WRITE array fixes the iteration space; outputs never broadcast. */
GPUARRAY_PUBLIC int GpuElemwise_call(GpuElemwise *ge, void **args, int flags);
#define GE_BROADCAST  0x0100  /* size-1 input dims stretch */
#define GE_NOCOLLAPSE 0x0200  /* keep the dims as given */
#define GE_PADSHAPE   0x0400  /* left-pad lower-rank arrays with 1s */

#ifdef __cplusplus
}
#endif
#endif
