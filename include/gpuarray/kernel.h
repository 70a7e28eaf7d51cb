/* GpuKernel: a compiled kernel plus its argument table.
 * Same layout and entry points as the reference's src/gpuarray/kernel.h:20-112
 * (impl src/gpuarray_kernel.c:10-103). */
#ifndef GPUARRAY_KERNEL_H
#define GPUARRAY_KERNEL_H

#include <gpuarray/array.h>
#include <gpuarray/buffer.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct _GpuKernel {
  gpukernel *k;   /* backend kernel */
  void **args;    /* argcount slots, owned by the struct */
} GpuKernel;

/* Compile `count` source strings and bind entry point `name`
 * (ref kernel.h:31-58).  On failure k is cleared. */
GPUARRAY_PUBLIC int GpuKernel_init(GpuKernel *k, gpucontext *ctx,
                                   unsigned int count, const char **strs,
                                   const size_t *lens, const char *name,
                                   unsigned int argcount, const int *types,
                                   int flags, char **err_str);
GPUARRAY_PUBLIC void GpuKernel_clear(GpuKernel *k);
GPUARRAY_PUBLIC gpucontext *GpuKernel_context(GpuKernel *k);
GPUARRAY_PUBLIC int GpuKernel_setarg(GpuKernel *k, unsigned int i, void *val);

/* Pick a 1-D launch for n work items (ref kernel.h:78-96,
 * src/gpuarray_kernel.c:38-89).  *gs and *ls are in/out: a non-zero value on
 * entry is kept.  The geometry targets 256 compute units: groups are a
 * multiple of the 64-lane wavefront, 256 lanes by default, and the grid is
 * capped at a fixed number of groups per compute unit so that kernels
 * written as grid-stride loops keep every unit busy. */
GPUARRAY_PUBLIC int GpuKernel_sched(GpuKernel *k, size_t n, size_t *gs,
                                    size_t *ls);

/* Launch on n (1..3) dimensions; gs counts groups, ls lanes per group
 * (ref kernel.h:98-110).  args == NULL uses the values given to setarg. */
GPUARRAY_PUBLIC int GpuKernel_call(GpuKernel *k, unsigned int n,
                                   const size_t *gs, const size_t *ls,
                                   size_t shared, void **args);
GPUARRAY_PUBLIC const char *GpuKernel_error(const GpuKernel *k, int err);

#ifdef __cplusplus
}
#endif
#endif
