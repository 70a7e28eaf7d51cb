/* Contexts, device buffers and kernels: the backend-neutral layer.
 *
 * Every declaration keeps the name, signature and constant values of the
 * reference's src/gpuarray/buffer.h (cited per item) so existing callers
 * relink unchanged.  The only backend behind it is "hip" (one MI355X, one
 * in-order stream); gpucontext_props_hip_dev is the one addition.
 *
 * Conventions (reference src/gpuarray_buffer.c:21-37,104-141):
 *   - int results are GA_NO_ERROR or an enum ga_error value; the text is
 *     read back with gpucontext_error(ctx, err) (ctx == NULL: process-global
 *     message, used before a context exists).
 *   - pointer results are NULL on failure with the code in *ret when given.
 *   - contexts, buffers and kernels are reference counted.
 */
#ifndef GPUARRAY_BUFFER_H
#define GPUARRAY_BUFFER_H

#include <stdarg.h>
#include <stdio.h>
#include <sys/types.h>

#include <gpuarray/config.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct _gpudata gpudata;         /* ref src/gpuarray/buffer.h:28-33 */
typedef struct _gpucontext gpucontext;   /* ref :35-41 */
typedef struct _gpukernel gpukernel;     /* ref :43-49 */
typedef struct _gpucontext_props gpucontext_props; /* ref :78 */

/* Device enumeration (ref :56-76).  name must be "hip"; there is one
 * platform, and as many devices as hipGetDeviceCount reports. */
GPUARRAY_PUBLIC int gpu_get_platform_count(const char *name,
                                           unsigned int *platcount);
GPUARRAY_PUBLIC int gpu_get_device_count(const char *name,
                                         unsigned int platform,
                                         unsigned int *devcount);

/* Context properties (ref :80-190; impl src/gpuarray_buffer.c:40-102). */
GPUARRAY_PUBLIC int gpucontext_props_new(gpucontext_props **res);
/* Select the HIP device ordinal; -1 (default) picks device 0.  New. */
GPUARRAY_PUBLIC int gpucontext_props_hip_dev(gpucontext_props *p, int devno);
/* Kept for source compatibility: both record the device ordinal exactly as
 * the reference does (cuda: devno; opencl: platno<<16|devno), and the "hip"
 * backend reads the low 16 bits. */
GPUARRAY_PUBLIC int gpucontext_props_cuda_dev(gpucontext_props *p, int devno);
GPUARRAY_PUBLIC int gpucontext_props_opencl_dev(gpucontext_props *p,
                                                int platno, int devno);
GPUARRAY_PUBLIC int gpucontext_props_sched(gpucontext_props *p, int sched);
#define GA_CTX_SCHED_AUTO   0
#define GA_CTX_SCHED_SINGLE 1
#define GA_CTX_SCHED_MULTI  2
GPUARRAY_PUBLIC int gpucontext_props_set_single_stream(gpucontext_props *p);
GPUARRAY_PUBLIC int gpucontext_props_kernel_cache(gpucontext_props *p,
                                                  const char *path);
GPUARRAY_PUBLIC int gpucontext_props_alloc_cache(gpucontext_props *p,
                                                 size_t initial, size_t max);
GPUARRAY_PUBLIC void gpucontext_props_del(gpucontext_props *p);

/* Context lifecycle (ref :192-265).  gpucontext_init consumes props (NULL
 * means defaults) whether it succeeds or not. */
GPUARRAY_PUBLIC int gpucontext_init(gpucontext **res, const char *name,
                                    gpucontext_props *props);
GPUARRAY_PUBLIC void gpucontext_deref(gpucontext *ctx);
GPUARRAY_PUBLIC int gpucontext_property(gpucontext *ctx, int prop_id,
                                        void *res);
GPUARRAY_PUBLIC const char *gpucontext_error(gpucontext *ctx, int err);

/* Buffers (ref :267-476; impl src/gpuarray_buffer.c:143-224).
 * alloc(sz == 0) is legal.  GA_BUFFER_INIT copies sz bytes from data.
 * memset fills from dstoff to the END of the buffer with the low byte of
 * data.  read/write block until the host memory is safe to reuse; all other
 * work is queued on the context's stream. */
GPUARRAY_PUBLIC gpudata *gpudata_alloc(gpucontext *ctx, size_t sz, void *data,
                                       int flags, int *ret);
#define GA_BUFFER_READ_WRITE 0x00
#define GA_BUFFER_DEV        0x00
#define GA_BUFFER_READ_ONLY  0x01
#define GA_BUFFER_WRITE_ONLY 0x02
#define GA_BUFFER_INIT       0x04
#define GA_BUFFER_HOST       0x08
#define GA_BUFFER_MASK       0xffff

GPUARRAY_PUBLIC void gpudata_retain(gpudata *b);
GPUARRAY_PUBLIC void gpudata_release(gpudata *b);
/* 1 if the byte ranges of a and b may overlap, 0 if not, -1 on error. */
GPUARRAY_PUBLIC int gpudata_share(gpudata *a, gpudata *b, int *ret);
GPUARRAY_PUBLIC int gpudata_move(gpudata *dst, size_t dstoff, gpudata *src,
                                 size_t srcoff, size_t sz);
GPUARRAY_PUBLIC int gpudata_transfer(gpudata *dst, size_t dstoff, gpudata *src,
                                     size_t srcoff, size_t sz);
GPUARRAY_PUBLIC int gpudata_read(void *dst, gpudata *src, size_t srcoff,
                                 size_t sz);
GPUARRAY_PUBLIC int gpudata_write(gpudata *dst, size_t dstoff, const void *src,
                                  size_t sz);
GPUARRAY_PUBLIC int gpudata_memset(gpudata *dst, size_t dstoff, int data);
GPUARRAY_PUBLIC int gpudata_sync(gpudata *b);
GPUARRAY_PUBLIC int gpudata_property(gpudata *buf, int prop_id, void *res);
GPUARRAY_PUBLIC gpucontext *gpudata_context(gpudata *b);

/* Kernels (ref :478-599; impl src/gpuarray_buffer.c:226-269).
 * The `count` strings are concatenated and compiled for gfx950 at run time;
 * `#include "cluda.h"` resolves to the built-in device prelude.  typecodes
 * describe the arguments: GA_BUFFER takes a gpudata*, GA_SIZE/GA_SSIZE a
 * pointer to size_t/ssize_t, anything else a pointer to a host value of that
 * type.  *err_str (when not NULL) receives a malloc'd compiler log that the
 * caller frees.  gs is the NUMBER OF GROUPS per dimension, ls the group size
 * (ref :553-570). */
GPUARRAY_PUBLIC gpukernel *gpukernel_init(gpucontext *ctx, unsigned int count,
                                          const char **strings,
                                          const size_t *lengths,
                                          const char *fname,
                                          unsigned int numargs,
                                          const int *typecodes, int flags,
                                          int *ret, char **err_str);
GPUARRAY_PUBLIC void gpukernel_retain(gpukernel *k);
GPUARRAY_PUBLIC void gpukernel_release(gpukernel *k);
GPUARRAY_PUBLIC int gpukernel_setarg(gpukernel *k, unsigned int i, void *a);
GPUARRAY_PUBLIC int gpukernel_call(gpukernel *k, unsigned int n,
                                   const size_t *gs, const size_t *ls,
                                   size_t shared, void **args);
GPUARRAY_PUBLIC int gpukernel_property(gpukernel *k, int prop_id, void *res);
GPUARRAY_PUBLIC gpucontext *gpukernel_context(gpukernel *k);

/* Property ids and result types (ref :600-807). */
#define GA_CTX_PROP_DEVNAME            1   /* char[256] */
#define GA_CTX_PROP_LMEMSIZE           3   /* size_t: LDS bytes per group */
#define GA_CTX_PROP_NUMPROCS           4   /* unsigned int: compute units */
#define GA_CTX_PROP_BIN_ID             7   /* const char *: "gfx950" */
#define GA_CTX_PROP_ERRBUF             8   /* gpudata *: 8 zeroed bytes */
#define GA_CTX_PROP_TOTAL_GMEM         9   /* size_t */
#define GA_CTX_PROP_FREE_GMEM          10  /* size_t */
#define GA_CTX_PROP_NATIVE_FLOAT16     11  /* int */
#define GA_CTX_PROP_MAXGSIZE0          12  /* size_t */
#define GA_CTX_PROP_MAXGSIZE1          13  /* size_t */
#define GA_CTX_PROP_MAXGSIZE2          14  /* size_t */
#define GA_CTX_PROP_MAXLSIZE0          15  /* size_t */
#define GA_CTX_PROP_MAXLSIZE1          16  /* size_t */
#define GA_CTX_PROP_MAXLSIZE2          17  /* size_t */
#define GA_CTX_PROP_UNIQUE_ID          19  /* char[16]: PCI bus id */
#define GA_CTX_PROP_LARGEST_MEMBLOCK   20  /* size_t */

#define GA_BUFFER_PROP_START           512
#define GA_BUFFER_PROP_CTX             512 /* gpucontext * */
#define GA_BUFFER_PROP_REFCNT          513 /* unsigned int */
#define GA_BUFFER_PROP_SIZE            514 /* size_t */

#define GA_KERNEL_PROP_START           1024
#define GA_KERNEL_PROP_CTX             1024 /* gpucontext * */
#define GA_KERNEL_PROP_MAXLSIZE        1025 /* size_t */
#define GA_KERNEL_PROP_PREFLSIZE       1026 /* size_t: 64, one wavefront */
#define GA_KERNEL_PROP_NUMARGS         1027 /* unsigned int */
#define GA_KERNEL_PROP_TYPES           1028 /* const int * */

/* Feature flags for gpukernel_init (ref :809-852).  GA_USE_CUDA and
 * GA_USE_OPENCL mark source written in another device language; the "hip"
 * backend refuses both with GA_DEVSUP_ERROR. */
typedef enum _ga_usefl {
  GA_USE_SMALL   = 0x02,
  GA_USE_DOUBLE  = 0x04,
  GA_USE_COMPLEX = 0x08,
  GA_USE_HALF    = 0x10,
  GA_USE_CUDA    = 0x2000,
  GA_USE_OPENCL  = 0x4000,
  GA_USE_HIP     = 0x8000
} ga_usefl;

#ifdef __cplusplus
}
#endif
#endif
