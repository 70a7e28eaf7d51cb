// Internal declarations shared by the host translation units.
//
// The layering is the reference's (src/private.h:43-121): generic code only
// touches a context through the leading members of `_gpucontext`, a buffer
// through `{devptr, ctx}` and a kernel through `{ctx}`, and reaches the
// device through a 21-entry function table.  There is exactly one table
// here, the HIP one.
#pragma once

#include <cerrno>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include <gpuarray/array.h>
#include <gpuarray/buffer.h>
#include <gpuarray/elemwise.h>
#include <gpuarray/error.h>
#include <gpuarray/extension.h>
#include <gpuarray/kernel.h>
#include <gpuarray/reduction.h>
#include <gpuarray/types.h>
#include <gpuarray/util.h>

#include "ga_tuning.hpp"
// A knob of the context's tuning table `t`, `dflt` when it is not set.
#define TUNE(t, NAME, dflt) ((t)->get(KNOB_##NAME, (unsigned long)(dflt)))

// ---- error record (reference src/util/error.h:10-22) ----------------------
#define GA_ERROR_MSGBUF_LEN 1020
struct ga_errrec {
  char msg[GA_ERROR_MSGBUF_LEN];
  int code;
};
extern ga_errrec *ga_global_err;
int ga_err_set(ga_errrec *e, int code, const char *msg);
int ga_err_fmt(ga_errrec *e, int code, const char *fmt, ...)
    __attribute__((format(printf, 3, 4)));
static inline int ga_err_sys(ga_errrec *e, const char *what) {
  return ga_err_fmt(e, GA_SYS_ERROR, "%s: %s", what, strerror(errno));
}

// 32-bit addressing limits (reference src/private.h:30-32).
#define GA_ADDR32_MAX 4294967295LL
#define GA_SADDR32_MIN (-2147483648LL)
#define GA_SADDR32_MAX 2147483647LL

// context flag bits (reference src/private.h:56-58)
#define GA_CTX_SINGLE_STREAM 0x01
#define GA_CTX_MULTI_THREAD 0x02

struct _gpucontext_props {  // reference src/private.h:60-67
  int dev;
  int sched;
  int flags;
  const char *kernel_cache_path;
  size_t max_cache_size;
  size_t initial_cache_size;
};

struct ga_buffer_ops;

// Leading members every context exposes to generic code
// (reference GPUCONTEXT_HEAD, src/private.h:43-54).
struct _gpucontext {
  const ga_buffer_ops *ops;
  const void *blas_ops;   // always NULL: dense contraction is not on this path
  const void *comm_ops;   // always NULL: one GPU
  void *blas_handle;
  ga_errrec *err;
  unsigned int refcnt;
  int flags;
  gpudata *errbuf;
  void *extcopy_cache;    // typecode-pair -> GpuElemwise* for strided/casting copies
  char bin_id[64];
  char tag[8];
};

struct _gpudata {         // prefix {devptr, ctx}: reference src/private.h:77-80
  void *devptr;
  gpucontext *ctx;
};

struct _gpukernel {       // prefix {ctx}: reference src/private.h:82-84
  gpucontext *ctx;
};

// The backend table (reference struct _gpuarray_buffer_ops,
// src/private.h:90-121; same members in the same order).
struct ga_buffer_ops {
  int (*get_platform_count)(unsigned int *platcount);
  int (*get_device_count)(unsigned int platform, unsigned int *devcount);
  gpucontext *(*buffer_init)(gpucontext_props *props);
  void (*buffer_deinit)(gpucontext *ctx);
  gpudata *(*buffer_alloc)(gpucontext *ctx, size_t sz, void *data, int flags);
  void (*buffer_retain)(gpudata *b);
  void (*buffer_release)(gpudata *b);
  int (*buffer_share)(gpudata *a, gpudata *b);
  int (*buffer_move)(gpudata *dst, size_t dstoff, gpudata *src, size_t srcoff,
                     size_t sz);
  int (*buffer_read)(void *dst, gpudata *src, size_t srcoff, size_t sz);
  int (*buffer_write)(gpudata *dst, size_t dstoff, const void *src, size_t sz);
  int (*buffer_memset)(gpudata *dst, size_t dstoff, int data);
  int (*kernel_alloc)(gpukernel **k, gpucontext *ctx, unsigned int count,
                      const char **strings, const size_t *lengths,
                      const char *fname, unsigned int numargs,
                      const int *typecodes, int flags, char **err_str);
  void (*kernel_retain)(gpukernel *k);
  void (*kernel_release)(gpukernel *k);
  int (*kernel_setarg)(gpukernel *k, unsigned int i, void *a);
  int (*kernel_call)(gpukernel *k, unsigned int n, const size_t *gs,
                     const size_t *ls, size_t shared, void **args);
  int (*buffer_sync)(gpudata *b);
  int (*buffer_transfer)(gpudata *dst, size_t dstoff, gpudata *src,
                         size_t srcoff, size_t sz);
  int (*property)(gpucontext *ctx, gpudata *buf, gpukernel *k, int prop_id,
                  void *res);
  const char *(*ctx_error)(gpucontext *ctx);
};

extern const ga_buffer_ops ga_hip_ops;
const ga_buffer_ops *gpuarray_get_ops(const char *name);

// array.cpp helpers used by other units (reference src/private.h:283-285)
extern "C" {
int GpuArray_is_c_contiguous(const GpuArray *a);
int GpuArray_is_f_contiguous(const GpuArray *a);
int GpuArray_is_aligned(const GpuArray *a);
}

// ---- HIP backend hooks used by the generators ------------------------------
// Device prelude and reduction templates, embedded at build time.
extern const char ga_device_rt_src[];
extern const char ga_cluda_hip_src[];
extern const char ga_reduce_kernels_src[];

// Grow-only scratch buffer owned by the context (partials of two-pass
// reductions).  Work on a context is in stream order, so one buffer is
// shared by consecutive calls.
gpudata *ga_hip_scratch(gpucontext *ctx, size_t bytes);
// Counters of split reductions that finish in one launch: a buffer of
// ga_hip_redux_counters_max 32-bit zeros, made on first use; every kernel
// that counts on it leaves it zeroed.  NULL (error set) when it cannot be made.
constexpr size_t ga_hip_redux_counters_max = 16384;
gpudata *ga_hip_redux_counters(gpucontext *ctx);
// Have they been made already?  (For callers that may not allocate.)
bool ga_hip_redux_counters_made(gpucontext *ctx);
bool ga_hip_capturing(gpucontext *ctx);
// The scratch of GpuReduction_call_noalloc: a file-scope device array of
// ga_static_scratch_bytes bytes in ga_static_scratch.hip, one copy per GPU.
// ga_static_scratch_setup, called with device `dev` current, looks its
// address on that device up once and returns it in *ptr (0 on success, else
// the HIP error code; *ptr is then NULL).
constexpr size_t ga_static_scratch_bytes = GA_REDUCTION_NOALLOC_SCRATCH;
int ga_static_scratch_setup(int dev, void **ptr);
// The address found for the context's device when the context was made, NULL
// when the lookup failed (the reason is then in *why, if not NULL).
void *ga_hip_static_scratch(gpucontext *ctx, const char **why);
// The same array as a buffer of the context (made with the context; releasing
// it never frees anything), NULL when the lookup failed.
gpudata *ga_hip_static_scratch_buf(gpucontext *ctx, const char **why);
// Bytes from a buffer's start that lie inside the memory behind it (at least
// its size; more when the allocation was rounded up).
size_t ga_hip_readable_bytes(gpudata *b);
// Device address, size and readable bytes (as above) of a buffer, in one call.
void ga_hip_buf_info(gpudata *b, uintptr_t *devptr, size_t *size, size_t *readable);
// Number of compute units of the context's device.
unsigned int ga_hip_numprocs(gpucontext *ctx);
// Frees the strided-copy operator cache of a context (array.cpp).
void ga_extcopy_cache_free(gpucontext *ctx);
// Frees the per-context cache behind GpuArray_maxandargmax (reduction.cpp).
void ga_redux_cache_free(gpucontext *ctx);
void **ga_hip_redux_cache_slot(gpucontext *ctx);
// Frees the per-context kernels of GpuArray_take1 (array.cpp).
void ga_take1_cache_free(gpucontext *ctx);
void **ga_hip_take1_cache_slot(gpucontext *ctx);

// Typecode of the opaque by-value "plan" kernel argument of `bytes` bytes
// (registered on first use through gpuarray_register_type).
int ga_plan_typecode(size_t bytes);
