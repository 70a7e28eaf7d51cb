// The HIP backend: one device, one in-order stream, kernels compiled at run
// time for gfx950 with hipRTC and launched with hipModuleLaunchKernel.
//
// It fills the same 21-entry table the reference's backends fill
// (src/private.h:90-121).  The shape is that of the reference's CUDA backend
// (src/gpuarray_buffer_cuda.c: runtime compile -> module -> launch with an
// array of argument pointers, where a buffer argument is passed as the address
// of the gpudata itself because the device pointer is its first member,
// :1494-1525) but none of its machinery is needed: a single in-order stream
// orders all work, so there are no per-buffer events.
#include "private.hpp"

#include <hip/hip_runtime_api.h>
#include <hip/hiprtc.h>

#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

namespace {

struct hip_module {
  hipModule_t mod = nullptr;
  unsigned refcnt = 0;
  std::string key;
};

struct hip_context : _gpucontext {
  int dev = 0;
  hipStream_t stream = nullptr;
  unsigned int numprocs = 0;
  size_t lmemsize = 0;
  size_t maxg[3] = {0, 0, 0};
  size_t maxl[3] = {0, 0, 0};
  size_t maxthreads = 0;
  char devname[256] = {0};
  char pciid[16] = {0};
  std::unordered_map<std::string, hip_module *> modcache;
  gpudata *scratch = nullptr;
  size_t scratch_sz = 0;
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  std::vector<hipEvent_t> evpool;   // timing marks for callers (hip_event_* hooks)
  void *redux_cache = nullptr;
  ga_errrec errstore;
};

#define BUF_OWNED 0x10000      /* devptr came from hipMalloc */
#define BUF_INTERNAL 0x20000   /* does not keep the context alive */

struct hip_data : _gpudata {
  size_t sz;
  unsigned int refcnt;
  int flags;
};

struct hip_kernel : _gpukernel {
  hipFunction_t fn;
  hip_module *mod;
  unsigned int refcnt;
  unsigned int argcount;
  int *types;
  size_t *argoff;        // byte offset of each by-value argument in argstore
  unsigned char *argstore;
  void **args;           // what setarg recorded: gpudata* or pointer into argstore
  size_t maxlsize;
};

inline hip_context *HC(gpucontext *c) { return static_cast<hip_context *>(c); }
inline hip_data *HD(gpudata *b) { return static_cast<hip_data *>(b); }
inline hip_kernel *HK(gpukernel *k) { return static_cast<hip_kernel *>(k); }

int hip_fail(ga_errrec *e, const char *what, hipError_t err) {
  return ga_err_fmt(e, GA_IMPL_ERROR, "%s: %s (%d)", what, hipGetErrorString(err),
                    (int)err);
}

#define HIP_TRY(ctx, call)                                       \
  do {                                                           \
    hipError_t _e = (call);                                      \
    if (_e != hipSuccess) return hip_fail((ctx)->err, #call, _e); \
  } while (0)

int enter(hip_context *ctx) {
  int cur = -1;
  if (hipGetDevice(&cur) == hipSuccess && cur == ctx->dev) return GA_NO_ERROR;
  HIP_TRY(ctx, hipSetDevice(ctx->dev));
  return GA_NO_ERROR;
}

// ---- enumeration ------------------------------------------------------------

int hip_get_platform_count(unsigned int *platcount) {
  *platcount = 1;
  return GA_NO_ERROR;
}

int hip_get_device_count(unsigned int platform, unsigned int *devcount) {
  if (platform != 0)
    return ga_err_set(ga_global_err, GA_VALUE_ERROR, "hip has a single platform (0)");
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess) {
    *devcount = 0;
    if (e == hipErrorNoDevice) return GA_NO_ERROR;
    return hip_fail(ga_global_err, "hipGetDeviceCount", e);
  }
  *devcount = (unsigned int)n;
  return GA_NO_ERROR;
}

// ---- context ------------------------------------------------------------------

void hip_release(gpudata *b);

void ctx_destroy(hip_context *ctx) {
  (void)hipSetDevice(ctx->dev);
  // internal buffers do not count as owners, so they are still here
  if (ctx->errbuf) { hip_release(ctx->errbuf); ctx->errbuf = nullptr; }
  if (ctx->scratch) { hip_release(ctx->scratch); ctx->scratch = nullptr; }
  for (auto &kv : ctx->modcache) {
    if (kv.second->mod) (void)hipModuleUnload(kv.second->mod);
    delete kv.second;
  }
  ctx->modcache.clear();
  for (hipEvent_t e : ctx->evpool) (void)hipEventDestroy(e);
  if (ctx->ev0) (void)hipEventDestroy(ctx->ev0);
  if (ctx->ev1) (void)hipEventDestroy(ctx->ev1);
  if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
  delete ctx;
}

void ctx_unref(hip_context *ctx) {
  if (--ctx->refcnt == 0) ctx_destroy(ctx);
}

gpudata *hip_alloc(gpucontext *c, size_t sz, void *data, int flags);

gpucontext *hip_init(gpucontext_props *p) {
  int ndev = 0;
  hipError_t e = hipGetDeviceCount(&ndev);
  if (e != hipSuccess || ndev == 0) {
    ga_err_fmt(ga_global_err, GA_NODEV_ERROR, "No HIP device available (%s)",
               e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
    return nullptr;
  }
  int dev = p->dev < 0 ? 0 : (p->dev & 0xffff);
  if (dev >= ndev) {
    ga_err_fmt(ga_global_err, GA_VALUE_ERROR,
               "Device %d requested but only %d present", dev, ndev);
    return nullptr;
  }
  hip_context *ctx = new (std::nothrow) hip_context();
  if (ctx == nullptr) {
    ga_err_set(ga_global_err, GA_MEMORY_ERROR, "Out of memory");
    return nullptr;
  }
  ctx->ops = &ga_hip_ops;
  ctx->blas_ops = nullptr;
  ctx->comm_ops = nullptr;
  ctx->blas_handle = nullptr;
  ctx->err = &ctx->errstore;
  ctx->errstore.code = 0;
  ctx->errstore.msg[0] = 0;
  ctx->refcnt = 1;
  ctx->flags = p->flags | GA_CTX_SINGLE_STREAM;
  ctx->errbuf = nullptr;
  ctx->extcopy_cache = nullptr;
  memset(ctx->bin_id, 0, sizeof(ctx->bin_id));
  memcpy(ctx->tag, "hipctx ", 8);
  ctx->dev = dev;

#define INIT_TRY(call)                                   \
  do {                                                   \
    hipError_t _e = (call);                              \
    if (_e != hipSuccess) {                              \
      hip_fail(ga_global_err, #call, _e);                \
      ctx_destroy(ctx);                                  \
      return nullptr;                                    \
    }                                                    \
  } while (0)

  INIT_TRY(hipSetDevice(dev));
  // Default priority on purpose: work on streams of different priorities is
  // never mixed.
  INIT_TRY(hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking));
  INIT_TRY(hipEventCreate(&ctx->ev0));
  INIT_TRY(hipEventCreate(&ctx->ev1));

  hipDeviceProp_t prop;
  INIT_TRY(hipGetDeviceProperties(&prop, dev));
  ctx->numprocs = (unsigned int)prop.multiProcessorCount;
  ctx->lmemsize = prop.sharedMemPerBlock;
  for (int i = 0; i < 3; i++) {
    ctx->maxg[i] = (size_t)prop.maxGridSize[i];
    ctx->maxl[i] = (size_t)prop.maxThreadsDim[i];
  }
  ctx->maxthreads = (size_t)prop.maxThreadsPerBlock;
  // some driver stacks leave the marketing name empty; the ISA name is always there
  snprintf(ctx->devname, sizeof(ctx->devname), "%s", prop.name[0] ? prop.name : prop.gcnArchName);
  snprintf(ctx->pciid, sizeof(ctx->pciid), "%04x:%02x:%02x.0", prop.pciDomainID,
           prop.pciBusID, prop.pciDeviceID);
  // Binaries are interchangeable between devices of the same ISA.
  const char *arch = prop.gcnArchName;
  size_t alen = strcspn(arch, ":");
  snprintf(ctx->bin_id, sizeof(ctx->bin_id), "%.*s", (int)alen, arch);
#undef INIT_TRY

  // 8 zeroed bytes kernels can use to report a fault
  // (reference GA_CTX_PROP_ERRBUF, src/gpuarray/buffer.h:646-658).
  uint64_t zero = 0;
  ctx->errbuf = hip_alloc(ctx, 8, &zero, GA_BUFFER_INIT | BUF_INTERNAL);
  if (ctx->errbuf == nullptr) {
    ga_err_set(ga_global_err, ctx->err->code, ctx->err->msg);
    ctx_destroy(ctx);
    return nullptr;
  }
  return ctx;
}

void hip_deinit(gpucontext *c) {
  hip_context *ctx = HC(c);
  // Cached operators hold kernels, which hold the context: drop them first.
  ga_extcopy_cache_free(c);
  ga_redux_cache_free(c);
  ctx_unref(ctx);
}

// ---- buffers ------------------------------------------------------------------

gpudata *hip_alloc(gpucontext *c, size_t sz, void *data, int flags) {
  hip_context *ctx = HC(c);
  if ((flags & GA_BUFFER_INIT) && data == nullptr) {
    ga_err_set(ctx->err, GA_VALUE_ERROR, "Requested buffer initialisation but no data given");
    return nullptr;
  }
  if ((flags & (GA_BUFFER_READ_ONLY | GA_BUFFER_WRITE_ONLY)) ==
      (GA_BUFFER_READ_ONLY | GA_BUFFER_WRITE_ONLY)) {
    ga_err_set(ctx->err, GA_VALUE_ERROR, "Invalid flags combination: READ_ONLY and WRITE_ONLY");
    return nullptr;
  }
  if (flags & GA_BUFFER_HOST) {
    ga_err_set(ctx->err, GA_DEVSUP_ERROR, "Host-mapped buffers are not supported");
    return nullptr;
  }
  if (enter(ctx) != GA_NO_ERROR) return nullptr;
  hip_data *b = (hip_data *)calloc(1, sizeof(hip_data));
  if (b == nullptr) {
    ga_err_sys(ctx->err, "calloc");
    return nullptr;
  }
  size_t asz = sz ? sz : 1;   // a zero-byte request still yields a valid buffer
  hipError_t e = hipMalloc(&b->devptr, asz);
  if (e != hipSuccess) {
    free(b);
    if (e == hipErrorOutOfMemory || e == hipErrorMemoryAllocation)
      ga_err_fmt(ctx->err, GA_MEMORY_ERROR, "hipMalloc(%zu): out of device memory", asz);
    else
      hip_fail(ctx->err, "hipMalloc", e);
    return nullptr;
  }
  b->ctx = ctx;
  b->sz = asz;
  b->refcnt = 1;
  b->flags = (flags & (GA_BUFFER_MASK | BUF_INTERNAL)) | BUF_OWNED;
  if (flags & GA_BUFFER_INIT) {
    e = hipMemcpyHtoDAsync(b->devptr, data, sz, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
      hip_fail(ctx->err, "hipMemcpyHtoDAsync", e);
      (void)hipFree(b->devptr);
      free(b);
      return nullptr;
    }
  }
  if (!(b->flags & BUF_INTERNAL)) ctx->refcnt++;
  return b;
}

void hip_retain(gpudata *b) { HD(b)->refcnt++; }

void hip_release(gpudata *bb) {
  hip_data *b = HD(bb);
  if (--b->refcnt != 0) return;
  hip_context *ctx = HC(b->ctx);
  if (b->flags & BUF_OWNED) {
    (void)hipSetDevice(ctx->dev);
    // hipFree waits for the device, so queued work that still uses the
    // memory completes first.
    (void)hipFree(b->devptr);
  }
  bool counted = !(b->flags & BUF_INTERNAL);
  free(b);
  if (counted) ctx_unref(ctx);
}

// 1 when the two byte ranges overlap in the same context
// (reference src/gpuarray_buffer_cuda.c:891-897).
int hip_share(gpudata *a, gpudata *b) {
  if (a->ctx != b->ctx) return 0;
  const char *pa = (const char *)a->devptr, *pb = (const char *)b->devptr;
  return (pa <= pb && pb < pa + HD(a)->sz) || (pb <= pa && pa < pb + HD(b)->sz);
}

int range_check(hip_context *ctx, hip_data *b, size_t off, size_t sz, const char *what) {
  if (off > b->sz || sz > b->sz - off)
    return ga_err_fmt(ctx->err, GA_VALUE_ERROR,
                      "%s: range [%zu, %zu) is outside the buffer of %zu bytes", what, off,
                      off + sz, b->sz);
  return GA_NO_ERROR;
}

int hip_move(gpudata *dst, size_t dstoff, gpudata *src, size_t srcoff, size_t sz) {
  hip_context *ctx = HC(dst->ctx);
  if (dst->ctx != src->ctx)
    return ga_err_set(ctx->err, GA_VALUE_ERROR, "Cannot move between contexts");
  if (sz == 0) return GA_NO_ERROR;
  int err;
  if ((err = range_check(ctx, HD(dst), dstoff, sz, "move dst")) != GA_NO_ERROR) return err;
  if ((err = range_check(ctx, HD(src), srcoff, sz, "move src")) != GA_NO_ERROR) return err;
  if ((err = enter(ctx)) != GA_NO_ERROR) return err;
  HIP_TRY(ctx, hipMemcpyDtoDAsync((char *)dst->devptr + dstoff,
                                  (char *)src->devptr + srcoff, sz, ctx->stream));
  return GA_NO_ERROR;
}

int hip_read(void *dst, gpudata *src, size_t srcoff, size_t sz) {
  hip_context *ctx = HC(src->ctx);
  if (sz == 0) return GA_NO_ERROR;
  int err;
  if ((err = range_check(ctx, HD(src), srcoff, sz, "read")) != GA_NO_ERROR) return err;
  if ((err = enter(ctx)) != GA_NO_ERROR) return err;
  HIP_TRY(ctx, hipMemcpyDtoHAsync(dst, (char *)src->devptr + srcoff, sz, ctx->stream));
  HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
  return GA_NO_ERROR;
}

int hip_write(gpudata *dst, size_t dstoff, const void *src, size_t sz) {
  hip_context *ctx = HC(dst->ctx);
  if (sz == 0) return GA_NO_ERROR;
  int err;
  if ((err = range_check(ctx, HD(dst), dstoff, sz, "write")) != GA_NO_ERROR) return err;
  if ((err = enter(ctx)) != GA_NO_ERROR) return err;
  HIP_TRY(ctx, hipMemcpyHtoDAsync((char *)dst->devptr + dstoff, const_cast<void *>(src), sz,
                                  ctx->stream));
  // the host memory belongs to the caller again on return
  HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
  return GA_NO_ERROR;
}

// Fill from dstoff to the end of the buffer with the low byte of `data`.
int hip_memset(gpudata *dst, size_t dstoff, int data) {
  hip_context *ctx = HC(dst->ctx);
  hip_data *b = HD(dst);
  if (dstoff > b->sz)
    return ga_err_set(ctx->err, GA_VALUE_ERROR, "memset offset is past the end of the buffer");
  size_t n = b->sz - dstoff;
  if (n == 0) return GA_NO_ERROR;
  int err;
  if ((err = enter(ctx)) != GA_NO_ERROR) return err;
  HIP_TRY(ctx, hipMemsetD8Async((hipDeviceptr_t)((char *)b->devptr + dstoff),
                                (unsigned char)(data & 0xff), n, ctx->stream));
  return GA_NO_ERROR;
}

int hip_sync(gpudata *b) {
  hip_context *ctx = HC(b->ctx);
  int err;
  if ((err = enter(ctx)) != GA_NO_ERROR) return err;
  HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
  return GA_NO_ERROR;
}

int hip_transfer(gpudata *dst, size_t dstoff, gpudata *src, size_t srcoff, size_t sz) {
  hip_context *sc = HC(src->ctx), *dc = HC(dst->ctx);
  if (sz == 0) return GA_NO_ERROR;
  int err;
  if ((err = range_check(dc, HD(dst), dstoff, sz, "transfer dst")) != GA_NO_ERROR) return err;
  if ((err = range_check(sc, HD(src), srcoff, sz, "transfer src")) != GA_NO_ERROR) return err;
  // Order after everything queued on the source, copy on the destination.
  HIP_TRY(sc, hipSetDevice(sc->dev));
  HIP_TRY(sc, hipStreamSynchronize(sc->stream));
  HIP_TRY(dc, hipSetDevice(dc->dev));
  HIP_TRY(dc, hipMemcpyPeerAsync((char *)dst->devptr + dstoff, dc->dev,
                                 (char *)src->devptr + srcoff, sc->dev, sz, dc->stream));
  HIP_TRY(dc, hipStreamSynchronize(dc->stream));
  return GA_NO_ERROR;
}

// ---- kernels ------------------------------------------------------------------

const char *const k_rtc_opts[] = {
    "--offload-arch=gfx950",
    "-O3",
    // a*b+c stays two roundings, as in IEEE host arithmetic
    "-ffp-contract=off",
    // scalar fp32 ops only; no packed fp32 instruction forms
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-value",
};

std::string join_sources(unsigned int count, const char **strs, const size_t *lens) {
  std::string src;
  for (unsigned int i = 0; i < count; i++) {
    size_t l = (lens != nullptr && lens[i] != 0) ? lens[i] : strlen(strs[i]);
    src.append(strs[i], l);
  }
  return src;
}

// Compile to a gfx950 code object.  Needs no device.
int rtc_compile(const std::string &src, std::vector<char> &code, std::string &log) {
  hiprtcProgram prog = nullptr;
  const char *hdr_src[] = {ga_cluda_hip_src};
  const char *hdr_name[] = {"cluda.h"};
  hiprtcResult r = hiprtcCreateProgram(&prog, src.c_str(), "ga_kernel.hip", 1, hdr_src, hdr_name);
  if (r != HIPRTC_SUCCESS) {
    log = std::string("hiprtcCreateProgram: ") + hiprtcGetErrorString(r);
    return GA_IMPL_ERROR;
  }
  r = hiprtcCompileProgram(prog, (int)(sizeof(k_rtc_opts) / sizeof(k_rtc_opts[0])), k_rtc_opts);
  size_t lsz = 0;
  if (hiprtcGetProgramLogSize(prog, &lsz) == HIPRTC_SUCCESS && lsz > 1) {
    log.resize(lsz);
    hiprtcGetProgramLog(prog, &log[0]);
    while (!log.empty() && log.back() == '\0') log.pop_back();
  }
  if (r != HIPRTC_SUCCESS) {
    if (log.empty()) log = hiprtcGetErrorString(r);
    hiprtcDestroyProgram(&prog);
    return GA_IMPL_ERROR;
  }
  size_t csz = 0;
  r = hiprtcGetCodeSize(prog, &csz);
  if (r == HIPRTC_SUCCESS) {
    code.resize(csz);
    r = hiprtcGetCode(prog, code.data());
  }
  hiprtcDestroyProgram(&prog);
  if (r != HIPRTC_SUCCESS) {
    log = std::string("hiprtcGetCode: ") + hiprtcGetErrorString(r);
    return GA_IMPL_ERROR;
  }
  return GA_NO_ERROR;
}

void mod_unref(hip_context *ctx, hip_module *m) {
  // Modules stay cached for the life of the context: recompiling costs
  // hundreds of milliseconds, keeping one costs a few kilobytes.
  (void)ctx;
  if (m->refcnt > 0) m->refcnt--;
}

int hip_newkernel(gpukernel **out, gpucontext *c, unsigned int count, const char **strings,
                  const size_t *lengths, const char *fname, unsigned int numargs,
                  const int *typecodes, int flags, char **err_str) {
  hip_context *ctx = HC(c);
  *out = nullptr;
  if (err_str) *err_str = nullptr;
  if (count == 0 || strings == nullptr || fname == nullptr)
    return ga_err_set(ctx->err, GA_VALUE_ERROR, "No kernel source or no entry point name");
  if (flags & (GA_USE_CUDA | GA_USE_OPENCL))
    return ga_err_set(ctx->err, GA_DEVSUP_ERROR,
                      "Kernel source is marked CUDA/OpenCL; this backend compiles HIP only");
  if (flags & GA_USE_COMPLEX)
    return ga_err_set(ctx->err, GA_UNSUPPORTED_ERROR, "Complex types are not supported");
  for (unsigned int i = 0; i < numargs; i++) {
    if (typecodes[i] != GA_BUFFER && gpuarray_get_elsize(typecodes[i]) == 0)
      return ga_err_fmt(ctx->err, GA_VALUE_ERROR, "Argument %u has unknown typecode %d", i,
                        typecodes[i]);
  }
  int err;
  if ((err = enter(ctx)) != GA_NO_ERROR) return err;

  std::string src = join_sources(count, strings, lengths);
  hip_module *m = nullptr;
  auto it = ctx->modcache.find(src);
  if (it != ctx->modcache.end()) {
    m = it->second;
  } else {
    std::vector<char> code;
    std::string log;
    err = rtc_compile(src, code, log);
    if (err != GA_NO_ERROR) {
      if (err_str) *err_str = strdup(log.c_str());
      return ga_err_fmt(ctx->err, GA_IMPL_ERROR, "Kernel compilation failed: %.900s", log.c_str());
    }
    m = new hip_module();
    hipError_t e = hipModuleLoadData(&m->mod, code.data());
    if (e != hipSuccess) {
      delete m;
      return hip_fail(ctx->err, "hipModuleLoadData", e);
    }
    m->key = src;
    ctx->modcache.emplace(m->key, m);
  }

  hipFunction_t fn = nullptr;
  hipError_t e = hipModuleGetFunction(&fn, m->mod, fname);
  if (e != hipSuccess)
    return ga_err_fmt(ctx->err, GA_IMPL_ERROR, "Kernel entry point \"%s\" not found: %s", fname,
                      hipGetErrorString(e));

  hip_kernel *k = (hip_kernel *)calloc(1, sizeof(hip_kernel));
  if (k == nullptr) return ga_err_sys(ctx->err, "calloc");
  k->ctx = ctx;
  k->fn = fn;
  k->mod = m;
  k->refcnt = 1;
  k->argcount = numargs;
  k->types = (int *)calloc(numargs ? numargs : 1, sizeof(int));
  k->argoff = (size_t *)calloc(numargs ? numargs : 1, sizeof(size_t));
  k->args = (void **)calloc(numargs ? numargs : 1, sizeof(void *));
  size_t store = 0;
  for (unsigned int i = 0; i < numargs; i++) {
    size_t s = typecodes[i] == GA_BUFFER ? 0 : gpuarray_get_elsize(typecodes[i]);
    store = (store + 15) & ~(size_t)15;
    if (k->argoff) k->argoff[i] = store;
    store += s;
  }
  k->argstore = (unsigned char *)calloc(store ? store : 1, 1);
  if (!k->types || !k->argoff || !k->args || !k->argstore) {
    free(k->types); free(k->argoff); free(k->args); free(k->argstore); free(k);
    return ga_err_sys(ctx->err, "calloc");
  }
  memcpy(k->types, typecodes, numargs * sizeof(int));
  int maxt = 0;
  if (hipFuncGetAttribute(&maxt, HIP_FUNC_ATTRIBUTE_MAX_THREADS_PER_BLOCK, fn) != hipSuccess ||
      maxt <= 0)
    maxt = (int)ctx->maxthreads;
  k->maxlsize = (size_t)maxt;
  m->refcnt++;
  ctx->refcnt++;
  *out = k;
  return GA_NO_ERROR;
}

void hip_retainkernel(gpukernel *k) { HK(k)->refcnt++; }

void hip_freekernel(gpukernel *kk) {
  hip_kernel *k = HK(kk);
  if (--k->refcnt != 0) return;
  hip_context *ctx = HC(k->ctx);
  mod_unref(ctx, k->mod);
  free(k->types);
  free(k->argoff);
  free(k->args);
  free(k->argstore);
  free(k);
  ctx_unref(ctx);
}

// By-value arguments are copied at once (the caller's variable may be gone by
// the time of the launch); buffer arguments record the gpudata, whose device
// pointer is read at launch.
int hip_setarg(gpukernel *kk, unsigned int i, void *a) {
  hip_kernel *k = HK(kk);
  if (i >= k->argcount)
    return ga_err_set(k->ctx->err, GA_VALUE_ERROR, "index is beyond the last argument");
  if (a == nullptr)
    return ga_err_fmt(k->ctx->err, GA_VALUE_ERROR, "NULL value for argument %u", i);
  if (k->types[i] == GA_BUFFER) {
    k->args[i] = a;
  } else {
    memcpy(k->argstore + k->argoff[i], a, gpuarray_get_elsize(k->types[i]));
    k->args[i] = k->argstore + k->argoff[i];
  }
  return GA_NO_ERROR;
}

int hip_callkernel(gpukernel *kk, unsigned int n, const size_t *gs, const size_t *ls,
                   size_t shared, void **args) {
  hip_kernel *k = HK(kk);
  hip_context *ctx = HC(k->ctx);
  if (n < 1 || n > 3)
    return ga_err_set(ctx->err, GA_VALUE_ERROR, "Call with a number of dimensions outside 1..3");
  if (args == nullptr) args = k->args;
  unsigned int g[3] = {1, 1, 1}, l[3] = {1, 1, 1};
  size_t lanes = 1;
  for (unsigned int d = 0; d < n; d++) {
    if (gs[d] == 0 || ls[d] == 0)
      return ga_err_fmt(ctx->err, GA_VALUE_ERROR, "Empty launch: gs[%u]=%zu ls[%u]=%zu", d, gs[d],
                        d, ls[d]);
    if (gs[d] > ctx->maxg[d] || ls[d] > ctx->maxl[d])
      return ga_err_fmt(ctx->err, GA_VALUE_ERROR,
                        "Launch size out of range on dimension %u: gs=%zu (max %zu) ls=%zu (max %zu)",
                        d, gs[d], ctx->maxg[d], ls[d], ctx->maxl[d]);
    g[d] = (unsigned int)gs[d];
    l[d] = (unsigned int)ls[d];
    lanes *= ls[d];
  }
  if (lanes > k->maxlsize)
    return ga_err_fmt(ctx->err, GA_VALUE_ERROR, "Group of %zu lanes exceeds the kernel's limit of %zu",
                      lanes, k->maxlsize);
  if (shared > ctx->lmemsize)
    return ga_err_fmt(ctx->err, GA_VALUE_ERROR, "%zu bytes of local memory requested, %zu available",
                      shared, ctx->lmemsize);
  void *stackp[32];
  std::vector<void *> heapp;
  void **params = stackp;
  if (k->argcount > 32) {
    heapp.resize(k->argcount);
    params = heapp.data();
  }
  for (unsigned int i = 0; i < k->argcount; i++) {
    if (args[i] == nullptr)
      return ga_err_fmt(ctx->err, GA_VALUE_ERROR, "Argument %u was never set", i);
    // a gpudata starts with its device pointer, so its address is the
    // address of the pointer argument
    params[i] = args[i];
  }
  int err;
  if ((err = enter(ctx)) != GA_NO_ERROR) return err;
  HIP_TRY(ctx, hipModuleLaunchKernel(k->fn, g[0], g[1], g[2], l[0], l[1], l[2],
                                     (unsigned int)shared, ctx->stream, params, nullptr));
  return GA_NO_ERROR;
}

// ---- properties ---------------------------------------------------------------

int hip_property(gpucontext *c, gpudata *buf, gpukernel *k, int prop_id, void *res) {
  hip_context *ctx = nullptr;
  if (c != nullptr) ctx = HC(c);
  else if (buf != nullptr) ctx = HC(buf->ctx);
  else if (k != nullptr) ctx = HC(k->ctx);
  ga_errrec *err = ctx ? ctx->err : ga_global_err;

  if (prop_id < GA_BUFFER_PROP_START) {
    if (ctx == nullptr)
      return ga_err_set(err, GA_VALUE_ERROR, "Attempting to get a context property with no context");
  } else if (prop_id < GA_KERNEL_PROP_START) {
    if (buf == nullptr)
      return ga_err_set(err, GA_VALUE_ERROR, "Attempting to get a buffer property with no buffer");
  } else if (k == nullptr) {
    return ga_err_set(err, GA_VALUE_ERROR, "Attempting to get a kernel property with no kernel");
  }

  switch (prop_id) {
  case GA_CTX_PROP_DEVNAME:
    memcpy(res, ctx->devname, 256);
    return GA_NO_ERROR;
  case GA_CTX_PROP_UNIQUE_ID:
    memcpy(res, ctx->pciid, 16);
    return GA_NO_ERROR;
  case GA_CTX_PROP_LMEMSIZE:
    *(size_t *)res = ctx->lmemsize;
    return GA_NO_ERROR;
  case GA_CTX_PROP_NUMPROCS:
    *(unsigned int *)res = ctx->numprocs;
    return GA_NO_ERROR;
  case GA_CTX_PROP_BIN_ID:
    *(const char **)res = ctx->bin_id;
    return GA_NO_ERROR;
  case GA_CTX_PROP_ERRBUF:
    *(gpudata **)res = ctx->errbuf;
    return GA_NO_ERROR;
  case GA_CTX_PROP_TOTAL_GMEM:
  case GA_CTX_PROP_FREE_GMEM:
  case GA_CTX_PROP_LARGEST_MEMBLOCK: {
    size_t fr = 0, tot = 0;
    int e;
    if ((e = enter(ctx)) != GA_NO_ERROR) return e;
    HIP_TRY(ctx, hipMemGetInfo(&fr, &tot));
    *(size_t *)res = prop_id == GA_CTX_PROP_TOTAL_GMEM ? tot : fr;
    return GA_NO_ERROR;
  }
  case GA_CTX_PROP_NATIVE_FLOAT16:
    *(int *)res = 1;
    return GA_NO_ERROR;
  case GA_CTX_PROP_MAXGSIZE0:
  case GA_CTX_PROP_MAXGSIZE1:
  case GA_CTX_PROP_MAXGSIZE2:
    *(size_t *)res = ctx->maxg[prop_id - GA_CTX_PROP_MAXGSIZE0];
    return GA_NO_ERROR;
  case GA_CTX_PROP_MAXLSIZE0:
  case GA_CTX_PROP_MAXLSIZE1:
  case GA_CTX_PROP_MAXLSIZE2:
    *(size_t *)res = ctx->maxl[prop_id - GA_CTX_PROP_MAXLSIZE0];
    return GA_NO_ERROR;
  case GA_BUFFER_PROP_REFCNT:
    *(unsigned int *)res = HD(buf)->refcnt;
    return GA_NO_ERROR;
  case GA_BUFFER_PROP_SIZE:
    *(size_t *)res = HD(buf)->sz;
    return GA_NO_ERROR;
  case GA_BUFFER_PROP_CTX:
  case GA_KERNEL_PROP_CTX:
    *(gpucontext **)res = ctx;
    return GA_NO_ERROR;
  case GA_KERNEL_PROP_MAXLSIZE:
    *(size_t *)res = HK(k)->maxlsize;
    return GA_NO_ERROR;
  case GA_KERNEL_PROP_PREFLSIZE:
    *(size_t *)res = 64;   // one wavefront
    return GA_NO_ERROR;
  case GA_KERNEL_PROP_NUMARGS:
    *(unsigned int *)res = HK(k)->argcount;
    return GA_NO_ERROR;
  case GA_KERNEL_PROP_TYPES:
    *(const int **)res = HK(k)->types;
    return GA_NO_ERROR;
  default:
    return ga_err_fmt(err, GA_INVALID_ERROR, "Invalid property: %d", prop_id);
  }
}

const char *hip_error(gpucontext *c) {
  if (c == nullptr) return ga_global_err->msg;
  return c->err->msg;
}

// ---- extension hooks ----------------------------------------------------------

void *ext_get_stream(gpucontext *c) { return (void *)HC(c)->stream; }
void *ext_get_ptr(gpudata *b) { return b->devptr; }
size_t ext_get_sz(gpudata *b) { return HD(b)->sz; }

gpudata *ext_make_buf(gpucontext *c, void *devptr, size_t sz) {
  hip_context *ctx = HC(c);
  hip_data *b = (hip_data *)calloc(1, sizeof(hip_data));
  if (b == nullptr) {
    ga_err_sys(ctx->err, "calloc");
    return nullptr;
  }
  b->devptr = devptr;
  b->ctx = ctx;
  b->sz = sz;
  b->refcnt = 1;
  b->flags = 0;   // not owned: release leaves the memory alone
  ctx->refcnt++;
  return b;
}

int ext_compile_only(unsigned int count, const char **strs, const size_t *lens, char **log) {
  std::vector<char> code;
  std::string l;
  int err = rtc_compile(join_sources(count, strs, lens), code, l);
  if (log) *log = l.empty() ? nullptr : strdup(l.c_str());
  if (err != GA_NO_ERROR) ga_err_fmt(ga_global_err, err, "Kernel compilation failed: %.900s", l.c_str());
  return err;
}

int ext_time_begin(gpucontext *c) {
  hip_context *ctx = HC(c);
  int err;
  if ((err = enter(ctx)) != GA_NO_ERROR) return err;
  HIP_TRY(ctx, hipEventRecord(ctx->ev0, ctx->stream));
  return GA_NO_ERROR;
}

float ext_time_end(gpucontext *c) {
  hip_context *ctx = HC(c);
  float ms = -1.0f;
  if (enter(ctx) != GA_NO_ERROR) return -1.0f;
  if (hipEventRecord(ctx->ev1, ctx->stream) != hipSuccess) return -1.0f;
  if (hipEventSynchronize(ctx->ev1) != hipSuccess) return -1.0f;
  if (hipEventElapsedTime(&ms, ctx->ev0, ctx->ev1) != hipSuccess) return -1.0f;
  return ms;
}

}  // namespace
// Kernel text generators, defined next to the planners that use them.
extern "C" char *ga_elemwise_gen_source(const char *preamble, const char *expr, unsigned int n,
                                        gpuelemwise_arg *args, int flags, int strided,
                                        unsigned int nd, int idx64, unsigned int tmask);
extern "C" char *ga_reduction_gen_source(int op, int src_tc, int d0_tc, int d1_tc, unsigned int G,
                                         unsigned int V, unsigned int U);
namespace {

// Numbered timing marks on the context's stream: record as many as wanted
// without waiting, read the spans afterwards.
int ext_event_record(gpucontext *c, unsigned int slot) {
  hip_context *ctx = HC(c);
  int err;
  if ((err = enter(ctx)) != GA_NO_ERROR) return err;
  while (ctx->evpool.size() <= slot) {
    hipEvent_t e = nullptr;
    HIP_TRY(ctx, hipEventCreate(&e));
    ctx->evpool.push_back(e);
  }
  HIP_TRY(ctx, hipEventRecord(ctx->evpool[slot], ctx->stream));
  return GA_NO_ERROR;
}

// Milliseconds between marks a and b; waits for b.  < 0 on error.
float ext_event_elapsed(gpucontext *c, unsigned int a, unsigned int b) {
  hip_context *ctx = HC(c);
  float ms = -1.0f;
  if (a >= ctx->evpool.size() || b >= ctx->evpool.size()) return -1.0f;
  if (enter(ctx) != GA_NO_ERROR) return -1.0f;
  if (hipEventSynchronize(ctx->evpool[b]) != hipSuccess) return -1.0f;
  if (hipEventElapsedTime(&ms, ctx->evpool[a], ctx->evpool[b]) != hipSuccess) return -1.0f;
  return ms;
}

struct ext_entry { const char *name; void *fn; };
const ext_entry k_exts[] = {
    {"hip_get_stream", (void *)ext_get_stream},
    {"hip_get_ptr", (void *)ext_get_ptr},
    {"hip_get_sz", (void *)ext_get_sz},
    {"hip_make_buf", (void *)ext_make_buf},
    {"hip_compile_only", (void *)ext_compile_only},
    {"hip_time_begin", (void *)ext_time_begin},
    {"hip_time_end", (void *)ext_time_end},
    {"hip_event_record", (void *)ext_event_record},
    {"hip_event_elapsed", (void *)ext_event_elapsed},
    {"hip_elemwise_source", (void *)ga_elemwise_gen_source},
    {"hip_reduction_source", (void *)ga_reduction_gen_source},
};

}  // namespace

extern "C" void *gpuarray_get_extension(const char *name) {
  if (name == nullptr) return nullptr;
  for (const auto &e : k_exts)
    if (strcmp(e.name, name) == 0) return e.fn;
  return nullptr;
}

gpudata *ga_hip_scratch(gpucontext *c, size_t bytes) {
  hip_context *ctx = HC(c);
  if (ctx->scratch != nullptr && ctx->scratch_sz >= bytes) return ctx->scratch;
  if (ctx->scratch != nullptr) {
    hip_release(ctx->scratch);   // hipFree waits for queued users
    ctx->scratch = nullptr;
    ctx->scratch_sz = 0;
  }
  size_t want = bytes < ((size_t)1 << 20) ? ((size_t)1 << 20) : bytes;
  ctx->scratch = hip_alloc(c, want, nullptr, BUF_INTERNAL);
  if (ctx->scratch != nullptr) ctx->scratch_sz = want;
  return ctx->scratch;
}

unsigned int ga_hip_numprocs(gpucontext *c) { return HC(c)->numprocs; }
void **ga_hip_redux_cache_slot(gpucontext *c) { return &HC(c)->redux_cache; }

const ga_buffer_ops ga_hip_ops = {
    hip_get_platform_count, hip_get_device_count, hip_init,        hip_deinit,
    hip_alloc,              hip_retain,           hip_release,     hip_share,
    hip_move,               hip_read,             hip_write,       hip_memset,
    hip_newkernel,          hip_retainkernel,     hip_freekernel,  hip_setarg,
    hip_callkernel,         hip_sync,             hip_transfer,    hip_property,
    hip_error};
