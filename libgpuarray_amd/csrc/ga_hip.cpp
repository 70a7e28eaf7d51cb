// The HIP backend: one device, one in-order stream, kernels compiled at run
// time for gfx950 through the code-object manager (libamd_comgr) and launched
// with hipModuleLaunchKernel.
//
// It fills the same 21-entry table the reference's backends fill
// (src/private.h:90-121).  The shape is that of the reference's CUDA backend
// (src/gpuarray_buffer_cuda.c: runtime compile -> module -> launch with an
// array of argument pointers, where a buffer argument is passed as the address
// of the gpudata itself because the device pointer is its first member,
// :1494-1525) but none of its machinery is needed: a single in-order stream
// orders all work, so there are no per-buffer events.
#include "private.hpp"

#ifdef DEBUG
#include <cassert>
#endif

#include <hip/hip_runtime_api.h>
#include <amd_comgr/amd_comgr.h>

#include <dlfcn.h>
#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>

#include <atomic>
#include <iterator>
#include <list>
#include <map>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

// Launch with a start and a stop event attached to the dispatch
// (declared in <hip/hip_ext.h>, which needs the device-side headers).
extern "C" hipError_t hipExtModuleLaunchKernel(hipFunction_t f, uint32_t globalWorkSizeX,
                                               uint32_t globalWorkSizeY, uint32_t globalWorkSizeZ,
                                               uint32_t localWorkSizeX, uint32_t localWorkSizeY,
                                               uint32_t localWorkSizeZ, size_t sharedMemBytes,
                                               hipStream_t hStream, void **kernelParams, void **extra,
                                               hipEvent_t startEvent, hipEvent_t stopEvent,
                                               uint32_t flags);

namespace {

struct hip_module {
  hipModule_t mod = nullptr;
  unsigned refcnt = 0;     // kernels made from this module
  bool cached = false;     // the module cache still lists it
  std::string key;
};

// ---- loaded-module cache ------------------------------------------------------
// Source text -> loaded code object, bounded by the reference's 2Q policy
// (src/cache/twoq.c:232-316, sized 64/128/64/8 by its CUDA backend,
// src/gpuarray_buffer_cuda.c:291): a new entry enters `hot`; when hot
// overflows its oldest entry moves to `cold`; a hit in cold promotes the entry
// to `warm`, whose overflow goes back to cold; cold is cut back to its size
// once it exceeds size + elasticity.  An entry that leaves the cache is
// unloaded when the last kernel made from it is gone.
class module_cache {
 public:
  typedef std::list<hip_module *> list_t;
  size_t hot_size = 64, warm_size = 128, cold_size = 64, elasticity = 8;

  hip_module *get(const std::string &key) {
    auto it = index_.find(key);
    if (it == index_.end()) return nullptr;
    slot &s = it->second;
    hip_module *m = *s.pos;
    switch (s.temp) {
    case HOT: hot_.splice(hot_.end(), hot_, s.pos); break;
    case WARM: warm_.splice(warm_.end(), warm_, s.pos); break;
    case COLD:
      warm_.splice(warm_.end(), cold_, s.pos);
      s.temp = WARM;
      if (warm_.size() > warm_size) {
        index_[warm_.front()->key].temp = COLD;
        cold_.splice(cold_.end(), warm_, warm_.begin());
      }
      break;
    }
    return m;
  }

  // Adds m (its key must not be listed); `evicted` receives what fell out.
  void add(hip_module *m, std::vector<hip_module *> &evicted) {
    hot_.push_back(m);
    index_[m->key] = {HOT, std::prev(hot_.end())};
    m->cached = true;
    while (hot_.size() > hot_size) {
      index_[hot_.front()->key].temp = COLD;
      cold_.splice(cold_.end(), hot_, hot_.begin());
    }
    if (cold_.size() > cold_size + elasticity) {
      while (cold_.size() > cold_size) {
        hip_module *old = cold_.front();
        cold_.pop_front();
        index_.erase(old->key);
        old->cached = false;
        evicted.push_back(old);
      }
    }
  }

  void counts(size_t out[3]) const { out[0] = hot_.size(); out[1] = warm_.size(); out[2] = cold_.size(); }

  // Empties the cache; every listed module is handed to `evicted`.
  void clear(std::vector<hip_module *> &evicted) {
    for (list_t *l : {&hot_, &warm_, &cold_}) {
      for (hip_module *m : *l) {
        m->cached = false;
        evicted.push_back(m);
      }
      l->clear();
    }
    index_.clear();
  }

 private:
  enum temp_t { HOT, WARM, COLD };
  struct slot {
    temp_t temp;
    list_t::iterator pos;
  };
  list_t hot_, warm_, cold_;
  std::unordered_map<std::string, slot> index_;
};

// ---- device memory cache ------------------------------------------------------
// hipMalloc and hipFree cost tens to hundreds of microseconds and hipFree
// waits for the device, so temporaries (results, copies) would dominate the
// time per call.  Freed buffers therefore go back to a per-context cache
// instead of to the driver.  The policy is the reference CUDA backend's
// (src/gpuarray_buffer_cuda.c:607-889): memory comes from the driver in
// segments of at least 4 MiB, requests are rounded up to a fragment size and
// served best-fit from the free blocks, a block is split when it is larger
// than needed and merged with free neighbours of the same segment when it
// comes back; `max` bounds what is taken from the driver (0 turns the cache
// off).  Unlike there, no events guard reuse: one in-order stream means work
// queued on a block before it was freed completes before anything queued
// after it is handed out again.  Fragments are 256 bytes, so every buffer is
// aligned for 16-byte vector access.  Lookups are O(log n): free blocks are
// indexed by size, all blocks by address.
struct mem_segment {
  char *base;
  size_t size;
};

struct mem_block {
  char *ptr;
  size_t size;
  bool is_free;
  mem_segment *seg;
};

struct mem_cache {
  static constexpr size_t FRAG = 256;
  static constexpr size_t SEG_MIN = (size_t)4 << 20;
  static constexpr size_t SEG_ROUND = (size_t)2 << 20;
  std::map<char *, mem_block *> by_addr;
  std::multimap<size_t, mem_block *> free_by_size;
  std::vector<mem_segment *> segs;
  size_t from_driver = 0;          // bytes currently held from hipMalloc
  size_t max = (size_t)-1;         // cap on from_driver; 0 = cache disabled

  void index_free(mem_block *b) { b->is_free = true; free_by_size.emplace(b->size, b); }
  void unindex_free(mem_block *b) {
    auto r = free_by_size.equal_range(b->size);
    for (auto it = r.first; it != r.second; ++it)
      if (it->second == b) { free_by_size.erase(it); break; }
    b->is_free = false;
  }

  // Give fully free segments back to the driver (when the device runs out).
  size_t trim() {
    size_t released = 0;
    for (size_t i = 0; i < segs.size();) {
      mem_segment *sg = segs[i];
      auto it = by_addr.find(sg->base);
      if (it != by_addr.end() && it->second->is_free && it->second->size == sg->size) {
        mem_block *b = it->second;
        unindex_free(b);
        by_addr.erase(it);
        delete b;
        (void)hipFree(sg->base);
        from_driver -= sg->size;
        released += sg->size;
        delete sg;
        segs.erase(segs.begin() + (long)i);
      } else {
        i++;
      }
    }
    return released;
  }

  // 0 ok, 1 cap reached, 2 device out of memory, 3 other driver error (*herr)
  int grow(size_t asize, hipError_t *herr) {
    size_t want = asize < SEG_MIN ? SEG_MIN : ((asize + SEG_ROUND - 1) / SEG_ROUND) * SEG_ROUND;
    if (want < asize) return 2;   // overflow
    if (max != (size_t)-1 && (from_driver > max || want > max - from_driver)) {
      // try again with exactly what is needed before giving up
      want = asize;
      if (from_driver > max || want > max - from_driver) {
        trim();
        if (from_driver > max || want > max - from_driver) return 1;
      }
    }
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, want);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      if (trim() > 0) e = hipMalloc(&p, want);
      if (e != hipSuccess && want != asize) { (void)hipGetLastError(); want = asize; e = hipMalloc(&p, want); }
    }
    if (e != hipSuccess) {
      (void)hipGetLastError();
      *herr = e;
      return (e == hipErrorOutOfMemory || e == hipErrorMemoryAllocation) ? 2 : 3;
    }
    mem_segment *sg = new mem_segment{(char *)p, want};
    segs.push_back(sg);
    from_driver += want;
    mem_block *b = new mem_block{(char *)p, want, false, sg};
    by_addr.emplace(b->ptr, b);
    index_free(b);
    return 0;
  }

  mem_block *take(size_t size, int *why, hipError_t *herr) {
    size_t asize = ((size ? size : 1) + FRAG - 1) / FRAG * FRAG;
    if (asize < size) { *why = 2; return nullptr; }
    auto it = free_by_size.lower_bound(asize);
    if (it == free_by_size.end()) {
      if ((*why = grow(asize, herr)) != 0) return nullptr;
      it = free_by_size.lower_bound(asize);
    }
    mem_block *b = it->second;
    free_by_size.erase(it);
    b->is_free = false;
    if (b->size - asize >= FRAG) {
      mem_block *rest = new mem_block{b->ptr + asize, b->size - asize, false, b->seg};
      b->size = asize;
      by_addr.emplace(rest->ptr, rest);
      index_free(rest);
    }
    return b;
  }

  void give_back(mem_block *b) {
    auto it = by_addr.find(b->ptr);
    // merge with the next block of the same segment
    auto nx = std::next(it);
    if (nx != by_addr.end() && nx->second->is_free && nx->second->seg == b->seg &&
        b->ptr + b->size == nx->second->ptr) {
      mem_block *n = nx->second;
      unindex_free(n);
      b->size += n->size;
      by_addr.erase(nx);
      delete n;
    }
    // and with the previous one
    if (it != by_addr.begin()) {
      auto pv = std::prev(it);
      mem_block *p = pv->second;
      if (p->is_free && p->seg == b->seg && p->ptr + p->size == b->ptr) {
        unindex_free(p);
        p->size += b->size;
        by_addr.erase(it);
        delete b;
        b = p;
      }
    }
    index_free(b);
  }

  void destroy() {
    for (auto &kv : by_addr) delete kv.second;
    by_addr.clear();
    free_by_size.clear();
    for (mem_segment *sg : segs) { (void)hipFree(sg->base); delete sg; }
    segs.clear();
    from_driver = 0;
  }

  size_t largest_free() const {
    return free_by_size.empty() ? 0 : free_by_size.rbegin()->first;
  }
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
  module_cache modcache;
  size_t live_modules = 0;   // loaded code objects, cached or still referenced
  gpudata *scratch = nullptr;
  size_t scratch_sz = 0;
  std::vector<gpudata *> retired_scratch;   // outgrown scratch buffers, kept until teardown
  void *static_scratch = nullptr;           // this device's copy of the static scratch array
  int static_scratch_err = 0;               // HIP error code of its lookup
  gpudata *static_buf = nullptr;            // that array as a buffer of the context (not owned, not counted)
  gpudata *redux_counters = nullptr;   // zeroed counters of single-launch split reductions
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  std::vector<hipEvent_t> evpool;   // timing marks for callers (hip_event_* hooks)
  // hip_kernel_timing: while on, every launch carries its own start and stop
  // event (pairs [2i], [2i+1] of ktime_ev; ktime_n launches recorded so far)
  bool ktime_on = false;
  std::vector<hipEvent_t> ktime_ev;
  size_t ktime_n = 0;
  std::vector<uint64_t> ktime_hash;   // text_hash of each recorded launch
  uint64_t last_launch_hash = 0;   // text_hash of the kernel launched last
  void *redux_cache = nullptr;
  void *take1_cache = nullptr;
  mem_cache mem;
  std::string disk_cache;   // directory of the on-disk kernel cache, empty = off
  void *stage = nullptr;    // pinned host memory that small reads and writes go through
  gpukernel *copy_kernel = nullptr;   // byte copy behind buffer_move
  gpukernel *fill_kernel = nullptr;   // byte fill behind buffer_memset
  bool stage_failed = false;
  ga_tuning tuning;        // the planners' knobs, as read from the environment when the context was made
  ga_errrec errstore;
};

// Small transfers bounce off pinned memory: the driver copies between a
// device and pageable host memory through a path that costs about 23 us for
// four bytes on MI355X; between a device and pinned memory the same copy
// takes 15 us.  Results read back one scalar at a time (the value of a full
// sum, the bounds flag of take1) are the common case.
const size_t STAGE_BYTES = 64 * 1024;

void *stage_of(hip_context *ctx) {
  if (ctx->stage == nullptr && !ctx->stage_failed) {
    if (hipHostMalloc(&ctx->stage, STAGE_BYTES, hipHostMallocDefault) != hipSuccess) {
      (void)hipGetLastError();
      ctx->stage = nullptr;
      ctx->stage_failed = true;
    }
  }
  return ctx->stage;
}

#define BUF_OWNED 0x10000      /* devptr came from hipMalloc */
#define BUF_INTERNAL 0x20000   /* does not keep the context alive */
#define BUF_HOSTMEM 0x40000    /* devptr is pinned host memory that kernels can write */

// The reference's debugging aid (src/private_cuda.h:12-40): in a DEBUG build
// contexts, buffers and kernels carry an 8-byte tag, set when the object is made
// and wiped when it is freed, and every entry of the backend asserts the tag of
// what it was handed: a stale or foreign pointer stops at the door instead of
// corrupting something later.  (A context carries its tag in every build: it is
// part of the struct's public head.)
#define CTX_TAG "hipctx "
#ifdef DEBUG
#define BUF_TAG "hipbuf  "
#define KER_TAG "hipkern "
#define TAG_BUF(b) memcpy((b)->tag, BUF_TAG, 8)
#define TAG_KER(k) memcpy((k)->tag, KER_TAG, 8)
#define ASSERT_CTX(c) assert(memcmp((c)->tag, CTX_TAG, 8) == 0)
#define ASSERT_BUF(b) assert(memcmp((b)->tag, BUF_TAG, 8) == 0)
#define ASSERT_KER(k) assert(memcmp((k)->tag, KER_TAG, 8) == 0)
#define CLEAR_TAG(o) memset((o)->tag, 0, 8)
#else
#define TAG_BUF(b)
#define TAG_KER(k)
#define ASSERT_CTX(c)
#define ASSERT_BUF(b)
#define ASSERT_KER(k)
#define CLEAR_TAG(o)
#endif

struct hip_data : _gpudata {
  size_t sz;
  unsigned int refcnt;
  int flags;
  mem_block *block;   // cache block behind devptr; NULL when taken straight from the driver
#ifdef DEBUG
  char tag[8];
#endif
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
  uint64_t text_hash;    // FNV-1a of the source text followed by the entry point's name
#ifdef DEBUG
  char tag[8];
#endif
};

// (a NULL passes: the callers that allow one test for it themselves)
inline hip_context *HC(gpucontext *c) {
  if (c != nullptr) { ASSERT_CTX(c); }
  return static_cast<hip_context *>(c);
}
inline hip_data *HD(gpudata *b) {
  if (b != nullptr) { ASSERT_BUF(static_cast<hip_data *>(b)); }
  return static_cast<hip_data *>(b);
}
inline hip_kernel *HK(gpukernel *k) {
  if (k != nullptr) { ASSERT_KER(static_cast<hip_kernel *>(k)); }
  return static_cast<hip_kernel *>(k);
}

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
void hip_freekernel(gpukernel *kk);

void ctx_destroy(hip_context *ctx) {
  (void)hipSetDevice(ctx->dev);
  // internal buffers do not count as owners, so they are still here
  if (ctx->errbuf) { hip_release(ctx->errbuf); ctx->errbuf = nullptr; }
  if (ctx->scratch) { hip_release(ctx->scratch); ctx->scratch = nullptr; }
  if (ctx->static_buf) { hip_release(ctx->static_buf); ctx->static_buf = nullptr; }
  for (gpudata *b : ctx->retired_scratch) hip_release(b);
  ctx->retired_scratch.clear();
  if (ctx->redux_counters) { hip_release(ctx->redux_counters); ctx->redux_counters = nullptr; }
  ctx->mem.destroy();
  {
    // every kernel is gone by now (each one holds a reference to the context)
    std::vector<hip_module *> gone;
    ctx->modcache.clear(gone);
    for (hip_module *m : gone) {
      if (m->mod) (void)hipModuleUnload(m->mod);
      delete m;
    }
  }
  for (hipEvent_t e : ctx->evpool) (void)hipEventDestroy(e);
  for (hipEvent_t e : ctx->ktime_ev) (void)hipEventDestroy(e);
  if (ctx->ev0) (void)hipEventDestroy(ctx->ev0);
  if (ctx->ev1) (void)hipEventDestroy(ctx->ev1);
  if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
  if (ctx->stage) (void)hipHostFree(ctx->stage);
  memset(ctx->tag, 0, 8);   // (in every build: a freed context no longer looks like one)
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
  memcpy(ctx->tag, CTX_TAG, 8);
  ctx->dev = dev;
  ga_tuning_read(&ctx->tuning);

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
  // Every kernel is compiled for gfx950 (wave64, its DPP and LDS forms): say
  // so here rather than at the first module load on another ISA.
  if (strcmp(ctx->bin_id, "gfx950") != 0 && TUNE(&ctx->tuning, ALLOW_OTHER_ISA, 0) == 0) {
    ga_err_fmt(ga_global_err, GA_DEVSUP_ERROR,
               "Device %d is %s; this library generates code for gfx950 (MI355X) only", dev, ctx->bin_id);
    ctx_destroy(ctx);
    return nullptr;
  }
  // Where this device keeps the library's static scratch array (the partials
  // of GpuReduction_call_noalloc).  A failed lookup only disables that entry
  // point, which then reports the code kept here.
  ctx->static_scratch_err = ga_static_scratch_setup(dev, &ctx->static_scratch);
  if (ctx->static_scratch != nullptr) {
    // made here, so that the entry point that may not allocate finds it ready
    hip_data *b = (hip_data *)calloc(1, sizeof(hip_data));
    if (b != nullptr) {
      TAG_BUF(b);
      b->devptr = ctx->static_scratch;
      b->ctx = ctx;
      b->sz = ga_static_scratch_bytes;
      b->refcnt = 1;
      b->flags = BUF_INTERNAL;   // not owned (release leaves the memory alone), does not keep the context alive
      ctx->static_buf = b;
    }
  }

  {
    const char *dc = p->kernel_cache_path ? p->kernel_cache_path : getenv("GPUARRAY_CACHE_PATH");
    if (dc != nullptr && *dc != 0) ctx->disk_cache = dc;
  }
  {
    // "hot,warm,cold,elasticity" overrides the module cache's sizes
    const char *mc = getenv("GPUARRAY_MODULE_CACHE");
    unsigned long h, w, c, el;
    if (mc != nullptr && sscanf(mc, "%lu,%lu,%lu,%lu", &h, &w, &c, &el) == 4 && h >= 1) {
      ctx->modcache.hot_size = h;
      ctx->modcache.warm_size = w;
      ctx->modcache.cold_size = c;
      ctx->modcache.elasticity = el;
    }
  }
  ctx->mem.max = p->max_cache_size;
  if (p->initial_cache_size != 0 && ctx->mem.max != 0) {
    // reserve the first segment now (reference src/gpuarray_buffer_cuda.c:349-356)
    gpudata *warm = hip_alloc(ctx, p->initial_cache_size, nullptr, BUF_INTERNAL);
    if (warm == nullptr) {
      ga_err_set(ga_global_err, ctx->err->code, ctx->err->msg);
      ctx_destroy(ctx);
      return nullptr;
    }
    hip_release(warm);
  }

  // 8 zeroed bytes kernels can use to report a fault
  // (reference GA_CTX_PROP_ERRBUF, src/gpuarray/buffer.h:646-658).
  // They live in pinned host memory: a kernel that finds a fault stores
  // there, and the host reads the flag after waiting for the stream, without
  // a copy (take1 of 64 rows: 27 us per call with a device flag read back, of
  // which 23 us were the blocking four-byte copy).
  uint64_t zero = 0;
  {
    void *flag = nullptr;
    hip_data *b = (hip_data *)calloc(1, sizeof(hip_data));
    if (b != nullptr && hipHostMalloc(&flag, 64, hipHostMallocCoherent) == hipSuccess) {
      memset(flag, 0, 64);
      TAG_BUF(b);
      b->devptr = flag;
      b->ctx = ctx;
      b->sz = 8;
      b->refcnt = 1;
      b->flags = BUF_INTERNAL | BUF_HOSTMEM;
      ctx->errbuf = b;
    } else {
      (void)hipGetLastError();
      free(b);
    }
  }
  if (ctx->errbuf == nullptr) ctx->errbuf = hip_alloc(ctx, 8, &zero, GA_BUFFER_INIT | BUF_INTERNAL);
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
  ga_take1_cache_free(c);
  if (ctx->fill_kernel) {
    hip_freekernel(ctx->fill_kernel);
    ctx->fill_kernel = nullptr;
  }
  if (ctx->copy_kernel) {
    hip_freekernel(ctx->copy_kernel);
    ctx->copy_kernel = nullptr;
  }
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
  TAG_BUF(b);
  size_t asz = sz ? sz : 1;   // a zero-byte request still yields a valid buffer
  if (ctx->mem.max != 0) {
    int why = 0;
    hipError_t herr = hipSuccess;
    mem_block *blk = ctx->mem.take(asz, &why, &herr);
    if (blk == nullptr) {
      free(b);
      if (why == 1)
        ga_err_set(ctx->err, GA_VALUE_ERROR, "Maximum cache size reached");
      else if (why == 2)
        ga_err_fmt(ctx->err, GA_MEMORY_ERROR, "hipMalloc(%zu): out of device memory", asz);
      else
        hip_fail(ctx->err, "hipMalloc", herr);
      return nullptr;
    }
    b->devptr = blk->ptr;
    b->block = blk;   // the block may be larger; sz stays the size asked for
  } else {
    hipError_t e = hipMalloc(&b->devptr, asz);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      free(b);
      if (e == hipErrorOutOfMemory || e == hipErrorMemoryAllocation)
        ga_err_fmt(ctx->err, GA_MEMORY_ERROR, "hipMalloc(%zu): out of device memory", asz);
      else
        hip_fail(ctx->err, "hipMalloc", e);
      return nullptr;
    }
  }
  b->ctx = ctx;
  b->sz = asz;
  b->refcnt = 1;
  b->flags = (flags & (GA_BUFFER_MASK | BUF_INTERNAL)) | BUF_OWNED;
  if (flags & GA_BUFFER_INIT) {
    hipError_t e = hipMemcpyHtoDAsync(b->devptr, data, sz, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
      hip_fail(ctx->err, "hipMemcpyHtoDAsync", e);
      if (b->block) ctx->mem.give_back(b->block);
      else (void)hipFree(b->devptr);
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
  if (b->flags & BUF_HOSTMEM) {
    (void)hipSetDevice(ctx->dev);
    (void)hipHostFree(b->devptr);
  } else if (b->block != nullptr) {
    // back to the cache; stream order protects work still queued on it
    ctx->mem.give_back(b->block);
  } else if (b->flags & BUF_OWNED) {
    (void)hipSetDevice(ctx->dev);
    // hipFree waits for the device, so queued work that still uses the
    // memory completes first.
    (void)hipFree(b->devptr);
  }
  bool counted = !(b->flags & BUF_INTERNAL);
  CLEAR_TAG(b);
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

int hip_newkernel(gpukernel **out, gpucontext *c, unsigned int count, const char **strings,
                  const size_t *lengths, const char *fname, unsigned int numargs,
                  const int *typecodes, int flags, char **err_str);
int hip_callkernel(gpukernel *kk, unsigned int n, const size_t *gs, const size_t *ls,
                   size_t shared, void **args);

// Copy of n bytes between ranges that sit equally far from a 16-byte
// boundary: one 16-byte streaming chunk per lane, the bytes before the first
// and after the last whole chunk one per lane.
const char COPY_KERNEL_SRC[] =
    "#include \"cluda.h\"\n"
    "typedef ga_uint __attribute__((ext_vector_type(4))) ga_chunk16;\n"
    "KERNEL void __launch_bounds__(256) ga_copy(GLOBAL_MEM char *dst, const ga_size doff,\n"
    "    GLOBAL_MEM const char *src, const ga_size soff, const ga_size head,\n"
    "    const ga_size nchunks, const ga_size n) {\n"
    "  dst += doff; src += soff;\n"
    "  const ga_size t = (ga_size)GID_0 * 256 + LID_0;\n"
    "  if (t < nchunks) {\n"
    "    const ga_chunk16 v = __builtin_nontemporal_load((const ga_chunk16 *)(src + head) + t);\n"
    "    __builtin_nontemporal_store(v, (ga_chunk16 *)(dst + head) + t);\n"
    "  }\n"
    "  const ga_size rest = n - nchunks * 16;\n"
    "  if (t < rest) {\n"
    "    const ga_size i = t < head ? t : t + nchunks * 16;\n"
    "    dst[i] = src[i];\n"
    "  }\n"
    "}\n";

int hip_move(gpudata *dst, size_t dstoff, gpudata *src, size_t srcoff, size_t sz) {
  hip_context *ctx = HC(dst->ctx);
  if (dst->ctx != src->ctx)
    return ga_err_set(ctx->err, GA_VALUE_ERROR, "Cannot move between contexts");
  if (sz == 0) return GA_NO_ERROR;
  int err;
  if ((err = range_check(ctx, HD(dst), dstoff, sz, "move dst")) != GA_NO_ERROR) return err;
  if ((err = range_check(ctx, HD(src), srcoff, sz, "move src")) != GA_NO_ERROR) return err;
  if ((err = enter(ctx)) != GA_NO_ERROR) return err;
  // Measured on MI355X, reads plus writes: 1 GiB at 5.1 TB/s with the driver's
  // device-to-device copy and 6.65 with the kernel above; 64 MiB 28.1 against
  // 23.8 us; 16 MiB 7.5 against 8.9 us, and below that no difference.
  const uintptr_t da = (uintptr_t)dst->devptr + dstoff, sa = (uintptr_t)src->devptr + srcoff;
  if (sz >= TUNE(&ctx->tuning, MOVE_KERNEL_MIN, 32u << 20) && (da - sa) % 16 == 0 &&
      !((HD(dst)->flags | HD(src)->flags) & BUF_HOSTMEM)) {
    if (ctx->copy_kernel == nullptr) {
      const char *strs[1] = {COPY_KERNEL_SRC};
      const int types[7] = {GA_BUFFER, GA_SIZE, GA_BUFFER, GA_SIZE, GA_SIZE, GA_SIZE, GA_SIZE};
      if ((err = hip_newkernel(&ctx->copy_kernel, ctx, 1, strs, nullptr, "ga_copy", 7, types, 0,
                               nullptr)) != GA_NO_ERROR)
        return err;
    }
    size_t head = (16 - da % 16) % 16;
    if (head > sz) head = sz;   // a range that ends before its first boundary
    size_t nchunks = (sz - head) / 16;
    const size_t rest = sz - nchunks * 16;
    size_t gs = (std::max(nchunks, rest) + 255) / 256, ls = 256;
    void *args[7] = {dst, &dstoff, src, &srcoff, &head, &nchunks, &sz};
    return hip_callkernel(ctx->copy_kernel, 1, &gs, &ls, 0, args);
  }
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
  if (HD(src)->flags & BUF_HOSTMEM) {   // the host can read it once queued kernels are done
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    memcpy(dst, (char *)src->devptr + srcoff, sz);
    return GA_NO_ERROR;
  }
  void *stage = sz <= STAGE_BYTES ? stage_of(ctx) : nullptr;
  HIP_TRY(ctx, hipMemcpyDtoHAsync(stage ? stage : dst, (char *)src->devptr + srcoff, sz, ctx->stream));
  HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
  if (stage) memcpy(dst, stage, sz);
  return GA_NO_ERROR;
}

int hip_write(gpudata *dst, size_t dstoff, const void *src, size_t sz) {
  hip_context *ctx = HC(dst->ctx);
  if (sz == 0) return GA_NO_ERROR;
  int err;
  if ((err = range_check(ctx, HD(dst), dstoff, sz, "write")) != GA_NO_ERROR) return err;
  if ((err = enter(ctx)) != GA_NO_ERROR) return err;
  if (HD(dst)->flags & BUF_HOSTMEM) {
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    memcpy((char *)dst->devptr + dstoff, src, sz);
    return GA_NO_ERROR;
  }
  void *stage = sz <= STAGE_BYTES ? stage_of(ctx) : nullptr;
  if (stage) memcpy(stage, src, sz);
  HIP_TRY(ctx, hipMemcpyHtoDAsync((char *)dst->devptr + dstoff,
                                  stage ? stage : const_cast<void *>(src), sz, ctx->stream));
  // the host memory belongs to the caller again on return
  HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
  return GA_NO_ERROR;
}

// Fill from dstoff to the end of the buffer with the low byte of `data`.
// Fill of n bytes with one value: one 16-byte streaming chunk per lane, the
// bytes before the first and after the last whole chunk one per lane.
const char FILL_KERNEL_SRC[] =
    "#include \"cluda.h\"\n"
    "typedef ga_uint __attribute__((ext_vector_type(4))) ga_chunk16;\n"
    "KERNEL void __launch_bounds__(256) ga_fill(GLOBAL_MEM char *dst, const ga_size doff,\n"
    "    const ga_size head, const ga_size nchunks, const ga_size n, const ga_uint word) {\n"
    "  dst += doff;\n"
    "  const ga_size t = (ga_size)GID_0 * 256 + LID_0;\n"
    "  if (t < nchunks) {\n"
    "    const ga_chunk16 v = {word, word, word, word};\n"
    "    __builtin_nontemporal_store(v, (ga_chunk16 *)(dst + head) + t);\n"
    "  }\n"
    "  const ga_size rest = n - nchunks * 16;\n"
    "  if (t < rest) dst[t < head ? t : t + nchunks * 16] = (char)word;\n"
    "}\n";

int hip_memset(gpudata *dst, size_t dstoff, int data) {
  hip_context *ctx = HC(dst->ctx);
  hip_data *b = HD(dst);
  if (dstoff > b->sz)
    return ga_err_set(ctx->err, GA_VALUE_ERROR, "memset offset is past the end of the buffer");
  size_t n = b->sz - dstoff;
  if (n == 0) return GA_NO_ERROR;
  int err;
  if ((err = enter(ctx)) != GA_NO_ERROR) return err;
  if (b->flags & BUF_HOSTMEM) {
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    memset((char *)b->devptr + dstoff, data & 0xff, n);
    return GA_NO_ERROR;
  }
  // The library's own kernel whenever the stream records a graph: a memset
  // recorded into a graph is a node of its own kind, and such nodes have
  // replayed wrongly.  Otherwise the driver's fill, which is as fast (measured
  // on MI355X, 30 fills back to back: 1 GiB 161.7 us against 160.1 with this
  // kernel, 64 MiB 11.7 / 11.5, 16 MiB 5.2 / 4.7, 1 MiB 4.4 / 4.7).
  if (ga_hip_capturing(dst->ctx) || n >= TUNE(&ctx->tuning, FILL_KERNEL_MIN, ~0ul)) {
    if (ctx->fill_kernel == nullptr) {
      const char *strs[1] = {FILL_KERNEL_SRC};
      const int types[6] = {GA_BUFFER, GA_SIZE, GA_SIZE, GA_SIZE, GA_SIZE, GA_UINT};
      if ((err = hip_newkernel(&ctx->fill_kernel, ctx, 1, strs, nullptr, "ga_fill", 6, types, 0,
                               nullptr)) != GA_NO_ERROR)
        return err;
    }
    const uintptr_t da = (uintptr_t)b->devptr + dstoff;
    size_t head = (16 - da % 16) % 16;
    if (head > n) head = n;
    size_t nchunks = (n - head) / 16;
    const size_t rest = n - nchunks * 16;
    size_t gs = (std::max(nchunks, rest) + 255) / 256, ls = 256;
    unsigned int word = (unsigned int)(data & 0xff) * 0x01010101u;
    void *args[6] = {dst, &dstoff, &head, &nchunks, &n, &word};
    return hip_callkernel(ctx->fill_kernel, 1, &gs, &ls, 0, args);
  }
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

// Options of every kernel compile.  The toolchain's own HIP headers are left
// out (-nogpuinc): the device runtime that kernel text may rely on is
// device_rt.h, put in front of the source below.
const char *const k_rtc_opts[] = {
    // -O3 gave the same kernel times as -O2 on every shape measured (the
    // kernels unroll and inline by their own pragmas and attributes) and took
    // a sixth longer to compile the larger reduction variants
    "-O2",
    "-nogpuinc",
    // a*b+c stays two roundings, as in IEEE host arithmetic
    "-ffp-contract=off",
    // scalar fp32 ops only; no packed fp32 instruction forms
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-value",
};
const char k_isa_name[] = "amdgcn-amd-amdhsa--gfx950";

std::string join_sources(unsigned int count, const char **strs, const size_t *lens) {
  std::string src;
  for (unsigned int i = 0; i < count; i++) {
    size_t l = (lens != nullptr && lens[i] != 0) ? lens[i] : strlen(strs[i]);
    src.append(strs[i], l);
  }
  return src;
}

// Compile to a gfx950 code object through the code-object manager (the
// library hipRTC itself drives): source -> relocatable, with the device
// libraries linked in as bitcode, then relocatable -> executable.  Going there
// directly leaves out the runtime header hipRTC puts in front of every
// program, whose parse alone takes 0.24 s per kernel; an empty kernel compiles
// in 0.035 s this way.  Needs no device.
struct comgr_objects {
  amd_comgr_data_t src = {0}, hdr = {0}, hip_hdr = {0};
  amd_comgr_data_set_t in = {0}, rel = {0}, exe = {0};
  amd_comgr_action_info_t compile = {0}, link = {0};
  ~comgr_objects() {
    if (compile.handle) amd_comgr_destroy_action_info(compile);
    if (link.handle) amd_comgr_destroy_action_info(link);
    if (in.handle) amd_comgr_destroy_data_set(in);
    if (rel.handle) amd_comgr_destroy_data_set(rel);
    if (exe.handle) amd_comgr_destroy_data_set(exe);
    if (src.handle) amd_comgr_release_data(src);
    if (hdr.handle) amd_comgr_release_data(hdr);
    if (hip_hdr.handle) amd_comgr_release_data(hip_hdr);
  }
};

void comgr_take_log(amd_comgr_data_set_t set, std::string &log) {
  size_t n = 0;
  if (amd_comgr_action_data_count(set, AMD_COMGR_DATA_KIND_LOG, &n) != AMD_COMGR_STATUS_SUCCESS) return;
  for (size_t i = 0; i < n; i++) {
    amd_comgr_data_t d;
    if (amd_comgr_action_data_get_data(set, AMD_COMGR_DATA_KIND_LOG, i, &d) != AMD_COMGR_STATUS_SUCCESS)
      continue;
    size_t sz = 0;
    if (amd_comgr_get_data(d, &sz, nullptr) == AMD_COMGR_STATUS_SUCCESS && sz > 0) {
      std::string part(sz, '\0');
      if (amd_comgr_get_data(d, &sz, &part[0]) == AMD_COMGR_STATUS_SUCCESS) log += part;
    }
    amd_comgr_release_data(d);
  }
  while (!log.empty() && log.back() == '\0') log.pop_back();
}

int rtc_compile(const std::string &src, std::vector<char> &code, std::string &log) {
  // the in-process compiler keeps global option state: one compile at a time
  static std::mutex compiler_lock;
  std::lock_guard<std::mutex> guard(compiler_lock);
  std::string text = ga_device_rt_src;
  text += "\n#line 1 \"ga_kernel.hip\"\n";
  text += src;
  comgr_objects o;
  const char *what = nullptr;
  amd_comgr_status_t st;
#define COMGR_TRY(call)                                   \
  if ((st = (call)) != AMD_COMGR_STATUS_SUCCESS) {        \
    what = #call;                                         \
    break;                                                \
  }
  do {
    COMGR_TRY(amd_comgr_create_data(AMD_COMGR_DATA_KIND_SOURCE, &o.src));
    COMGR_TRY(amd_comgr_set_data(o.src, text.size(), text.data()));
    COMGR_TRY(amd_comgr_set_data_name(o.src, "ga_kernel.hip"));
    COMGR_TRY(amd_comgr_create_data(AMD_COMGR_DATA_KIND_INCLUDE, &o.hdr));
    COMGR_TRY(amd_comgr_set_data(o.hdr, strlen(ga_cluda_hip_src), ga_cluda_hip_src));
    COMGR_TRY(amd_comgr_set_data_name(o.hdr, "cluda.h"));
    // kernel text written for hipcc may include the runtime header: what it
    // would use of it is already there
    static const char k_empty_header[] = "#pragma once\n";
    COMGR_TRY(amd_comgr_create_data(AMD_COMGR_DATA_KIND_INCLUDE, &o.hip_hdr));
    COMGR_TRY(amd_comgr_set_data(o.hip_hdr, sizeof(k_empty_header) - 1, k_empty_header));
    COMGR_TRY(amd_comgr_set_data_name(o.hip_hdr, "hip/hip_runtime.h"));
    COMGR_TRY(amd_comgr_create_data_set(&o.in));
    COMGR_TRY(amd_comgr_create_data_set(&o.rel));
    COMGR_TRY(amd_comgr_create_data_set(&o.exe));
    COMGR_TRY(amd_comgr_data_set_add(o.in, o.src));
    COMGR_TRY(amd_comgr_data_set_add(o.in, o.hdr));
    COMGR_TRY(amd_comgr_data_set_add(o.in, o.hip_hdr));
    COMGR_TRY(amd_comgr_create_action_info(&o.compile));
    COMGR_TRY(amd_comgr_action_info_set_language(o.compile, AMD_COMGR_LANGUAGE_HIP));
    COMGR_TRY(amd_comgr_action_info_set_isa_name(o.compile, k_isa_name));
    COMGR_TRY(amd_comgr_action_info_set_logging(o.compile, true));
    COMGR_TRY(amd_comgr_action_info_set_option_list(o.compile, (const char **)k_rtc_opts,
                                                    sizeof(k_rtc_opts) / sizeof(k_rtc_opts[0])));
    st = amd_comgr_do_action(AMD_COMGR_ACTION_COMPILE_SOURCE_TO_RELOCATABLE, o.compile, o.in, o.rel);
    comgr_take_log(o.rel, log);
    if (st != AMD_COMGR_STATUS_SUCCESS) {
      what = "compile";
      break;
    }
    COMGR_TRY(amd_comgr_create_action_info(&o.link));
    COMGR_TRY(amd_comgr_action_info_set_isa_name(o.link, k_isa_name));
    COMGR_TRY(amd_comgr_action_info_set_logging(o.link, true));
    st = amd_comgr_do_action(AMD_COMGR_ACTION_LINK_RELOCATABLE_TO_EXECUTABLE, o.link, o.rel, o.exe);
    if (st != AMD_COMGR_STATUS_SUCCESS) {
      comgr_take_log(o.exe, log);
      what = "link";
      break;
    }
    amd_comgr_data_t out;
    COMGR_TRY(amd_comgr_action_data_get_data(o.exe, AMD_COMGR_DATA_KIND_EXECUTABLE, 0, &out));
    size_t sz = 0;
    st = amd_comgr_get_data(out, &sz, nullptr);
    if (st == AMD_COMGR_STATUS_SUCCESS) {
      code.resize(sz);
      st = amd_comgr_get_data(out, &sz, code.data());
    }
    amd_comgr_release_data(out);
    if (st != AMD_COMGR_STATUS_SUCCESS) what = "reading the code object";
  } while (false);
#undef COMGR_TRY
  if (what != nullptr) {
    const char *msg = nullptr;
    if (amd_comgr_status_string(st, &msg) != AMD_COMGR_STATUS_SUCCESS || msg == nullptr) msg = "error";
    if (log.empty()) log = std::string("code object manager: ") + what + ": " + msg;
    code.clear();
    return GA_IMPL_ERROR;
  }
  return GA_NO_ERROR;
}

// The same through hipRTC, with the toolchain's HIP headers in front of the
// text instead of device_rt.h.  Kernel text handed to GpuKernel_init may be
// written against those headers (hip_fp16.h types, __shfl and __ballot,
// float4 / make_float4, printf, clock64, cooperative groups); the contract is
// "any source the backend's compiler accepts" (reference
// src/gpuarray/kernel.h:54-70, whose CUDA backend compiles with NVRTC and its
// full device vocabulary).  Used only as a second try for text that fails
// against device_rt.h on something a header would supply: it costs the
// quarter of a second per kernel that the first path is there to save.
// libhiprtc is loaded when the first such kernel arrives.
struct hiprtc_api {
  void *lib = nullptr;
  int (*create)(void **, const char *, const char *, int, const char *const *, const char *const *) = nullptr;
  int (*compile)(void *, int, const char *const *) = nullptr;
  int (*log_size)(void *, size_t *) = nullptr;
  int (*get_log)(void *, char *) = nullptr;
  int (*code_size)(void *, size_t *) = nullptr;
  int (*get_code)(void *, char *) = nullptr;
  int (*destroy)(void **) = nullptr;
  bool ok = false;
};

const hiprtc_api &hiprtc() {
  static const hiprtc_api api = [] {
    hiprtc_api a;
    for (const char *name : {"libhiprtc.so", "libhiprtc.so.7"}) {
      a.lib = dlopen(name, RTLD_NOW | RTLD_LOCAL);
      if (a.lib != nullptr) break;
    }
    if (a.lib == nullptr) return a;
    a.create = (decltype(a.create))dlsym(a.lib, "hiprtcCreateProgram");
    a.compile = (decltype(a.compile))dlsym(a.lib, "hiprtcCompileProgram");
    a.log_size = (decltype(a.log_size))dlsym(a.lib, "hiprtcGetProgramLogSize");
    a.get_log = (decltype(a.get_log))dlsym(a.lib, "hiprtcGetProgramLog");
    a.code_size = (decltype(a.code_size))dlsym(a.lib, "hiprtcGetCodeSize");
    a.get_code = (decltype(a.get_code))dlsym(a.lib, "hiprtcGetCode");
    a.destroy = (decltype(a.destroy))dlsym(a.lib, "hiprtcDestroyProgram");
    a.ok = a.create && a.compile && a.log_size && a.get_log && a.code_size && a.get_code && a.destroy;
    return a;
  }();
  return api;
}

// Does a failed compile against device_rt.h look like text that wants the
// toolchain's headers (rather than text that is simply wrong)?
bool wants_toolchain_headers(const std::string &log) {
  for (const char *sign : {"file not found", "undeclared identifier", "unknown type name",
                           "no matching function", "no member named", "use of undeclared"})
    if (log.find(sign) != std::string::npos) return true;
  return false;
}

int hiprtc_compile(const std::string &src, std::vector<char> &code, std::string &log) {
  const hiprtc_api &rt = hiprtc();
  if (!rt.ok) {
    log += "\n(libhiprtc could not be loaded for a second try with the toolchain's headers)";
    return GA_IMPL_ERROR;
  }
  static std::mutex compiler_lock;
  std::lock_guard<std::mutex> guard(compiler_lock);
  void *prog = nullptr;
  const char *headers[1] = {ga_cluda_hip_src};
  const char *names[1] = {"cluda.h"};
  if (rt.create(&prog, src.c_str(), "ga_kernel.hip", 1, headers, names) != 0) return GA_IMPL_ERROR;
  // headers beyond the ones hipRTC carries inside itself come from the installation
  const char *root = getenv("ROCM_PATH");
  const std::string inc = std::string("-I") + ((root && *root) ? root : "/opt/rocm") + "/include";
  const char *const opts[] = {"--offload-arch=gfx950", "-O2", "-ffp-contract=off",
                              "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                              "-Wno-unused-value", inc.c_str()};
  const int rc = rt.compile(prog, (int)(sizeof(opts) / sizeof(opts[0])), opts);
  size_t n = 0;
  std::string second;
  if (rt.log_size(prog, &n) == 0 && n > 1) {
    second.resize(n);
    if (rt.get_log(prog, &second[0]) != 0) second.clear();
    while (!second.empty() && second.back() == '\0') second.pop_back();
  }
  int err = GA_IMPL_ERROR;
  if (rc == 0 && rt.code_size(prog, &n) == 0 && n > 0) {
    code.resize(n);
    if (rt.get_code(prog, code.data()) == 0) err = GA_NO_ERROR;
  }
  if (err != GA_NO_ERROR) {
    code.clear();
    log += "\n--- second try, with the toolchain's HIP headers (hipRTC) ---\n" + second;
  }
  rt.destroy(&prog);
  return err;
}

// Compile kernel text: against device_rt.h first; text that fails there on
// something the toolchain's headers would supply gets one more try through hipRTC.
int compile_kernel_text(const std::string &src, std::vector<char> &code, std::string &log) {
  int err = rtc_compile(src, code, log);
  if (err != GA_NO_ERROR && wants_toolchain_headers(log)) err = hiprtc_compile(src, code, log);
#ifdef DEBUG
  // (the reference's DEBUG builds print the compiler's log, src/gpuarray_elemwise.c:682-690)
  if (err != GA_NO_ERROR) fprintf(stderr, "%s\n", log.c_str());
#endif
  return err;
}

// ---- on-disk cache of compiled kernels ------------------------------------------
// A compile costs 0.3-0.5 s; a process that builds a few hundred operators
// spends minutes in the compiler.  With a cache directory (property
// kernel_cache_path or environment GPUARRAY_CACHE_PATH, the reference's
// names: src/gpuarray_buffer_cuda.c:301-331) code objects are kept across
// processes.  Layout follows the reference's disk cache (src/cache/disk.c:
// 214-289): the key is {format tag, compiler version, ISA, options, source},
// the file name is the hex of a hash of the key under a two-level directory,
// the file holds 8-byte big-endian key and value lengths, then key, then
// value, and is written under a temporary name and renamed.  The stored key
// is compared in full on load, so a hash collision is a miss, not a wrong
// kernel; a checksum of the value follows it, so a damaged file is a miss too
// and is never handed to the loader.
std::string disk_key(const std::string &src, const char *isa) {
  std::string k = "ga-hip-kcache-2|";
  size_t maj = 0, min = 0;
  amd_comgr_get_version(&maj, &min);
  k += std::to_string(maj) + "." + std::to_string(min);
  // the runtime's full version too: a patch release of the compiler must not
  // be served code objects its predecessor made
  int rtv = 0;
  if (hipRuntimeGetVersion(&rtv) == hipSuccess) k += "/" + std::to_string(rtv);
  else (void)hipGetLastError();
  k += "|";
  k += isa;
  for (const char *o : k_rtc_opts) { k += "|"; k += o; }
  k += "|";
  k += ga_device_rt_src;
  k += "|";
  k += ga_cluda_hip_src;
  k += "|";
  k += src;
  return k;
}

void hash128(const std::string &k, uint64_t out[2]) {
  // two independent FNV-1a style streams; only used to name files
  uint64_t a = 0xcbf29ce484222325ull, b = 0x84222325cbf29ce4ull;
  for (unsigned char c : k) {
    a = (a ^ c) * 0x100000001b3ull;
    b = (b ^ (c + 0x9e)) * 0x100000001b5ull;
    b ^= b >> 29;
  }
  out[0] = a;
  out[1] = b;
}

std::string disk_path(const std::string &dir, const std::string &key, bool mkdirs) {
  uint64_t h[2];
  hash128(key, h);
  char name[64];
  snprintf(name, sizeof(name), "%016llx%016llx", (unsigned long long)h[0], (unsigned long long)h[1]);
  std::string sub = dir + "/" + std::string(name, 4);
  if (mkdirs) {
    (void)mkdir(dir.c_str(), 0777);
    (void)mkdir(sub.c_str(), 0777);
  }
  return sub + "/" + (name + 4);
}

void put_be64(unsigned char *p, uint64_t v) {
  for (int i = 7; i >= 0; i--) { p[i] = (unsigned char)(v & 0xff); v >>= 8; }
}
uint64_t get_be64(const unsigned char *p) {
  uint64_t v = 0;
  for (int i = 0; i < 8; i++) v = (v << 8) | p[i];
  return v;
}

uint64_t checksum64(const std::vector<char> &v) {
  uint64_t a = 0xcbf29ce484222325ull;
  for (char c : v) a = (a ^ (unsigned char)c) * 0x100000001b3ull;
  return a;
}

bool disk_load(const std::string &dir, const std::string &key, std::vector<char> &code) {
  FILE *f = fopen(disk_path(dir, key, false).c_str(), "rb");
  if (f == nullptr) return false;
  unsigned char hdr[16];
  bool ok = fread(hdr, 1, 16, f) == 16;
  uint64_t kl = ok ? get_be64(hdr) : 0, vl = ok ? get_be64(hdr + 8) : 0;
  ok = ok && kl == key.size() && vl > 0 && vl < ((uint64_t)1 << 31);
  if (ok) {
    std::string stored(kl, '\0');
    ok = fread(&stored[0], 1, kl, f) == kl && stored == key;
  }
  if (ok) {
    code.resize(vl);
    ok = fread(code.data(), 1, vl, f) == vl;
  }
  unsigned char sum[8];
  ok = ok && fread(sum, 1, 8, f) == 8 && get_be64(sum) == checksum64(code);
  fclose(f);
  return ok;
}

void disk_store(const std::string &dir, const std::string &key, const std::vector<char> &code) {
  std::string path = disk_path(dir, key, true);
  // unique per store: two contexts or threads of one process may store the same key
  static std::atomic<unsigned long> serial{0};
  std::string tmp = path + ".tmp." + std::to_string((long)getpid()) + "." + std::to_string(serial++);
  FILE *f = fopen(tmp.c_str(), "wb");
  if (f == nullptr) return;   // a cache that cannot be written is only slower
  unsigned char hdr[16];
  put_be64(hdr, key.size());
  put_be64(hdr + 8, code.size());
  unsigned char sum[8];
  put_be64(sum, checksum64(code));
  bool ok = fwrite(hdr, 1, 16, f) == 16 && fwrite(key.data(), 1, key.size(), f) == key.size() &&
            fwrite(code.data(), 1, code.size(), f) == code.size() && fwrite(sum, 1, 8, f) == 8;
  ok = fclose(f) == 0 && ok;
  if (!ok || rename(tmp.c_str(), path.c_str()) != 0) (void)unlink(tmp.c_str());
}

// A module is unloaded when the cache has dropped it and no kernel uses it.
void mod_reap(hip_context *ctx, hip_module *m) {
  if (m->cached || m->refcnt != 0) return;
  if (m->mod) (void)hipModuleUnload(m->mod);
  if (ctx->live_modules > 0) ctx->live_modules--;
  delete m;
}

void mod_unref(hip_context *ctx, hip_module *m) {
  if (m->refcnt > 0) m->refcnt--;
  mod_reap(ctx, m);
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
  hip_module *m = ctx->modcache.get(src);
  if (m == nullptr) {
    std::vector<char> code;
    std::string log, dkey;
    bool from_disk = false;
    if (!ctx->disk_cache.empty()) {
      dkey = disk_key(src, ctx->bin_id);
      from_disk = disk_load(ctx->disk_cache, dkey, code);
    }
    if (!from_disk) {
      err = compile_kernel_text(src, code, log);
      if (err != GA_NO_ERROR) {
        if (err_str) *err_str = strdup(log.c_str());
        return ga_err_fmt(ctx->err, GA_IMPL_ERROR, "Kernel compilation failed: %.900s", log.c_str());
      }
      if (!ctx->disk_cache.empty()) disk_store(ctx->disk_cache, dkey, code);
    }
    m = new hip_module();
    hipError_t e = hipModuleLoadData(&m->mod, code.data());
    if (e != hipSuccess && from_disk) {
      // a damaged cache entry: compile afresh and replace it
      (void)hipGetLastError();
      err = compile_kernel_text(src, code, log);
      if (err != GA_NO_ERROR) {
        delete m;
        if (err_str) *err_str = strdup(log.c_str());
        return ga_err_fmt(ctx->err, GA_IMPL_ERROR, "Kernel compilation failed: %.900s", log.c_str());
      }
      disk_store(ctx->disk_cache, dkey, code);
      e = hipModuleLoadData(&m->mod, code.data());
    }
    if (e != hipSuccess) {
      delete m;
      return hip_fail(ctx->err, "hipModuleLoadData", e);
    }
    m->key = src;
    ctx->live_modules++;
    m->refcnt++;   // keeps it alive across the eviction pass below
    std::vector<hip_module *> evicted;
    ctx->modcache.add(m, evicted);
    m->refcnt--;
    for (hip_module *old : evicted) mod_reap(ctx, old);
  }

  hipFunction_t fn = nullptr;
  hipError_t e = hipModuleGetFunction(&fn, m->mod, fname);
  if (e != hipSuccess) {
    mod_reap(ctx, m);
    return ga_err_fmt(ctx->err, GA_IMPL_ERROR, "Kernel entry point \"%s\" not found: %s", fname,
                      hipGetErrorString(e));
  }

  hip_kernel *k = (hip_kernel *)calloc(1, sizeof(hip_kernel));
  if (k == nullptr) return ga_err_sys(ctx->err, "calloc");
  TAG_KER(k);
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
  {
    uint64_t h = 1469598103934665603ull;
    for (unsigned char ch : m->key) h = (h ^ ch) * 1099511628211ull;
    for (const char *c = fname; *c; c++) h = (h ^ (unsigned char)*c) * 1099511628211ull;
    k->text_hash = h;
  }
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
  CLEAR_TAG(k);
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
  ctx->last_launch_hash = k->text_hash;
  // Timed launches (the hip_kernel_timing hook): the dispatch itself carries
  // a start and a stop event, so their distance is the kernel's own duration,
  // without the gap between a mark on the stream and the kernel's start.
  if (ctx->ktime_on && (uint64_t)g[0] * l[0] <= 0xffffffffull && (uint64_t)g[1] * l[1] <= 0xffffffffull &&
      (uint64_t)g[2] * l[2] <= 0xffffffffull) {
    while (ctx->ktime_ev.size() < 2 * (ctx->ktime_n + 1)) {
      hipEvent_t e = nullptr;
      HIP_TRY(ctx, hipEventCreate(&e));
      ctx->ktime_ev.push_back(e);
    }
    HIP_TRY(ctx, hipExtModuleLaunchKernel(k->fn, g[0] * l[0], g[1] * l[1], g[2] * l[2], l[0], l[1], l[2],
                                          shared, ctx->stream, params, nullptr,
                                          ctx->ktime_ev[2 * ctx->ktime_n],
                                          ctx->ktime_ev[2 * ctx->ktime_n + 1], 0));
    if (ctx->ktime_hash.size() <= ctx->ktime_n) ctx->ktime_hash.resize(ctx->ktime_n + 1);
    ctx->ktime_hash[ctx->ktime_n] = k->text_hash;
    ctx->ktime_n++;
    return GA_NO_ERROR;
  }
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
    if (prop_id == GA_CTX_PROP_TOTAL_GMEM) {
      *(size_t *)res = tot;
    } else if (prop_id == GA_CTX_PROP_FREE_GMEM) {
      // what the driver still has plus what the cache can hand out again
      size_t cached = 0;
      for (const auto &kv : ctx->mem.free_by_size) cached += kv.first;
      *(size_t *)res = fr + cached;
    } else {
      // the reference guesses a quarter of the driver's free memory, or the
      // largest cached block if that is bigger (src/gpuarray_buffer_cuda.c:621-635)
      size_t guess = fr / 4, big = ctx->mem.largest_free();
      *(size_t *)res = big > guess ? big : guess;
    }
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
  TAG_BUF(b);
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
  int err = compile_kernel_text(join_sources(count, strs, lens), code, l);
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
extern "C" char *ga_take1_gen_source(int chunks, int a_tc, int v_tc, int i_tc, unsigned int tnd);
extern "C" char *ga_mapreduce_gen_source(int op, const char *reduce_expr, const char *neutral,
                                         int acc_tc, const char *preamble, const char *map_expr,
                                         unsigned int n, const gpuelemwise_arg *args, int d0_tc,
                                         unsigned int G, unsigned int V, unsigned int U,
                                         unsigned int vecmask);
namespace {

// Numbered timing marks on the context's stream: record as many as wanted
// without waiting, read the spans afterwards.  A mark orders nothing for the
// host (ext_event_elapsed waits for the later mark itself), so its event is
// made without the system-scope fence a default event carries: with that
// fence every mark has the device write its caches back for the host to see,
// which put 1.5 us between two marks around one kernel (2^24-element flat
// kernel: 34.96 us between default events, 33.45 between these, 32.4 for the
// kernel's own dispatch).  GPUARRAY_MARK_EVENT_FLAGS overrides the flags.
int ext_event_record(gpucontext *c, unsigned int slot) {
  hip_context *ctx = HC(c);
  int err;
  if ((err = enter(ctx)) != GA_NO_ERROR) return err;
  while (ctx->evpool.size() <= slot) {
    hipEvent_t e = nullptr;
    HIP_TRY(ctx, hipEventCreateWithFlags(&e, (unsigned)TUNE(&ctx->tuning, MARK_EVENT_FLAGS, hipEventDisableSystemFence)));
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

// Per-launch timing.  on != 0: forget earlier records and give every launch
// from now on its own pair of events; on == 0: back to plain launches (the
// records stay readable).
int ext_kernel_timing(gpucontext *c, int on) {
  hip_context *ctx = HC(c);
  if (on) ctx->ktime_n = 0;
  ctx->ktime_on = on != 0;
  return GA_NO_ERROR;
}

// Durations in milliseconds of the launches recorded since timing was turned
// on, in launch order, into out[0..max); waits for the last of them.  Returns
// how many were recorded, < 0 on error.
int ext_kernel_times(gpucontext *c, float *out, unsigned int max) {
  hip_context *ctx = HC(c);
  if (enter(ctx) != GA_NO_ERROR) return -1;
  const size_t n = ctx->ktime_n;
  if (n > 0 && hipEventSynchronize(ctx->ktime_ev[2 * n - 1]) != hipSuccess) return -1;
  for (size_t i = 0; i < n && i < max; i++)
    if (hipEventElapsedTime(&out[i], ctx->ktime_ev[2 * i], ctx->ktime_ev[2 * i + 1]) != hipSuccess)
      return -1;
  return (int)n;
}

// The text hashes (see ext_last_launch_hash) of the launches recorded since
// timing was turned on, in launch order, into out[0..max).  Returns how many
// were recorded.
int ext_kernel_hashes(gpucontext *c, unsigned long long *out, unsigned int max) {
  hip_context *ctx = HC(c);
  const size_t n = ctx->ktime_n;
  for (size_t i = 0; i < n && i < max; i++) out[i] = ctx->ktime_hash[i];
  return (int)n;
}

// Identifies the text of the kernel the context launched last: a 64-bit hash
// of its source followed by its entry point's name.  Lets a measurement say
// which generated kernel it belongs to.
uint64_t ext_last_launch_hash(gpucontext *c) { return HC(c)->last_launch_hash; }

// Entries in the hot, warm and cold lists of the module cache, and the number
// of code objects currently loaded (cached or kept alive by a kernel).
int ext_module_cache_stats(gpucontext *c, size_t out[4]) {
  hip_context *ctx = HC(c);
  ctx->modcache.counts(out);
  out[3] = ctx->live_modules;
  return GA_NO_ERROR;
}

int ext_reload_tuning(gpucontext *c) {
  ga_tuning_read(&HC(c)->tuning);
  return GA_NO_ERROR;
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
    {"hip_kernel_timing", (void *)ext_kernel_timing},
    {"hip_kernel_times", (void *)ext_kernel_times},
    {"hip_kernel_hashes", (void *)ext_kernel_hashes},
    {"hip_last_launch_hash", (void *)ext_last_launch_hash},
    {"hip_elemwise_source", (void *)ga_elemwise_gen_source},
    {"hip_reduction_source", (void *)ga_reduction_gen_source},
    {"hip_mapreduce_source", (void *)ga_mapreduce_gen_source},
    {"hip_module_cache_stats", (void *)ext_module_cache_stats},
    {"hip_take1_source", (void *)ga_take1_gen_source},
    {"hip_reload_tuning", (void *)ext_reload_tuning},
};

}  // namespace

extern "C" void *gpuarray_get_extension(const char *name) {
  if (name == nullptr) return nullptr;
  for (const auto &e : k_exts)
    if (strcmp(e.name, name) == 0) return e.fn;
  return nullptr;
}

// A scratch buffer that is outgrown is kept until the context goes: launches
// already recorded into a HIP graph hold its address, and a block given back
// to the memory cache would be handed to the caller's next array while every
// replay of that graph still writes partials into it.  Sizes double, so the
// buffers kept this way add up to less than the one in use.
gpudata *ga_hip_scratch(gpucontext *c, size_t bytes) {
  hip_context *ctx = HC(c);
  if (ctx->scratch != nullptr && ctx->scratch_sz >= bytes) return ctx->scratch;
  size_t want = ctx->scratch_sz ? ctx->scratch_sz * 2 : ((size_t)1 << 20);
  while (want < bytes) want *= 2;
  gpudata *grown = hip_alloc(c, want, nullptr, BUF_INTERNAL);
  if (grown == nullptr && want > bytes) grown = hip_alloc(c, want = bytes, nullptr, BUF_INTERNAL);
  if (grown == nullptr) return nullptr;
  if (ctx->scratch != nullptr) ctx->retired_scratch.push_back(ctx->scratch);
  ctx->scratch = grown;
  ctx->scratch_sz = want;
  return ctx->scratch;
}

gpudata *ga_hip_static_scratch_buf(gpucontext *c, const char **why) {
  hip_context *ctx = HC(c);
  if (why != nullptr)
    *why = ctx->static_scratch != nullptr ? (ctx->static_buf ? "" : "out of host memory")
                                          : hipGetErrorString((hipError_t)ctx->static_scratch_err);
  return ctx->static_buf;
}

void *ga_hip_static_scratch(gpucontext *c, const char **why) {
  hip_context *ctx = HC(c);
  if (why != nullptr)
    *why = ctx->static_scratch != nullptr ? "" : hipGetErrorString((hipError_t)ctx->static_scratch_err);
  return ctx->static_scratch;
}

// Is the context's stream recording a graph?  Work recorded now runs again at
// every replay, on the addresses it was recorded with.
bool ga_hip_capturing(gpucontext *c) {
  hip_context *ctx = HC(c);
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(ctx->stream, &cap) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return cap != hipStreamCaptureStatusNone;
}

bool ga_hip_redux_counters_made(gpucontext *c) { return HC(c)->redux_counters != nullptr; }

gpudata *ga_hip_redux_counters(gpucontext *c) {
  hip_context *ctx = HC(c);
  if (ctx->redux_counters != nullptr) return ctx->redux_counters;
  // Not while the stream records a graph: the memset that zeroes the counters
  // would be recorded instead of run.  The caller then takes two launches.
  if (ga_hip_capturing(c)) return nullptr;
  gpudata *b = hip_alloc(c, ga_hip_redux_counters_max * sizeof(uint32_t), nullptr, BUF_INTERNAL);
  if (b == nullptr) return nullptr;
  if (hip_memset(b, 0, 0) != GA_NO_ERROR) {
    hip_release(b);
    return nullptr;
  }
  ctx->redux_counters = b;
  return b;
}

// Bytes from the start of a buffer that a kernel may read without leaving the
// memory behind it: the cache block for the library's own allocations (a
// multiple of 256), the stated size for memory wrapped by hip_make_buf.
size_t ga_hip_readable_bytes(gpudata *b) {
  hip_data *d = HD(b);
  if (d->block != nullptr) return d->block->size;
  if (!(d->flags & BUF_OWNED)) return d->sz;     // caller's memory
  return (d->sz + 15) & ~(size_t)15;             // straight from the driver
}

void ga_hip_buf_info(gpudata *b, uintptr_t *devptr, size_t *size, size_t *readable) {
  hip_data *d = HD(b);
  *devptr = (uintptr_t)d->devptr;
  *size = d->sz;
  *readable = d->block != nullptr ? d->block->size : !(d->flags & BUF_OWNED) ? d->sz : ((d->sz + 15) & ~(size_t)15);
}

unsigned int ga_hip_numprocs(gpucontext *c) { return HC(c)->numprocs; }
const ga_tuning *ga_hip_tuning(gpucontext *c) { return c ? &HC(c)->tuning : ga_tuning_default(); }

const ga_tuning *ga_tuning_default() {
  static const ga_tuning t = [] { ga_tuning r; ga_tuning_read(&r); return r; }();
  return &t;
}

void ga_tuning_read(ga_tuning *t) {
  static std::atomic<unsigned long> generations{0};
  t->generation = ++generations;
  static const char *const names[GA_NKNOBS] = {
#define X(name) "GPUARRAY_" #name,
      GA_KNOBS(X)
#undef X
  };
  for (unsigned k = 0; k < GA_NKNOBS; k++) {
    const char *v = getenv(names[k]);
    char *end = nullptr;
    t->set[k] = false;
    t->val[k] = 0;
    if (v == nullptr || *v == 0) continue;
    const unsigned long r = strtoul(v, &end, 10);
    if (end == v) continue;   // not a number: as if unset
    t->set[k] = true;
    t->val[k] = r;
  }
  const char *fam = getenv("GPUARRAY_REDUX_FAMILY");
  snprintf(t->redux_family, sizeof(t->redux_family), "%s", fam ? fam : "");
}
void **ga_hip_redux_cache_slot(gpucontext *c) { return &HC(c)->redux_cache; }
void **ga_hip_take1_cache_slot(gpucontext *c) { return &HC(c)->take1_cache; }

const ga_buffer_ops ga_hip_ops = {
    hip_get_platform_count, hip_get_device_count, hip_init,        hip_deinit,
    hip_alloc,              hip_retain,           hip_release,     hip_share,
    hip_move,               hip_read,             hip_write,       hip_memset,
    hip_newkernel,          hip_retainkernel,     hip_freekernel,  hip_setarg,
    hip_callkernel,         hip_sync,             hip_transfer,    hip_property,
    hip_error};
