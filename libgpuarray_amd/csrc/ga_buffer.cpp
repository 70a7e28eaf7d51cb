// Backend-neutral entry points: name -> backend table, context properties,
// and the thin gpudata_*/gpukernel_* forwards.
// Behaviour follows the reference's src/gpuarray_buffer.c:15-269.
#include "private.hpp"

const ga_buffer_ops *gpuarray_get_ops(const char *name) {
  if (name != nullptr && strcmp(name, "hip") == 0) return &ga_hip_ops;
  return nullptr;
}

static const ga_buffer_ops *ops_or_err(const char *name) {
  const ga_buffer_ops *ops = gpuarray_get_ops(name);
  if (ops == nullptr)
    ga_err_fmt(ga_global_err, GA_INVALID_ERROR,
               "Invalid platform \"%s\": this library only has the \"hip\" backend",
               name ? name : "(null)");
  return ops;
}

extern "C" {

int gpu_get_platform_count(const char *name, unsigned int *platcount) {
  const ga_buffer_ops *ops = ops_or_err(name);
  if (ops == nullptr) return GA_INVALID_ERROR;
  return ops->get_platform_count(platcount);
}

int gpu_get_device_count(const char *name, unsigned int platform,
                         unsigned int *devcount) {
  const ga_buffer_ops *ops = ops_or_err(name);
  if (ops == nullptr) return GA_INVALID_ERROR;
  return ops->get_device_count(platform, devcount);
}

int gpucontext_props_new(gpucontext_props **res) {
  gpucontext_props *p = (gpucontext_props *)calloc(1, sizeof(*p));
  if (p == nullptr) return ga_err_sys(ga_global_err, "calloc");
  p->dev = -1;
  p->sched = GA_CTX_SCHED_AUTO;
  p->max_cache_size = (size_t)-1;
  *res = p;
  return GA_NO_ERROR;
}

int gpucontext_props_hip_dev(gpucontext_props *p, int devno) {
  p->dev = devno;
  return GA_NO_ERROR;
}

int gpucontext_props_cuda_dev(gpucontext_props *p, int devno) {
  p->dev = devno;
  return GA_NO_ERROR;
}

int gpucontext_props_opencl_dev(gpucontext_props *p, int platno, int devno) {
  p->dev = (platno << 16) | devno;
  return GA_NO_ERROR;
}

int gpucontext_props_sched(gpucontext_props *p, int sched) {
  if (sched != GA_CTX_SCHED_AUTO && sched != GA_CTX_SCHED_SINGLE &&
      sched != GA_CTX_SCHED_MULTI)
    return ga_err_fmt(ga_global_err, GA_INVALID_ERROR,
                      "Invalid value for sched: %d", sched);
  p->sched = sched;
  if (sched == GA_CTX_SCHED_MULTI)
    p->flags |= GA_CTX_MULTI_THREAD;
  else
    p->flags &= ~GA_CTX_MULTI_THREAD;
  return GA_NO_ERROR;
}

int gpucontext_props_set_single_stream(gpucontext_props *p) {
  p->flags |= GA_CTX_SINGLE_STREAM;
  return GA_NO_ERROR;
}

int gpucontext_props_kernel_cache(gpucontext_props *p, const char *path) {
  p->kernel_cache_path = path;
  return GA_NO_ERROR;
}

int gpucontext_props_alloc_cache(gpucontext_props *p, size_t initial,
                                 size_t max) {
  if (initial > max)
    return ga_err_set(ga_global_err, GA_VALUE_ERROR,
                      "Initial size can't be bigger than max size");
  p->initial_cache_size = initial;
  p->max_cache_size = max;
  return GA_NO_ERROR;
}

void gpucontext_props_del(gpucontext_props *p) { free(p); }

int gpucontext_init(gpucontext **res, const char *name, gpucontext_props *p) {
  const ga_buffer_ops *ops = ops_or_err(name);
  if (ops == nullptr) {
    gpucontext_props_del(p);
    return ga_global_err->code;
  }
  if (p == nullptr && gpucontext_props_new(&p) != GA_NO_ERROR)
    return ga_global_err->code;
  gpucontext *ctx = ops->buffer_init(p);
  gpucontext_props_del(p);
  if (ctx == nullptr) return ga_global_err->code;
  ctx->ops = ops;
  ctx->extcopy_cache = nullptr;
  *res = ctx;
  return GA_NO_ERROR;
}

void gpucontext_deref(gpucontext *ctx) {
  if (ctx == nullptr) return;
  ctx->ops->buffer_deinit(ctx);
}

int gpucontext_property(gpucontext *ctx, int prop_id, void *res) {
  return ctx->ops->property(ctx, nullptr, nullptr, prop_id, res);
}

const char *gpucontext_error(gpucontext *ctx, int err) {
  (void)err;
  if (ctx == nullptr) return ga_global_err->msg;
  return ctx->ops->ctx_error(ctx);
}

gpudata *gpudata_alloc(gpucontext *ctx, size_t sz, void *data, int flags,
                       int *ret) {
  gpudata *b = ctx->ops->buffer_alloc(ctx, sz, data, flags);
  if (b == nullptr && ret) *ret = ctx->err->code;
  return b;
}

void gpudata_retain(gpudata *b) { b->ctx->ops->buffer_retain(b); }

void gpudata_release(gpudata *b) {
  if (b) b->ctx->ops->buffer_release(b);
}

int gpudata_share(gpudata *a, gpudata *b, int *ret) {
  int r = a->ctx->ops->buffer_share(a, b);
  if (r == -1 && ret) *ret = a->ctx->err->code;
  return r;
}

int gpudata_move(gpudata *dst, size_t dstoff, gpudata *src, size_t srcoff,
                 size_t sz) {
  return src->ctx->ops->buffer_move(dst, dstoff, src, srcoff, sz);
}

// Same context: device copy.  Same backend, other context: peer copy, and if
// that is refused, bounce through host memory (reference
// src/gpuarray_buffer.c:172-202).
int gpudata_transfer(gpudata *dst, size_t dstoff, gpudata *src, size_t srcoff,
                     size_t sz) {
  gpucontext *sc = src->ctx, *dc = dst->ctx;
  if (sc == dc) return sc->ops->buffer_move(dst, dstoff, src, srcoff, sz);
  if (sc->ops == dc->ops &&
      sc->ops->buffer_transfer(dst, dstoff, src, srcoff, sz) == GA_NO_ERROR)
    return GA_NO_ERROR;
  void *tmp = malloc(sz ? sz : 1);
  if (tmp == nullptr) {
    ga_err_sys(sc->err, "malloc");
    return ga_err_sys(dc->err, "malloc");
  }
  int err = sc->ops->buffer_read(tmp, src, srcoff, sz);
  if (err == GA_NO_ERROR) err = dc->ops->buffer_write(dst, dstoff, tmp, sz);
  free(tmp);
  return err;
}

int gpudata_read(void *dst, gpudata *src, size_t srcoff, size_t sz) {
  return src->ctx->ops->buffer_read(dst, src, srcoff, sz);
}

int gpudata_write(gpudata *dst, size_t dstoff, const void *src, size_t sz) {
  return dst->ctx->ops->buffer_write(dst, dstoff, src, sz);
}

int gpudata_memset(gpudata *dst, size_t dstoff, int data) {
  return dst->ctx->ops->buffer_memset(dst, dstoff, data);
}

int gpudata_sync(gpudata *b) { return b->ctx->ops->buffer_sync(b); }

int gpudata_property(gpudata *b, int prop_id, void *res) {
  return b->ctx->ops->property(nullptr, b, nullptr, prop_id, res);
}

gpucontext *gpudata_context(gpudata *b) { return b->ctx; }

gpukernel *gpukernel_init(gpucontext *ctx, unsigned int count,
                          const char **strings, const size_t *lengths,
                          const char *fname, unsigned int numargs,
                          const int *typecodes, int flags, int *ret,
                          char **err_str) {
  gpukernel *k = nullptr;
  int err = ctx->ops->kernel_alloc(&k, ctx, count, strings, lengths, fname,
                                   numargs, typecodes, flags, err_str);
  if (err != GA_NO_ERROR && ret) *ret = ctx->err->code;
  return k;
}

void gpukernel_retain(gpukernel *k) { k->ctx->ops->kernel_retain(k); }
void gpukernel_release(gpukernel *k) {
  if (k) k->ctx->ops->kernel_release(k);
}
int gpukernel_setarg(gpukernel *k, unsigned int i, void *a) {
  return k->ctx->ops->kernel_setarg(k, i, a);
}
int gpukernel_call(gpukernel *k, unsigned int n, const size_t *gs,
                   const size_t *ls, size_t shared, void **args) {
  return k->ctx->ops->kernel_call(k, n, gs, ls, shared, args);
}
int gpukernel_property(gpukernel *k, int prop_id, void *res) {
  return k->ctx->ops->property(nullptr, nullptr, k, prop_id, res);
}
gpucontext *gpukernel_context(gpukernel *k) { return k->ctx; }

}  // extern "C"
