// GpuKernel: argument table + launch geometry for 256 compute units.
// Entry points follow the reference's src/gpuarray_kernel.c:10-103.
#include "private.hpp"

extern "C" {

int GpuKernel_init(GpuKernel *k, gpucontext *ctx, unsigned int count, const char **strs,
                   const size_t *lens, const char *name, unsigned int argcount,
                   const int *types, int flags, char **err_str) {
  int res = GA_NO_ERROR;
  k->k = nullptr;
  k->args = (void **)calloc(argcount ? argcount : 1, sizeof(void *));
  if (k->args == nullptr) return ga_err_sys(ctx->err, "calloc");
  k->k = gpukernel_init(ctx, count, strs, lens, name, argcount, types, flags, &res, err_str);
  if (k->k == nullptr && res == GA_NO_ERROR) res = ctx->err->code;
  if (res != GA_NO_ERROR) GpuKernel_clear(k);
  return res;
}

void GpuKernel_clear(GpuKernel *k) {
  if (k->k) gpukernel_release(k->k);
  free(k->args);
  k->k = nullptr;
  k->args = nullptr;
}

gpucontext *GpuKernel_context(GpuKernel *k) { return gpukernel_context(k->k); }

// 1-D geometry.  The reference (src/gpuarray_kernel.c:38-89) starts from one
// preferred-size group, caps the grid at 32 groups per processor and then
// grows the group up to 512 lanes.  Here a group is 256 lanes (4 wavefronts,
// one per SIMD of a compute unit) whenever n reaches that, smaller counts
// round up to whole wavefronts, and the grid is capped at 16 groups per
// compute unit: with 256 CUs that is 4096 groups, more than ten rounds of
// the chip, which is what a grid-stride loop needs to keep all eight XCDs
// streaming.  Caller-fixed values are kept as given.
int GpuKernel_sched(GpuKernel *k, size_t n, size_t *gs, size_t *ls) {
  size_t max_l, pref_l, max_g;
  unsigned int numprocs;
  int err;
  if ((err = gpukernel_property(k->k, GA_KERNEL_PROP_MAXLSIZE, &max_l)) != GA_NO_ERROR) return err;
  if ((err = gpukernel_property(k->k, GA_KERNEL_PROP_PREFLSIZE, &pref_l)) != GA_NO_ERROR) return err;
  if ((err = gpukernel_property(k->k, GA_CTX_PROP_NUMPROCS, &numprocs)) != GA_NO_ERROR) return err;
  if ((err = gpukernel_property(k->k, GA_CTX_PROP_MAXGSIZE0, &max_g)) != GA_NO_ERROR) return err;

  if (n == 0) n = 1;
  if (*ls == 0) {
    size_t want = 256;
    if (want > max_l) want = (max_l / pref_l) * pref_l;
    if (want == 0) want = max_l;
    if (n < want) want = ((n + pref_l - 1) / pref_l) * pref_l;
    if (want > max_l) want = max_l;
    *ls = want;
  }
  if (*gs == 0) {
    size_t cap = (size_t)numprocs * 16;
    if (cap > max_g) cap = max_g;
    size_t g = (n - 1) / *ls + 1;
    *gs = g > cap ? cap : g;
  }
  return GA_NO_ERROR;
}

int GpuKernel_setarg(GpuKernel *k, unsigned int i, void *a) { return gpukernel_setarg(k->k, i, a); }

int GpuKernel_call(GpuKernel *k, unsigned int n, const size_t *gs, const size_t *ls,
                   size_t shared, void **args) {
  return gpukernel_call(k->k, n, gs, ls, shared, args);
}

const char *GpuKernel_error(const GpuKernel *k, int err) {
  return gpucontext_error(gpukernel_context(k->k), err);
}

}  // extern "C"
