// GpuArray: views, slicing, reshaping and data movement.
// Semantics follow the reference's src/gpuarray_array.c (cited per function);
// strided and type-converting copies run through GpuElemwise("dst = src").
#include "private.hpp"

#include <map>
#include <string>
#include <utility>
#include <vector>

// ---- strided / converting copy ------------------------------------------------
// One GpuElemwise per (source type, destination type), kept for the life of
// the context (reference ga_extcopy, src/gpuarray_array.c:42-86, which keeps
// them in a small 2Q cache; there are at most a few hundred type pairs, so a
// map that never evicts is simpler and never recompiles).
typedef std::map<std::pair<int, int>, GpuElemwise *> extcopy_map;

void ga_extcopy_cache_free(gpucontext *ctx) {
  extcopy_map *m = (extcopy_map *)ctx->extcopy_cache;
  if (m == nullptr) return;
  ctx->extcopy_cache = nullptr;
  for (auto &kv : *m) GpuElemwise_free(kv.second);
  delete m;
}

static int ga_extcopy(GpuArray *dst, const GpuArray *src) {
  gpucontext *ctx = GpuArray_context(dst);
  if (ctx != GpuArray_context(src))
    return ga_err_set(ctx->err, GA_INVALID_ERROR, "src and dst context differ");
  if (ctx->extcopy_cache == nullptr) ctx->extcopy_cache = new extcopy_map();
  extcopy_map &m = *(extcopy_map *)ctx->extcopy_cache;
  auto key = std::make_pair(src->typecode, dst->typecode);
  GpuElemwise *ge = nullptr;
  auto it = m.find(key);
  if (it != m.end()) {
    ge = it->second;
  } else {
    gpuelemwise_arg gargs[2];
    gargs[0].name = "src";
    gargs[0].typecode = src->typecode;
    gargs[0].flags = GE_READ;
    gargs[1].name = "dst";
    gargs[1].typecode = dst->typecode;
    gargs[1].flags = GE_WRITE;
    // Into a boolean the value is its truth, not its low byte: the reference
    // assigns straight through ("dst = src" into an unsigned char,
    // src/gpuarray_array.c:64), which stores 62 for 62.5 and 0 for 256.
    const char *expr = dst->typecode == GA_BOOL && src->typecode != GA_BOOL ? "dst = (src != 0)"
                                                                            : "dst = src";
    ge = GpuElemwise_new(ctx, "", expr, 2, gargs, 0, GE_CONVERT_F16);
    if (ge == nullptr) return ctx->err->code;
    m[key] = ge;
  }
  void *args[2] = {(void *)src, (void *)dst};
  return GpuElemwise_call(ge, args, GE_BROADCAST);
}

void ga_take1_cache_free(gpucontext *ctx) {
  typedef std::map<std::string, GpuKernel> cache_t;
  void **slot = ga_hip_take1_cache_slot(ctx);
  if (*slot == nullptr) return;
  cache_t *cache = (cache_t *)*slot;
  *slot = nullptr;
  for (auto &kv : *cache) GpuKernel_clear(&kv.second);
  delete cache;
}

// ---- flags ----------------------------------------------------------------------
// A dim of extent 1 never breaks contiguity (reference :1159-1194).

extern "C" int GpuArray_is_c_contiguous(const GpuArray *a) {
  size_t run = GpuArray_ITEMSIZE(a);
  for (unsigned int i = a->nd; i > 0; i--) {
    if (a->dimensions[i - 1] != 1 && a->strides[i - 1] != (ssize_t)run) return 0;
    run *= a->dimensions[i - 1];
  }
  return 1;
}

extern "C" int GpuArray_is_f_contiguous(const GpuArray *a) {
  size_t run = GpuArray_ITEMSIZE(a);
  for (unsigned int i = 0; i < a->nd; i++) {
    if (a->dimensions[i] != 1 && a->strides[i] != (ssize_t)run) return 0;
    run *= a->dimensions[i];
  }
  return 1;
}

extern "C" int GpuArray_is_aligned(const GpuArray *a) {
  size_t al = gpuarray_get_type(a->typecode)->align;
  if (al == 0) al = 1;
  if (a->offset % al != 0) return 0;
  for (unsigned int i = 0; i < a->nd; i++)
    if (a->strides[i] % (ssize_t)al != 0) return 0;
  return 1;
}

static bool mul_overflows(size_t a, size_t b) {
  return b != 0 && a > SIZE_MAX / b;
}

static void contiguous_strides(ssize_t *str, const size_t *dims, unsigned int nd,
                               size_t elsize, ga_order ord) {
  size_t run = elsize;
  if (ord == GA_F_ORDER) {
    for (unsigned int i = 0; i < nd; i++) { str[i] = (ssize_t)run; run *= dims[i]; }
  } else {
    for (unsigned int i = nd; i > 0; i--) { str[i - 1] = (ssize_t)run; run *= dims[i - 1]; }
  }
}

extern "C" {

// A struct that was cleared (or never filled) has no buffer and no context to
// report through: INVALID with a message in the process-wide record, rather
// than a fault further down.
#define NEED_BUFFER(arr)                                                                    \
  do {                                                                                      \
    if ((arr) == nullptr || (arr)->data == nullptr)                                         \
      return ga_err_set(ga_global_err, GA_INVALID_ERROR, "Array has no buffer (cleared?)"); \
  } while (0)

void GpuArray_fix_flags(GpuArray *a) {
  a->flags &= GA_WRITEABLE;
  if (GpuArray_is_c_contiguous(a)) a->flags |= GA_C_CONTIGUOUS;
  if (GpuArray_is_f_contiguous(a)) a->flags |= GA_F_CONTIGUOUS;
  if (GpuArray_is_aligned(a)) a->flags |= GA_ALIGNED;
}

// reference :100-178
int GpuArray_empty(GpuArray *a, gpucontext *ctx, int typecode, unsigned int nd,
                   const size_t *dims, ga_order ord) {
  if (typecode == GA_SIZE || typecode == GA_SSIZE)
    return ga_err_set(ctx->err, GA_VALUE_ERROR, "Cannot create array with size type");
  size_t elsize = gpuarray_get_elsize(typecode);
  if (elsize == 0)
    return ga_err_fmt(ctx->err, GA_VALUE_ERROR, "Unknown typecode %d", typecode);
  if (ord == GA_ANY_ORDER) ord = GA_C_ORDER;
  if (ord != GA_C_ORDER && ord != GA_F_ORDER)
    return ga_err_set(ctx->err, GA_VALUE_ERROR, "Invalid order");

  size_t bytes = elsize;
  for (unsigned int i = 0; i < nd; i++) {
    if (mul_overflows(bytes, dims[i]))
      return ga_err_set(ctx->err, GA_XLARGE_ERROR,
                        "Total array size greater than addressable space");
    bytes *= dims[i];
  }
  // A DEBUG build puts 64 bytes in front of every array, as the reference
  // does (src/gpuarray_array.c:124-137): code that forgets an array's offset
  // then reads or writes the wrong elements in every test instead of only on
  // views.
#ifdef DEBUG
  const size_t lead = 64;
  if (bytes > SIZE_MAX - lead)
    return ga_err_set(ctx->err, GA_XLARGE_ERROR, "Total array size greater than addressable space");
#else
  const size_t lead = 0;
#endif
  memset(a, 0, sizeof(*a));
  int res = GA_NO_ERROR;
  a->data = gpudata_alloc(ctx, bytes + lead, nullptr, 0, &res);
  if (a->data == nullptr) return ctx->err->code;
  a->nd = nd;
  a->offset = lead;
  a->typecode = typecode;
  a->dimensions = (size_t *)calloc(nd ? nd : 1, sizeof(size_t));
  a->strides = (ssize_t *)calloc(nd ? nd : 1, sizeof(ssize_t));
  if (a->dimensions == nullptr || a->strides == nullptr) {
    GpuArray_clear(a);
    return ga_err_sys(ctx->err, "calloc");
  }
  if (nd) memcpy(a->dimensions, dims, nd * sizeof(size_t));
  contiguous_strides(a->strides, a->dimensions, nd, elsize, ord);
  // The reference sets the flag of the requested order only, plus both for
  // nd <= 1 (:160-175).  Computing them also marks shapes like (1, n) or
  // (n, 1) as contiguous both ways, which they are, as NumPy does.
  a->flags = GA_WRITEABLE;
  GpuArray_fix_flags(a);
  return GA_NO_ERROR;
}

int GpuArray_zeros(GpuArray *a, gpucontext *ctx, int typecode, unsigned int nd,
                   const size_t *dims, ga_order ord) {
  int err = GpuArray_empty(a, ctx, typecode, nd, dims, ord);
  if (err != GA_NO_ERROR) return err;
  err = gpudata_memset(a->data, a->offset, 0);
  if (err != GA_NO_ERROR) GpuArray_clear(a);
  return err;
}

// reference :196-222
int GpuArray_fromdata(GpuArray *a, gpudata *data, size_t offset, int typecode,
                      unsigned int nd, const size_t *dims, const ssize_t *strides,
                      int writeable) {
  gpucontext *ctx = gpudata_context(data);
  if (typecode == GA_SIZE || typecode == GA_SSIZE)
    return ga_err_set(ctx->err, GA_VALUE_ERROR, "Cannot create array with size type");
  memset(a, 0, sizeof(*a));
  a->data = data;
  gpudata_retain(data);
  a->nd = nd;
  a->offset = offset;
  a->typecode = typecode;
  a->flags = writeable ? GA_WRITEABLE : 0;
  a->dimensions = (size_t *)calloc(nd ? nd : 1, sizeof(size_t));
  a->strides = (ssize_t *)calloc(nd ? nd : 1, sizeof(ssize_t));
  if (a->dimensions == nullptr || a->strides == nullptr) {
    GpuArray_clear(a);
    return ga_err_set(ctx->err, GA_MEMORY_ERROR, "Out of memory");
  }
  if (nd) {
    memcpy(a->dimensions, dims, nd * sizeof(size_t));
    memcpy(a->strides, strides, nd * sizeof(ssize_t));
  }
  GpuArray_fix_flags(a);
  return GA_NO_ERROR;
}

// reference :224-241
int GpuArray_view(GpuArray *v, const GpuArray *a) {
  gpucontext *ctx = GpuArray_context(a);
  v->data = a->data;
  gpudata_retain(a->data);
  v->nd = a->nd;
  v->offset = a->offset;
  v->typecode = a->typecode;
  v->flags = a->flags;
  v->dimensions = (size_t *)calloc(a->nd ? a->nd : 1, sizeof(size_t));
  v->strides = (ssize_t *)calloc(a->nd ? a->nd : 1, sizeof(ssize_t));
  if (v->dimensions == nullptr || v->strides == nullptr) {
    GpuArray_clear(v);
    return ga_err_set(ctx->err, GA_MEMORY_ERROR, "Out of memory");
  }
  if (a->nd) {
    memcpy(v->dimensions, a->dimensions, a->nd * sizeof(size_t));
    memcpy(v->strides, a->strides, a->nd * sizeof(ssize_t));
  }
  return GA_NO_ERROR;
}

int GpuArray_sync(GpuArray *a) {
  NEED_BUFFER(a);
  return gpudata_sync(a->data);
}

// reference :243-313.  Per dim: start in [-1, len]; with step 0 the start
// must be a valid index; otherwise stop in [-1, len] and the span must run in
// the step's direction.  New extent = (stop-start+step-sign(step))/step.
int GpuArray_index_inplace(GpuArray *a, const ssize_t *starts, const ssize_t *stops,
                           const ssize_t *steps) {
  gpucontext *ctx = GpuArray_context(a);
  if (starts == nullptr || stops == nullptr || steps == nullptr)
    return ga_err_set(ctx->err, GA_VALUE_ERROR, "Invalid slice (contains NULL)");

  std::vector<size_t> nd_dims;
  std::vector<ssize_t> nd_strs;
  size_t off = a->offset;
  for (unsigned int i = 0; i < a->nd; i++) {
    const ssize_t st = starts[i], sp = stops[i], step = steps[i];
    const size_t len = a->dimensions[i];
    bool bad = st < -1 || (st > 0 && (size_t)st > len);
    if (!bad && step == 0) bad = st == -1 || (size_t)st >= len;
    if (!bad && step != 0)
      bad = sp < -1 || (sp > 0 && (size_t)sp > len) || (sp - st) / step < 0;
    if (bad)
      return ga_err_fmt(ctx->err, GA_VALUE_ERROR,
                        "Invalid slice value: slice(%lld, %lld, %lld) when indexing array on "
                        "dimension %u of length %lld",
                        (long long)st, (long long)sp, (long long)step, i, (long long)len);
    off += (size_t)(st * a->strides[i]);
    if (step != 0) {
      nd_strs.push_back(step * a->strides[i]);
      nd_dims.push_back((size_t)((sp - st + step - (step < 0 ? -1 : 1)) / step));
    }
  }
  unsigned int nnd = (unsigned int)nd_dims.size();
  size_t *newdims = (size_t *)calloc(nnd ? nnd : 1, sizeof(size_t));
  ssize_t *newstrs = (ssize_t *)calloc(nnd ? nnd : 1, sizeof(ssize_t));
  if (newdims == nullptr || newstrs == nullptr) {
    free(newdims);
    free(newstrs);
    return ga_err_sys(ctx->err, "calloc");
  }
  for (unsigned int i = 0; i < nnd; i++) {
    newdims[i] = nd_dims[i];
    newstrs[i] = nd_strs[i];
  }
  free(a->dimensions);
  free(a->strides);
  a->dimensions = newdims;
  a->strides = newstrs;
  a->nd = nnd;
  a->offset = off;
  GpuArray_fix_flags(a);
  return GA_NO_ERROR;
}

int GpuArray_index(GpuArray *r, const GpuArray *a, const ssize_t *starts,
                   const ssize_t *stops, const ssize_t *steps) {
  int err = GpuArray_view(r, a);
  if (err != GA_NO_ERROR) return err;
  err = GpuArray_index_inplace(r, starts, stops, steps);
  if (err != GA_NO_ERROR) GpuArray_clear(r);
  return err;
}

// reference :550-609
int GpuArray_setarray(GpuArray *a, const GpuArray *v) {
  gpucontext *ctx = GpuArray_context(a);
  if (a->nd < v->nd)
    return ga_err_fmt(ctx->err, GA_VALUE_ERROR, "Dimension error. a->nd = %u, v->nd = %u", a->nd,
                      v->nd);
  if (!GpuArray_ISWRITEABLE(a))
    return ga_err_set(ctx->err, GA_VALUE_ERROR, "Destination array not writable");
  if (!GpuArray_ISALIGNED(v) || !GpuArray_ISALIGNED(a))
    return ga_err_set(ctx->err, GA_UNALIGNED_ERROR, "One of the inputs is unaligned");

  const unsigned int off = a->nd - v->nd;
  bool same_shape = true;
  for (unsigned int i = 0; i < v->nd; i++) {
    if (v->dimensions[i] == a->dimensions[i + off]) continue;
    if (v->dimensions[i] != 1)
      return ga_err_fmt(ctx->err, GA_VALUE_ERROR,
                        "Shape error. v->dimensions[%u] = %zu, a->dimensions[%u + %u] = %zu", i,
                        v->dimensions[i], i, off, a->dimensions[i + off]);
    same_shape = false;
  }
  if (same_shape && a->nd == v->nd && a->typecode == v->typecode &&
      GpuArray_ISONESEGMENT(a) && GpuArray_ISONESEGMENT(v) &&
      GpuArray_ISFORTRAN(a) == GpuArray_ISFORTRAN(v)) {
    size_t sz = gpuarray_get_elsize(a->typecode);
    for (unsigned int i = 0; i < a->nd; i++) sz *= a->dimensions[i];
    return gpudata_move(a->data, a->offset, v->data, v->offset, sz);
  }
  // View v with a's shape: broadcast dims get stride 0.
  std::vector<ssize_t> strs(a->nd ? a->nd : 1, 0);
  for (unsigned int i = off; i < a->nd; i++)
    if (v->dimensions[i - off] == a->dimensions[i]) strs[i] = v->strides[i - off];
  GpuArray tv = *v;
  tv.nd = a->nd;
  tv.dimensions = a->dimensions;
  tv.strides = strs.data();
  if (tv.nd != 0) GpuArray_fix_flags(&tv);
  return ga_extcopy(a, &tv);
}

// No-copy reshape (reference :625-772).  The old and new shapes are cut into
// groups of equal element count; a group of old dims can be re-split iff the
// array walks it as one evenly strided run in the requested order.  Old dims
// of extent 1 carry no layout information and are dropped first.
int GpuArray_reshape_inplace(GpuArray *a, unsigned int nd, const size_t *newdims,
                             ga_order ord) {
  gpucontext *ctx = GpuArray_context(a);
  if (ord == GA_ANY_ORDER) ord = (GpuArray_ISFORTRAN(a) && a->nd > 1) ? GA_F_ORDER : GA_C_ORDER;

  size_t oldsize = 1, newsize = 1;
  for (unsigned int i = 0; i < a->nd; i++) oldsize *= a->dimensions[i];
  for (unsigned int i = 0; i < nd; i++) {
    if (mul_overflows(newsize, newdims[i]))
      return ga_err_set(ctx->err, GA_XLARGE_ERROR,
                        "Output array size greater than addressable space");
    newsize *= newdims[i];
  }
  if (newsize != oldsize)
    return ga_err_set(ctx->err, GA_INVALID_ERROR, "New shape differs in total size");

  const size_t elsize = gpuarray_get_elsize(a->typecode);
  std::vector<ssize_t> ns(nd ? nd : 1, 0);

  const bool already = (ord == GA_C_ORDER && GpuArray_CHKFLAGS(a, GA_C_CONTIGUOUS)) ||
                       (ord == GA_F_ORDER && GpuArray_CHKFLAGS(a, GA_F_CONTIGUOUS));
  if (already || newsize == 0) {
    contiguous_strides(ns.data(), newdims, nd, elsize, ord);
  } else {
    // Work in "slowest first" order; F order is the mirror image.
    std::vector<size_t> od, nw(nd);
    std::vector<ssize_t> os;
    for (unsigned int i = 0; i < a->nd; i++) {
      unsigned int k = ord == GA_F_ORDER ? a->nd - 1 - i : i;
      if (a->dimensions[k] == 1) continue;
      od.push_back(a->dimensions[k]);
      os.push_back(a->strides[k]);
    }
    for (unsigned int i = 0; i < nd; i++) nw[i] = newdims[ord == GA_F_ORDER ? nd - 1 - i : i];
    std::vector<ssize_t> res(nd ? nd : 1, (ssize_t)elsize);
    size_t oi = 0, ni = 0;
    while (ni < nd && oi < od.size()) {
      size_t np = nw[ni], op = od[oi], nj = ni + 1, oj = oi + 1;
      while (np != op) {
        if (np < op) np *= nw[nj++];
        else op *= od[oj++];
      }
      for (size_t k = oi; k + 1 < oj; k++)
        if (os[k] != (ssize_t)od[k + 1] * os[k + 1])
          return ga_err_set(ctx->err, GA_COPY_ERROR,
                            "Copy is needed but disallowed by parameters");
      res[nj - 1] = os[oj - 1];
      for (size_t k = nj - 1; k > ni; k--) res[k - 1] = res[k] * (ssize_t)nw[k];
      ni = nj;
      oi = oj;
    }
    // what is left on the new side are extents of 1: any stride does, use
    // the element size
    for (unsigned int i = 0; i < nd; i++) ns[ord == GA_F_ORDER ? nd - 1 - i : i] = res[i];
  }

  size_t *dcopy = (size_t *)calloc(nd ? nd : 1, sizeof(size_t));
  ssize_t *scopy = (ssize_t *)calloc(nd ? nd : 1, sizeof(ssize_t));
  if (dcopy == nullptr || scopy == nullptr) {
    free(dcopy);
    free(scopy);
    return ga_err_sys(ctx->err, "calloc");
  }
  for (unsigned int i = 0; i < nd; i++) {
    dcopy[i] = newdims[i];
    scopy[i] = ns[i];
  }
  free(a->dimensions);
  free(a->strides);
  a->dimensions = dcopy;
  a->strides = scopy;
  a->nd = nd;
  GpuArray_fix_flags(a);
  return GA_NO_ERROR;
}

// reference :611-623
int GpuArray_reshape(GpuArray *res, const GpuArray *a, unsigned int nd, const size_t *newdims,
                     ga_order ord, int nocopy) {
  int err = GpuArray_view(res, a);
  if (err != GA_NO_ERROR) return err;
  err = GpuArray_reshape_inplace(res, nd, newdims, ord);
  if (err == GA_COPY_ERROR && !nocopy) {
    GpuArray_clear(res);
    err = GpuArray_copy(res, a, ord);
    if (err != GA_NO_ERROR) return err;
    err = GpuArray_reshape_inplace(res, nd, newdims, ord);
  }
  if (err != GA_NO_ERROR) GpuArray_clear(res);
  return err;
}

// reference :785-828: NULL reverses the axes; a repeated axis is an error.
int GpuArray_transpose_inplace(GpuArray *a, const unsigned int *new_axes) {
  gpucontext *ctx = GpuArray_context(a);
  const unsigned int nd = a->nd;
  std::vector<size_t> d(nd ? nd : 1);
  std::vector<ssize_t> s(nd ? nd : 1);
  std::vector<char> seen(nd ? nd : 1, 0);
  for (unsigned int i = 0; i < nd; i++) {
    unsigned int j = new_axes == nullptr ? nd - 1 - i : new_axes[i];
    if (j >= nd)
      return ga_err_fmt(ctx->err, GA_VALUE_ERROR, "Axis %u out of range in transpose (nd = %u)", j,
                        nd);
    if (seen[j])
      return ga_err_fmt(ctx->err, GA_VALUE_ERROR, "Repeated axes in transpose: axis %u", j);
    seen[j] = 1;
    d[i] = a->dimensions[j];
    s[i] = a->strides[j];
  }
  for (unsigned int i = 0; i < nd; i++) {
    a->dimensions[i] = d[i];
    a->strides[i] = s[i];
  }
  GpuArray_fix_flags(a);
  return GA_NO_ERROR;
}

int GpuArray_transpose(GpuArray *res, const GpuArray *a, const unsigned int *new_axes) {
  int err = GpuArray_view(res, a);
  if (err != GA_NO_ERROR) return err;
  err = GpuArray_transpose_inplace(res, new_axes);
  if (err != GA_NO_ERROR) GpuArray_clear(res);
  return err;
}

void GpuArray_clear(GpuArray *a) {
  if (a->data) gpudata_release(a->data);
  free(a->dimensions);
  free(a->strides);
  memset(a, 0, sizeof(*a));
}

int GpuArray_share(const GpuArray *a, const GpuArray *b) {
  if (a->data != b->data) return 0;
  return gpudata_share(a->data, b->data, nullptr);
}

gpucontext *GpuArray_context(const GpuArray *a) { return gpudata_context(a->data); }

// reference :849-877
int GpuArray_move(GpuArray *dst, const GpuArray *src) {
  NEED_BUFFER(dst);
  NEED_BUFFER(src);
  gpucontext *ctx = GpuArray_context(dst);
  if (!GpuArray_ISWRITEABLE(dst))
    return ga_err_set(ctx->err, GA_VALUE_ERROR, "Destination array (dst) not writeable");
  if (!GpuArray_ISALIGNED(src))
    return ga_err_set(ctx->err, GA_UNALIGNED_ERROR, "Source array (src) not aligned");
  if (!GpuArray_ISALIGNED(dst))
    return ga_err_set(ctx->err, GA_UNALIGNED_ERROR, "Destination array (dst) not aligned");
  if (src->nd != dst->nd)
    return ga_err_fmt(ctx->err, GA_VALUE_ERROR, "Dimension mismatch. src->nd = %u, dst->nd = %u",
                      src->nd, dst->nd);
  for (unsigned int i = 0; i < src->nd; i++)
    if (src->dimensions[i] != dst->dimensions[i])
      return ga_err_fmt(ctx->err, GA_VALUE_ERROR,
                        "Dimension mismatch. src->dimensions[%u] = %zu, dst->dimensions[%u] = %zu",
                        i, src->dimensions[i], i, dst->dimensions[i]);
  if (!GpuArray_ISONESEGMENT(dst) || !GpuArray_ISONESEGMENT(src) ||
      GpuArray_ISFORTRAN(dst) != GpuArray_ISFORTRAN(src) || dst->typecode != src->typecode)
    return ga_extcopy(dst, src);
  size_t sz = gpuarray_get_elsize(dst->typecode);
  for (unsigned int i = 0; i < dst->nd; i++) sz *= dst->dimensions[i];
  return gpudata_move(dst->data, dst->offset, src->data, src->offset, sz);
}

// reference :879-900
int GpuArray_write(GpuArray *dst, const void *src, size_t src_sz) {
  NEED_BUFFER(dst);
  gpucontext *ctx = GpuArray_context(dst);
  if (!GpuArray_ISWRITEABLE(dst))
    return ga_err_set(ctx->err, GA_VALUE_ERROR, "Destination array (dst) not writeable");
  if (!GpuArray_ISONESEGMENT(dst))
    return ga_err_set(ctx->err, GA_UNSUPPORTED_ERROR, "Destination array (dst) not one segment");
  return gpudata_write(dst->data, dst->offset, src, src_sz);
}

int GpuArray_read(void *dst, size_t dst_sz, const GpuArray *src) {
  NEED_BUFFER(src);
  gpucontext *ctx = GpuArray_context(src);
  if (!GpuArray_ISONESEGMENT(src))
    return ga_err_set(ctx->err, GA_UNSUPPORTED_ERROR, "Array (src) not one segment");
  return gpudata_read(dst, src->data, src->offset, dst_sz);
}

int GpuArray_memset(GpuArray *a, int data) {
  NEED_BUFFER(a);
  gpucontext *ctx = GpuArray_context(a);
  if (!GpuArray_ISONESEGMENT(a))
    return ga_err_set(ctx->err, GA_UNSUPPORTED_ERROR, "Array (a) not one segment");
  return gpudata_memset(a->data, a->offset, data);
}

int GpuArray_copy(GpuArray *res, const GpuArray *a, ga_order order) {
  NEED_BUFFER(a);
  int err = GpuArray_empty(res, GpuArray_context(a), a->typecode, a->nd, a->dimensions, order);
  if (err != GA_NO_ERROR) return err;
  err = GpuArray_move(res, a);
  if (err != GA_NO_ERROR) GpuArray_clear(res);
  return err;
}

// reference :913-932
int GpuArray_transfer(GpuArray *res, const GpuArray *a) {
  NEED_BUFFER(res);
  NEED_BUFFER(a);
  gpucontext *ctx = GpuArray_context(res);
  if (!GpuArray_ISONESEGMENT(res))
    return ga_err_set(ctx->err, GA_UNSUPPORTED_ERROR, "Array (res) not one segment");
  if (!GpuArray_ISONESEGMENT(a))
    return ga_err_set(ctx->err, GA_UNSUPPORTED_ERROR, "Array (a) not one segment");
  if (res->typecode != a->typecode)
    return ga_err_set(ctx->err, GA_UNSUPPORTED_ERROR, "typecode mismatch");
  size_t sz = gpuarray_get_elsize(a->typecode);
  for (unsigned int i = 0; i < a->nd; i++) sz *= a->dimensions[i];
  return gpudata_transfer(res->data, res->offset, a->data, a->offset, sz);
}

// reference :934-980: n cut points give n+1 views along `axis`.
int GpuArray_split(GpuArray **rs, const GpuArray *a, size_t n, size_t *p, unsigned int axis) {
  gpucontext *ctx = GpuArray_context(a);
  if (axis >= a->nd)
    return ga_err_fmt(ctx->err, GA_VALUE_ERROR, "Invalid axis %u for an array of %u dimensions",
                      axis, a->nd);
  std::vector<ssize_t> starts(a->nd, 0), stops(a->nd), steps(a->nd, 1);
  for (unsigned int i = 0; i < a->nd; i++) stops[i] = (ssize_t)a->dimensions[i];
  int err = GA_NO_ERROR;
  size_t i;
  for (i = 0; i <= n; i++) {
    starts[axis] = i > 0 ? (ssize_t)p[i - 1] : 0;
    stops[axis] = i < n ? (ssize_t)p[i] : (ssize_t)a->dimensions[axis];
    err = GpuArray_index(rs[i], a, starts.data(), stops.data(), steps.data());
    if (err != GA_NO_ERROR) break;
  }
  if (err != GA_NO_ERROR)
    for (size_t k = 0; k < i; k++) GpuArray_clear(rs[k]);
  return err;
}

// reference :982-1065: all inputs share every extent but `axis`; the result
// is filled piece by piece through a window of the result array.
int GpuArray_concatenate(GpuArray *r, const GpuArray **as, size_t n, unsigned int axis,
                         int restype) {
  gpucontext *ctx = GpuArray_context(as[0]);
  const unsigned int nd = as[0]->nd;
  if (axis >= nd)
    return ga_err_fmt(ctx->err, GA_VALUE_ERROR, "Invalid axis. axis = %u, as[0]->nd = %u", axis, nd);
  std::vector<size_t> dims(as[0]->dimensions, as[0]->dimensions + nd);
  for (size_t i = 0; i < n; i++) {
    if (!GpuArray_ISALIGNED(as[i]))
      return ga_err_fmt(ctx->err, GA_UNALIGNED_ERROR, "Unaligned array (as[%zu]).", i);
    if (i == 0) continue;
    if (as[i]->nd != nd)
      return ga_err_fmt(ctx->err, GA_VALUE_ERROR,
                        "Shape mismatch. as[%zu]->nd = %u, as[0]->nd = %u", i, as[i]->nd, nd);
    for (unsigned int d = 0; d < nd; d++) {
      if (d == axis) {
        dims[d] += as[i]->dimensions[d];
      } else if (dims[d] != as[i]->dimensions[d]) {
        return ga_err_fmt(ctx->err, GA_VALUE_ERROR,
                          "Dimension mismatch. as[%zu]->dimensions[%u] = %zu, "
                          "as[0]->dimensions[%u] = %zu",
                          i, d, as[i]->dimensions[d], d, dims[d]);
      }
    }
  }
  int err = GpuArray_empty(r, ctx, restype, nd, dims.data(), GA_ANY_ORDER);
  if (err != GA_NO_ERROR) return err;

  GpuArray win = *r;   // borrowed window over r's storage
  std::vector<size_t> wdims(nd);
  win.dimensions = wdims.data();
  for (size_t i = 0; i < n; i++) {
    for (unsigned int d = 0; d < nd; d++) wdims[d] = as[i]->dimensions[d];
    GpuArray_fix_flags(&win);
    err = ga_extcopy(&win, as[i]);
    if (err != GA_NO_ERROR) {
      GpuArray_clear(r);
      return err;
    }
    win.offset += (size_t)(r->strides[axis] * (ssize_t)as[i]->dimensions[axis]);
  }
  return GA_NO_ERROR;
}

const char *GpuArray_error(const GpuArray *a, int err) {
  return gpucontext_error(gpudata_context(a->data), err);
}

void GpuArray_fprintf(FILE *fd, const GpuArray *a) {
  fprintf(fd, "GpuArray <%p, data: %p (%p)> nd=%u\n", (const void *)a, (void *)a->data,
          a->data ? a->data->devptr : nullptr, a->nd);
  fprintf(fd, "\tITEMSIZE: %zu\n\tTYPECODE: %d\n\tOFFSET: %zu\n\tHOST_DIMS:      ",
          GpuArray_ITEMSIZE(a), a->typecode, a->offset);
  for (unsigned int i = 0; i < a->nd; i++) fprintf(fd, "%zu\t", a->dimensions[i]);
  fprintf(fd, "\n\tHOST_STRIDES: ");
  for (unsigned int i = 0; i < a->nd; i++) fprintf(fd, "%zd\t", a->strides[i]);
  fprintf(fd, "\nFLAGS:");
  const struct { int bit; const char *name; } names[] = {
      {GA_C_CONTIGUOUS, "GA_C_CONTIGUOUS"}, {GA_F_CONTIGUOUS, "GA_F_CONTIGUOUS"},
      {GA_ALIGNED, "GA_ALIGNED"},           {GA_WRITEABLE, "GA_WRITEABLE"}};
  bool first = true;
  for (const auto &nm : names) {
    if (!(a->flags & nm.bit)) continue;
    fprintf(fd, "%s %s", first ? "" : ",", nm.name);
    first = false;
  }
  fputc('\n', fd);
}

// reference :1113-1157: one "[k] = value" line per element, four types only.
int GpuArray_fdump(FILE *fd, const GpuArray *a) {
  gpucontext *ctx = GpuArray_context(a);
  const size_t el = GpuArray_ITEMSIZE(a);
  size_t count = 1;
  for (unsigned int i = 0; i < a->nd; i++) count *= a->dimensions[i];
  if (a->typecode != GA_UINT && a->typecode != GA_LONG && a->typecode != GA_FLOAT &&
      a->typecode != GA_SSIZE) {
    fprintf(fd, "<unsupported data type %d>\n", a->typecode);
    return ga_err_fmt(ctx->err, GA_UNSUPPORTED_ERROR, "Unsupported data type for dump: %d",
                      a->typecode);
  }
  std::vector<char> buf(count * el != 0 ? count * el : 1);
  int err = GpuArray_read(buf.data(), count * el, a);
  if (err != GA_NO_ERROR) return err;
  for (size_t k = 0; k < count; k++) {
    const char *p = buf.data() + k * el;
    fprintf(fd, "[%zu] = ", k);
    switch (a->typecode) {
    case GA_UINT: { uint32_t v; memcpy(&v, p, 4); fprintf(fd, "%u", v); break; }
    case GA_LONG: { int64_t v; memcpy(&v, p, 8); fprintf(fd, "%lld", (long long)v); break; }
    case GA_FLOAT: { float v; memcpy(&v, p, 4); fprintf(fd, "%f", v); break; }
    default: { ssize_t v; memcpy(&v, p, sizeof(v)); fprintf(fd, "%zd", v); break; }
    }
    fputc('\n', fd);
  }
  return GA_NO_ERROR;
}

}  // extern "C"

// Kernel text of GpuArray_take1 for one combination of types and collapsed
// trailing rank; `types` receives the argument typecodes.
// Short dense rows (at most 128 chunks of 16 bytes): a power-of-two number of
// lanes covers a row with one chunk each, and a lane moves the same chunk of
// four rows, so that one load instruction fetches whole rows and the four
// index loads, the four row loads and the four stores each go out together.
// Same arguments as the general kernel (gx is 1 and unused).
static std::string take1_short_rows_source(int i_tc, std::vector<int> &types) {
  const gpuarray_type *ti = gpuarray_get_type(i_tc);
  std::string s =
      "#include \"cluda.h\"\n"
      "typedef ga_uint t1_chunk __attribute__((ext_vector_type(4)));\n"
      "KERNEL void __launch_bounds__(256) take1(GLOBAL_MEM t1_chunk *r, const ga_size r_off, "
      "GLOBAL_MEM const char *v, const ga_size v_off, const ga_ssize s0, const ga_size d0, "
      "const ga_ssize s1, const ga_size d1, GLOBAL_MEM const ";
  s += ti->cluda_name;
  s += " *ind, const ga_size i_off, const ga_size n0, const ga_size n1, const ga_uint gx, "
       "const ga_uint lsh, GLOBAL_MEM ga_int *err) {\n"
       "  const ga_uint lane = LID_0 & ((1u << lsh) - 1u);\n"
       "  const ga_uint rpg = 256u >> lsh;\n"
       "  const ga_size row0 = (ga_size)GID_0 * 4u * rpg + (LID_0 >> lsh);\n"
       "  ind = (GLOBAL_MEM const ";
  s += ti->cluda_name;
  s += " *)((GLOBAL_MEM const char *)ind + i_off);\n"
       "  r = (GLOBAL_MEM t1_chunk *)((GLOBAL_MEM char *)r + r_off);\n"
       "  v += v_off + (ga_size)lane * 16u;\n"
       "  ga_long ii[4];\n"
       "#pragma unroll\n"
       "  for (int e = 0; e < 4; e++) {\n"
       "    const ga_size row = row0 + (ga_size)e * rpg;\n"
       // the reference reads the index as signed (src/gpuarray_array.c:385-391)
       "    ii[e] = row < n0 ? (ga_long)ind[row] : 0;\n"
       "  }\n"
       "  bool ok[4];\n"
       "  bool bad = false;\n"
       "#pragma unroll\n"
       "  for (int e = 0; e < 4; e++) {\n"
       "    if (ii[e] < 0) ii[e] += (ga_long)d0;\n"
       "    const bool in_range = ii[e] >= 0 && ii[e] < (ga_long)d0;\n"
       "    const bool live = row0 + (ga_size)e * rpg < n0;\n"
       "    bad = bad || (live && !in_range);\n"
       "    ok[e] = live && in_range && lane < n1;\n"
       "  }\n"
       "  if (bad && lane == 0) *err = -1;\n"
       "  t1_chunk t[4];\n"
       "#pragma unroll\n"
       "  for (int e = 0; e < 4; e++)\n"
       "    if (ok[e]) t[e] = __builtin_nontemporal_load((GLOBAL_MEM const t1_chunk *)(v + ii[e] * s0));\n"
       "#pragma unroll\n"
       "  for (int e = 0; e < 4; e++)\n"
       "    if (ok[e]) __builtin_nontemporal_store(t[e], r + (row0 + (ga_size)e * rpg) * n1 + lane);\n"
       "}\n";
  types = {GA_BUFFER, GA_SIZE, GA_BUFFER, GA_SIZE, GA_SSIZE, GA_SIZE, GA_SSIZE, GA_SIZE,
           GA_BUFFER, GA_SIZE, GA_SIZE, GA_SIZE, GA_UINT, GA_UINT, GA_BUFFER};
  return s;
}

static std::string take1_source(bool chunks, int a_tc, int v_tc, int i_tc, unsigned int tnd,
                                std::vector<int> &types) {
    const gpuarray_type *ta = gpuarray_get_type(a_tc), *tv = gpuarray_get_type(v_tc),
                      *ti = gpuarray_get_type(i_tc);
    // halves move as their 16 bits (both sides are half then)
    const std::string rt = chunks ? "t1_chunk" : (a_tc == GA_HALF ? "ga_ushort" : ta->cluda_name),
                      vt = chunks ? "t1_chunk" : (v_tc == GA_HALF ? "ga_ushort" : tv->cluda_name);
    std::string s = "#include \"cluda.h\"\n"
                    "typedef ga_uint t1_chunk __attribute__((ext_vector_type(4)));\n"
                    "KERNEL void __launch_bounds__(256) take1(GLOBAL_MEM " + rt +
                    " *r, const ga_size r_off, GLOBAL_MEM const char *v, const ga_size v_off, "
                    "const ga_ssize s0, const ga_size d0";
    types = {GA_BUFFER, GA_SIZE, GA_BUFFER, GA_SIZE, GA_SSIZE, GA_SIZE};
    for (unsigned int d = 0; d < tnd; d++) {
      char b[96];
      snprintf(b, sizeof(b), ", const ga_ssize s%u, const ga_size d%u", d + 1, d + 1);
      s += b;
      types.push_back(GA_SSIZE);
      types.push_back(GA_SIZE);
    }
    s += std::string(", GLOBAL_MEM const ") + ti->cluda_name +
         " *ind, const ga_size i_off, const ga_size n0, const ga_size n1, const ga_uint gx, "
         "const ga_uint lsh, GLOBAL_MEM ga_int *err) {\n"
         "  const ga_uint lane = LID_0 & ((1u << lsh) - 1u);\n"
         "  const ga_size row = (ga_size)(GID_0 / gx) * (256u >> lsh) + (LID_0 >> lsh);\n"
         "  if (row >= n0) return;\n"
         "  const ga_size x0 = (ga_size)(GID_0 % gx) * (4u << lsh) + lane;\n"
         "  ind = (GLOBAL_MEM const " + ti->cluda_name + " *)((GLOBAL_MEM const char *)ind + i_off);\n"
         // as the reference (`ssize ii0 = ind[i0]`, src/gpuarray_array.c:385-391): an
         // unsigned 64-bit index of 2^63 or more is seen as negative and wraps once
         "  ga_long ii = (ga_long)ind[row];\n"
         "  if (ii < 0) ii += (ga_long)d0;\n"
         "  if (ii < 0 || ii >= (ga_long)d0) { if (lane == 0) *err = -1; return; }\n"
         "  v += v_off + ii * s0;\n"
         "  r = (GLOBAL_MEM " + rt + " *)((GLOBAL_MEM char *)r + r_off) + row * n1;\n"
         "  " + vt + " t[4];\n"
         "#pragma unroll\n"
         "  for (int e = 0; e < 4; e++) {\n"
         "    const ga_size x = x0 + ((ga_size)e << lsh);\n"
         "    if (x < n1) {\n"
         "      ga_ssize p = 0; ga_size c = x;\n";
    for (unsigned int d = tnd; d > 1; d--) {
      char b[128];
      snprintf(b, sizeof(b), "      p += (ga_ssize)(c %% d%u) * s%u; c /= d%u;\n", d, d, d);
      s += b;
    }
    s += "      p += (ga_ssize)c * s1;\n"
         "      t[e] = __builtin_nontemporal_load((GLOBAL_MEM const " + vt + " *)(v + p));\n"
         "    }\n  }\n"
         "#pragma unroll\n"
         "  for (int e = 0; e < 4; e++) {\n"
         "    const ga_size x = x0 + ((ga_size)e << lsh);\n";
    if (chunks || a_tc == v_tc)
      s += "    if (x < n1) __builtin_nontemporal_store(t[e], r + x);\n";
    else
      s += "    if (x < n1) r[x] = t[e];\n";
    s += "  }\n}\n";
    for (int t : {GA_BUFFER, GA_SIZE, GA_SIZE, GA_SIZE, GA_UINT, GA_UINT, GA_BUFFER}) types.push_back(t);
    return s;
}

extern "C" GPUARRAY_PUBLIC char *ga_take1_gen_source(int chunks, int a_tc, int v_tc, int i_tc,
                                                     unsigned int tnd) {
  std::vector<int> types;
  // chunks: 0 element by element, 1 rows as 16-byte chunks, 2 the kernel for short dense rows
  if (chunks == 2) return strdup(take1_short_rows_source(i_tc, types).c_str());
  return strdup(take1_source(chunks != 0, a_tc, v_tc, i_tc, tnd, types).c_str());
}

extern "C" {

// a[k, ...] = v[i[k], ...]  (reference :325-548).  Rules kept: a and i are
// C-contiguous, i is 1-D with a's leading extent, trailing extents of a and v
// agree, every array is aligned; a negative index counts from the end; an
// index out of range leaves its row untouched and sets the context's error
// word, which `check_error` reads back (blocking), resets, and reports as
// GA_VALUE_ERROR "Index out of bounds".
// The kernel is a row copy: the trailing dims of v are collapsed on the host
// (one dim when v's rows are dense); a power-of-two number of lanes shares an
// output row (a group of 256 lanes holds 256/lanes rows, so short rows still
// fill it), lanes run along the columns so both sides are coalesced, every
// lane has up to four streaming loads in flight before it stores, and the
// index is read once per lane instead of once per element.  Dense aligned
// rows of one type on both sides move as 16-byte chunks.  Kernels are
// kept per context by (types, collapsed rank), so repeated calls compile
// nothing; the reference rebuilds its kernel on every call (:469-477).
int GpuArray_take1(GpuArray *a, const GpuArray *v, const GpuArray *i, int check_error) {
  gpucontext *ctx = GpuArray_context(a);
  if (!GpuArray_ISWRITEABLE(a))
    return ga_err_set(ctx->err, GA_VALUE_ERROR, "Destination array not writeable");
  if (!GpuArray_ISALIGNED(a) || !GpuArray_ISALIGNED(v) || !GpuArray_ISALIGNED(i))
    return ga_err_fmt(ctx->err, GA_UNALIGNED_ERROR,
                      "Not all arrays are aligned: a (%d), b (%d), i (%d)", GpuArray_ISALIGNED(a),
                      GpuArray_ISALIGNED(v), GpuArray_ISALIGNED(i));
  if (!GpuArray_IS_C_CONTIGUOUS(a))
    return ga_err_set(ctx->err, GA_INVALID_ERROR, "Destination array (a) not C-contiguous");
  if (!GpuArray_IS_C_CONTIGUOUS(i))
    return ga_err_set(ctx->err, GA_INVALID_ERROR, "Index array (i) not C-contiguous");
  if (v->nd == 0 || a->nd == 0 || i->nd != 1 || a->nd != v->nd)
    return ga_err_fmt(ctx->err, GA_INVALID_ERROR,
                      "Dimension mismatch. v->nd = %u, a->nd = %u, i->nd = %u", v->nd, a->nd, i->nd);
  if (a->dimensions[0] != i->dimensions[0])
    return ga_err_fmt(ctx->err, GA_INVALID_ERROR,
                      "Dimension mismatch. a->dimensions[0] = %zu, i->dimensions[0] = %zu",
                      a->dimensions[0], i->dimensions[0]);
  size_t n0 = i->dimensions[0], n1 = 1;
  for (unsigned int j = 1; j < v->nd; j++) {
    if (a->dimensions[j] != v->dimensions[j])
      return ga_err_fmt(ctx->err, GA_INVALID_ERROR,
                        "Dimension mismatch. a->dimensions[%u] = %zu, v->dimensions[%u] = %zu", j,
                        a->dimensions[j], j, v->dimensions[j]);
    n1 *= v->dimensions[j];
  }
  const gpuarray_type *tv = gpuarray_get_type(v->typecode);
  if (i->typecode < GA_BYTE || i->typecode > GA_ULONG)
    return ga_err_set(ctx->err, GA_VALUE_ERROR, "Index array must have an integer type");
  if (gpuarray_type_flags(a->typecode, v->typecode, -1) & GA_USE_COMPLEX)
    return ga_err_set(ctx->err, GA_UNSUPPORTED_ERROR, "Complex types are not supported");
  if (n0 == 0 || n1 == 0) return GA_NO_ERROR;

  // collapse v's trailing dims into as few strided runs as possible
  unsigned int tnd = v->nd - 1;
  std::vector<size_t> tdims(v->dimensions + 1, v->dimensions + v->nd);
  std::vector<ssize_t> tstr(v->strides + 1, v->strides + v->nd);
  if (tnd == 0) {
    tnd = 1;
    tdims.assign(1, 1);
    tstr.assign(1, 0);
  } else {
    ssize_t *row = tstr.data();
    gpuarray_elemwise_collapse(1, &tnd, tdims.data(), &row);
  }

  if ((a->typecode == GA_HALF) != (v->typecode == GA_HALF))
    return ga_err_set(ctx->err, GA_UNSUPPORTED_ERROR, "take1 between half and another type");

  // Rows that are dense, of the same type on both sides and 16-byte aligned
  // move as 16-byte chunks whatever the element type.
  const size_t elsz = tv->size;
  bool chunks = a->typecode == v->typecode && tnd == 1 && (tstr[0] == (ssize_t)elsz || n1 == 1) &&
                (n1 * elsz) % 16 == 0 && v->strides[0] % 16 == 0 &&
                ((uintptr_t)v->data->devptr + v->offset) % 16 == 0 &&
                ((uintptr_t)a->data->devptr + a->offset) % 16 == 0;
  size_t n1e = n1;               // elements (or chunks) per row
  if (chunks) {
    n1e = n1 * elsz / 16;
    tdims[0] = n1e;
    tstr[0] = 16;
  }
  // Rows of at most 128 chunks: one chunk per lane, four rows per lane.
  // Kernel time for a 256 MiB table gathered in random order, general kernel
  // against this one: rows of 64 floats 139 -> 91 us, of 32 floats 344 -> 92,
  // of 16 floats 684 -> 139, of 8 floats 466 -> 225; from 128 floats on both
  // take 90 to 91 us.
  const bool short_rows = chunks && n1e <= TUNE(ga_hip_tuning(ctx), TAKE1_SHORT_ROWS, 128);
  // lanes per row: a power of two, each lane moves up to four elements
  unsigned int lsh = 0;
  while (lsh < 8 && ((size_t)(short_rows ? 1 : 4) << lsh) < n1e) lsh++;
  const size_t rpg = ((size_t)256 >> lsh) * (short_rows ? 4 : 1);   // rows per group
  const size_t gx = short_rows ? 1 : (n1e + ((size_t)4 << lsh) - 1) / ((size_t)4 << lsh);
  const size_t gy = (n0 + rpg - 1) / rpg;
  if (gx > 0xffffffffull || gy > 0x7fffffffull / gx)
    return ga_err_set(ctx->err, GA_XLARGE_ERROR, "take1 needs more groups than one launch has");

  typedef std::map<std::string, GpuKernel> cache_t;
  void **slot = ga_hip_take1_cache_slot(ctx);
  if (*slot == nullptr) *slot = new cache_t();
  cache_t &cache = *(cache_t *)*slot;
  char key[64];
  if (short_rows) snprintf(key, sizeof(key), "r:%d", i->typecode);
  else if (chunks) snprintf(key, sizeof(key), "c:%d", i->typecode);
  else snprintf(key, sizeof(key), "%d:%d:%d:%u", a->typecode, v->typecode, i->typecode, tnd);
  GpuKernel *k;
  auto it = cache.find(key);
  if (it != cache.end()) {
    k = &it->second;
  } else {
    std::vector<int> types;
    std::string s = short_rows ? take1_short_rows_source(i->typecode, types)
                               : take1_source(chunks, a->typecode, v->typecode, i->typecode, tnd, types);
    const char *strs[1] = {s.c_str()};
    size_t lens[1] = {s.size()};
    GpuKernel nk = {nullptr, nullptr};
    int flags = gpuarray_type_flags(a->typecode, v->typecode, i->typecode, -1);
    int err = GpuKernel_init(&nk, ctx, 1, strs, lens, "take1", (unsigned)types.size(), types.data(),
                             flags, nullptr);
    if (err != GA_NO_ERROR) return err;
    k = &cache.emplace(key, nk).first->second;
  }

  gpudata *errbuf = nullptr;
  int err = gpudata_property(v->data, GA_CTX_PROP_ERRBUF, &errbuf);
  if (err != GA_NO_ERROR) return err;
  unsigned int gx32 = (unsigned int)gx, p = 0;
  GpuKernel_setarg(k, p++, a->data);
  GpuKernel_setarg(k, p++, (void *)&a->offset);
  GpuKernel_setarg(k, p++, v->data);
  GpuKernel_setarg(k, p++, (void *)&v->offset);
  GpuKernel_setarg(k, p++, &v->strides[0]);
  GpuKernel_setarg(k, p++, &v->dimensions[0]);
  for (unsigned int d = 0; d < tnd; d++) {
    GpuKernel_setarg(k, p++, &tstr[d]);
    GpuKernel_setarg(k, p++, &tdims[d]);
  }
  GpuKernel_setarg(k, p++, i->data);
  GpuKernel_setarg(k, p++, (void *)&i->offset);
  GpuKernel_setarg(k, p++, &n0);
  GpuKernel_setarg(k, p++, &n1e);
  GpuKernel_setarg(k, p++, &gx32);
  GpuKernel_setarg(k, p++, &lsh);
  GpuKernel_setarg(k, p++, errbuf);
  size_t groups = gx * gy, ls = 256;
  // The error word belongs to the context and is sticky, as in the reference
  // (src/gpuarray_array.c:480, :534-543): a kernel sets it on a bad index
  // whether or not its caller asked for the check, and the next call that does
  // ask reports it and clears it - also when the bad index was an earlier
  // call's.
  err = GpuKernel_call(k, 1, &groups, &ls, 0, nullptr);
  if (check_error && err == GA_NO_ERROR) {
    int kerr = 0;
    err = gpudata_read(&kerr, errbuf, 0, sizeof(int));
    if (err == GA_NO_ERROR && kerr != 0) {
      err = ga_err_set(ctx->err, GA_VALUE_ERROR, "Index out of bounds");
      kerr = 0;
      gpudata_write(errbuf, 0, &kerr, sizeof(int));
    }
  }
  return err;
}

}  // extern "C"
