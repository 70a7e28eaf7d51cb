// GpuReduction: argument checks, iteration-space planning and launch of the
// wave64 reduction kernels; GpuArray_maxandargmax on top of it.
//
// Reference behaviour kept:
//   - GpuArray_maxandargmax argument rules: non-NULL arrays, 1 <= reduxLen <=
//     nd, axes unique and in range, else GA_INVALID_ERROR
//     (src/gpuarray_reduction.c:198-261); destination addressed through its
//     own strides in ascending free-axis order (:504-518, :616-626);
//   - flattened index in reduxList order, strict compare, first index on ties
//     (src/gpuarray/array.h:607-644);
//   - sum/prod/any/all: accumulate in the result's type, neutrals 0/1, any/all
//     test truthiness and give 0/1 (pygpu/reduction.py:83-132,
//     pygpu/_array.py:238-294).
// Reference behaviour replaced: it gives every output to ONE lane that scans
// the reduced axes alone (src/gpuarray_reduction.c:545-607), compiles on every
// call and uploads five small tables per call (:634-667, :790-799); the Python
// sum gives every output to one work-group, so a full reduction is a single
// group (pygpu/reduction.py:256-261).  Here the reduced and free dims are
// sorted by stride and collapsed, lanes run along whichever of the two is
// contiguous in memory, rows that are too few to fill 256 compute units are
// split into partials with a second pass, and kernels are cached per operator.
#include "private.hpp"

#include <algorithm>
#include <map>
#include <mutex>
#include <string>
#include <vector>

namespace {

constexpr int RD_MAXD = 8;

// Must match `struct rd_plan` in reduce_kernels.h.
struct rd_plan {
  int64_t fdim[RD_MAXD], fsstr[RD_MAXD], fd0str[RD_MAXD], fd1str[RD_MAXD];
  int64_t rdim[RD_MAXD], rsstr[RD_MAXD], rmul[RD_MAXD];
  int64_t nrows, rtotal, nseg, units, upb, gx;
  int32_t nf, nr, nsplit, pad;
};

enum rd_kind { K_SUM, K_PROD, K_PRODNZ, K_MIN, K_MAX, K_AND, K_OR, K_XOR, K_ALL, K_ANY };

bool is_float_type(int tc) { return tc == GA_FLOAT || tc == GA_DOUBLE || tc == GA_HALF; }
bool is_int_type(int tc) { return tc >= GA_BOOL && tc <= GA_ULONG; }

unsigned long env_ul(const char *name, unsigned long dflt) {
  const char *v = getenv(name);
  if (v == nullptr || *v == 0) return dflt;
  char *end = nullptr;
  unsigned long r = strtoul(v, &end, 10);
  return end == v ? dflt : r;
}

struct op_info {
  rd_kind kind;
  bool has_d0, has_d1;
};

bool op_lookup(ga_reduce_op op, op_info *o) {
  switch (op) {
  case GA_REDUCE_SUM: *o = {K_SUM, true, false}; return true;
  case GA_REDUCE_PROD: *o = {K_PROD, true, false}; return true;
  case GA_REDUCE_PRODNZ: *o = {K_PRODNZ, true, false}; return true;
  case GA_REDUCE_MIN: *o = {K_MIN, true, false}; return true;
  case GA_REDUCE_MAX: *o = {K_MAX, true, false}; return true;
  case GA_REDUCE_ARGMIN: *o = {K_MIN, false, true}; return true;
  case GA_REDUCE_ARGMAX: *o = {K_MAX, false, true}; return true;
  case GA_REDUCE_MINANDARGMIN: *o = {K_MIN, true, true}; return true;
  case GA_REDUCE_MAXANDARGMAX: *o = {K_MAX, true, true}; return true;
  case GA_REDUCE_AND: *o = {K_AND, true, false}; return true;
  case GA_REDUCE_OR: *o = {K_OR, true, false}; return true;
  case GA_REDUCE_XOR: *o = {K_XOR, true, false}; return true;
  case GA_REDUCE_ALL: *o = {K_ALL, true, false}; return true;
  case GA_REDUCE_ANY: *o = {K_ANY, true, false}; return true;
  default: return false;
  }
}

// Device spelling of an accumulator for results of type tc.  Integer sums and
// products run in the unsigned type of the same width: wrap-around is then
// defined, and the bits are those of the signed result.
const char *acc_type_for(int tc, rd_kind kind) {
  const bool arith = kind == K_SUM || kind == K_PROD || kind == K_PRODNZ;
  switch (tc) {
  case GA_BOOL: case GA_UBYTE: case GA_USHORT: case GA_UINT: return "ga_uint";
  case GA_BYTE: case GA_SHORT: case GA_INT: return arith ? "ga_uint" : "ga_int";
  case GA_LONG: return arith ? "ga_ulong" : "ga_long";
  case GA_ULONG: return "ga_ulong";
  case GA_HALF: case GA_FLOAT: return "ga_float";
  case GA_DOUBLE: return "ga_double";
  default: return nullptr;
  }
}
size_t acc_size_for(int tc) { return (tc == GA_LONG || tc == GA_ULONG || tc == GA_DOUBLE) ? 8 : 4; }

std::string neutral_for(rd_kind kind, int acc_tc) {
  switch (kind) {
  case K_SUM: case K_OR: case K_XOR: case K_ANY: return "0";
  case K_PROD: case K_PRODNZ: case K_ALL: return "1";
  case K_AND: return "(~(RD_ACC_T)0)";
  case K_MAX:
    switch (acc_tc) {
    case GA_HALF: case GA_FLOAT: case GA_DOUBLE: return "(-INFINITY)";
    case GA_BYTE: case GA_SHORT: case GA_INT: return "(-2147483647 - 1)";
    case GA_LONG: return "(-9223372036854775807LL - 1)";
    default: return "0";
    }
  case K_MIN:
    switch (acc_tc) {
    case GA_HALF: case GA_FLOAT: case GA_DOUBLE: return "INFINITY";
    case GA_BYTE: case GA_SHORT: case GA_INT: return "2147483647";
    case GA_LONG: return "9223372036854775807LL";
    case GA_ULONG: return "18446744073709551615ULL";
    default: return "4294967295u";
    }
  }
  return "0";
}

struct variant {
  GpuKernel row = {nullptr, nullptr}, col = {nullptr, nullptr}, fin = {nullptr, nullptr},
            wrows = {nullptr, nullptr};   // wrows only exists in 64-lane variants
};

struct dimrec {
  int64_t dim, s, a, b;   // extent, source stride, (d0 stride | index multiplier), d1 stride
};

inline int64_t iabs(int64_t v) { return v < 0 ? -v : v; }

}  // namespace

struct _GpuReduction {
  gpucontext *ctx;
  ga_reduce_op op;
  op_info info;
  int src_tc;
  std::map<std::string, variant> variants;
};

int ga_plan_typecode(size_t bytes) {
  static std::mutex mu;
  static std::map<size_t, gpuarray_type *> reg;
  std::lock_guard<std::mutex> lk(mu);
  auto it = reg.find(bytes);
  if (it != reg.end()) return it->second->typecode;
  gpuarray_type *t = new gpuarray_type{"ga_plan", bytes, 8, 0};
  int tc = gpuarray_register_type(t, nullptr);
  reg[bytes] = t;
  return tc;
}

namespace {

// The #define block that specialises reduce_kernels.h.
int gen_defines(const op_info &info, int src_tc, int d0_tc, int d1_tc, unsigned G, unsigned V,
                unsigned U, std::string &s, ga_errrec *errrec, unsigned opts = 3,
                unsigned ES = 1) {
  const rd_kind kind = info.kind;
  const bool minmax = kind == K_MIN || kind == K_MAX;
  // min/max compare in the source's type; everything else in the result's
  const int acc_tc = minmax ? src_tc : d0_tc;
  const char *acc_t = kind == K_ALL || kind == K_ANY ? "ga_uint" : acc_type_for(acc_tc, kind);
  if (acc_t == nullptr)
    return ga_err_fmt(errrec, GA_UNSUPPORTED_ERROR, "No accumulator for typecode %d", acc_tc);
  const bool srcf = is_float_type(src_tc);
  // floating min/max track the index even when it is not returned: the
  // lowest-index rule is what makes -0.0 / +0.0 come out as in a sequential scan
  const bool arg = info.has_d1 || (minmax && srcf);
  char line[256];
#define DEF(...) do { snprintf(line, sizeof(line), __VA_ARGS__); s += line; } while (0)
  DEF("#define RD_SRC_T %s\n", src_tc == GA_HALF ? "ga_ushort" : gpuarray_get_type(src_tc)->cluda_name);
  DEF("#define RD_SRC_HALF %d\n", src_tc == GA_HALF ? 1 : 0);
  DEF("#define RD_ACC_T %s\n", acc_t);
  DEF("#define RD_DST_T %s\n", info.has_d0 ? gpuarray_get_type(d0_tc)->cluda_name : "ga_int");
  DEF("#define RD_DST_HALF %d\n", info.has_d0 && d0_tc == GA_HALF ? 1 : 0);
  DEF("#define RD_IDX_T %s\n", info.has_d1 ? gpuarray_get_type(d1_tc)->cluda_name : "ga_long");
  DEF("#define RD_KIND %d\n", (int)kind);
  DEF("#define RD_ARG %d\n", arg ? 1 : 0);
  DEF("#define RD_HAS_D0 %d\n#define RD_HAS_D1 %d\n", info.has_d0 ? 1 : 0, info.has_d1 ? 1 : 0);
  DEF("#define RD_FLT %d\n", srcf ? 1 : 0);
  DEF("#define RD_NEUTRAL ((RD_ACC_T)%s)\n",
      neutral_for(kind, kind == K_ALL || kind == K_ANY ? GA_UINT : acc_tc).c_str());
  DEF("#define RD_G %u\n#define RD_VEC %u\n#define RD_U %u\n", G, V, U);
  DEF("#define RD_NT %u\n#define RD_INTERLEAVE %u\n#define RD_ES %u\n", opts & 1u,
      (opts >> 1) & 1u, ES);
#undef DEF
  return GA_NO_ERROR;
}

int get_variant(GpuReduction *gr, int d0_tc, int d1_tc, unsigned G, unsigned V, unsigned U,
                unsigned opts, unsigned ES, variant **out) {
  gpucontext *ctx = gr->ctx;
  char key[96];
  snprintf(key, sizeof(key), "%d:%d:%u:%u:%u:%u:%u", d0_tc, d1_tc, G, V, U, opts, ES);
  auto it = gr->variants.find(key);
  if (it != gr->variants.end()) {
    *out = &it->second;
    return GA_NO_ERROR;
  }
  std::string s;
  int herr = gen_defines(gr->info, gr->src_tc, d0_tc, d1_tc, G, V, U, s, ctx->err, opts, ES);
  if (herr != GA_NO_ERROR) return herr;
  const char *strs[2] = {s.c_str(), ga_reduce_kernels_src};
  size_t lens[2] = {s.size(), strlen(ga_reduce_kernels_src)};
  const int plan_tc = ga_plan_typecode(sizeof(rd_plan));
  const int types[9] = {GA_BUFFER, GA_SIZE, GA_BUFFER, GA_SIZE, GA_BUFFER,
                        GA_SIZE,   GA_BUFFER, GA_BUFFER, plan_tc};
  const int kflags = gpuarray_type_flags(gr->src_tc, d0_tc, -1);
  variant v;
  int err;
  if ((err = GpuKernel_init(&v.row, ctx, 2, strs, lens, "redux_row", 9, types, kflags, nullptr)) != GA_NO_ERROR)
    return err;
  if ((err = GpuKernel_init(&v.col, ctx, 2, strs, lens, "redux_col", 9, types, kflags, nullptr)) != GA_NO_ERROR) {
    GpuKernel_clear(&v.row);
    return err;
  }
  if ((err = GpuKernel_init(&v.fin, ctx, 2, strs, lens, "redux_final", 9, types, kflags, nullptr)) != GA_NO_ERROR) {
    GpuKernel_clear(&v.row);
    GpuKernel_clear(&v.col);
    return err;
  }
  if (G == 64 &&
      (err = GpuKernel_init(&v.wrows, ctx, 2, strs, lens, "redux_wrows", 9, types, kflags, nullptr)) != GA_NO_ERROR) {
    GpuKernel_clear(&v.row);
    GpuKernel_clear(&v.col);
    GpuKernel_clear(&v.fin);
    return err;
  }
  *out = &gr->variants.emplace(key, v).first->second;
  return GA_NO_ERROR;
}

// Sort slowest-stride first, then fuse neighbours that every listed stride
// walks as one run.
void sort_and_fuse(std::vector<dimrec> &v, bool use_b) {
  std::stable_sort(v.begin(), v.end(),
                   [](const dimrec &x, const dimrec &y) { return iabs(x.s) > iabs(y.s); });
  for (size_t i = v.size(); i-- > 1;) {
    const dimrec &in = v[i];
    dimrec &out = v[i - 1];
    if (out.s == in.dim * in.s && out.a == in.dim * in.a && (!use_b || out.b == in.dim * in.b)) {
      out.dim *= in.dim;
      out.s = in.s;
      out.a = in.a;
      out.b = in.b;
      v.erase(v.begin() + (long)i);
    }
  }
}

}  // namespace

extern "C" {

// Full kernel text of one variant, for checks that have no device.  The
// caller frees the result.
GPUARRAY_PUBLIC char *ga_reduction_gen_source(int op, int src_tc, int d0_tc, int d1_tc,
                                              unsigned int G, unsigned int V, unsigned int U) {
  op_info info;
  if (!op_lookup((ga_reduce_op)op, &info)) return nullptr;
  // bits 8.. of V carry the element step of strided loads (0 means 1)
  const unsigned ES = (V >> 8) ? (V >> 8) : 1;
  V &= 0xffu;
  std::string s;
  if (gen_defines(info, src_tc, d0_tc, d1_tc, G, V, U, s, ga_global_err, 3, ES) != GA_NO_ERROR)
    return nullptr;
  s += ga_reduce_kernels_src;
  return strdup(s.c_str());
}

int GpuReduction_new(GpuReduction **grp, gpucontext *ctx, ga_reduce_op op, unsigned ndf,
                     unsigned ndr, int s0Typecode, int flags) {
  (void)ndf; (void)ndr; (void)flags;
  if (grp == nullptr) return GA_INVALID_ERROR;
  *grp = nullptr;
  if (ctx == nullptr) return ga_err_set(ga_global_err, GA_INVALID_ERROR, "GpuReduction_new: no context");
  op_info info;
  if (!op_lookup(op, &info))
    return ga_err_fmt(ctx->err, GA_INVALID_ERROR, "Unknown reduction operation %d", (int)op);
  if (!is_int_type(s0Typecode) && !is_float_type(s0Typecode))
    return ga_err_fmt(ctx->err, GA_UNSUPPORTED_ERROR, "Reductions over typecode %d are not supported",
                      s0Typecode);
  if ((info.kind == K_AND || info.kind == K_OR || info.kind == K_XOR) && !is_int_type(s0Typecode))
    return ga_err_set(ctx->err, GA_UNSUPPORTED_ERROR, "Bitwise reductions need an integer source");
  GpuReduction *gr = new (std::nothrow) GpuReduction();
  if (gr == nullptr) return ga_err_set(ctx->err, GA_MEMORY_ERROR, "Out of memory");
  gr->ctx = ctx;
  gr->op = op;
  gr->info = info;
  gr->src_tc = s0Typecode;
  *grp = gr;
  return GA_NO_ERROR;
}

void GpuReduction_free(GpuReduction *gr) {
  if (gr == nullptr) return;
  for (auto &kv : gr->variants) {
    GpuKernel_clear(&kv.second.row);
    GpuKernel_clear(&kv.second.col);
    GpuKernel_clear(&kv.second.fin);
    if (kv.second.wrows.k != nullptr) GpuKernel_clear(&kv.second.wrows);
  }
  delete gr;
}

int GpuReduction_call(const GpuReduction *cgr, GpuArray *d0, GpuArray *d1, const GpuArray *s0,
                      unsigned reduxLen, const int *reduxList, int flags) {
  (void)flags;
  GpuReduction *gr = const_cast<GpuReduction *>(cgr);
  if (gr == nullptr || s0 == nullptr) return GA_INVALID_ERROR;
  gpucontext *ctx = gr->ctx;
  const op_info &info = gr->info;
  if ((info.has_d0 && d0 == nullptr) || (info.has_d1 && d1 == nullptr))
    return ga_err_set(ctx->err, GA_INVALID_ERROR, "A destination array required by the operation is NULL");
  if (!info.has_d0) d0 = nullptr;
  if (!info.has_d1) d1 = nullptr;
  if (s0->nd == 0 || reduxLen == 0 || reduxLen > s0->nd || reduxList == nullptr)
    return ga_err_fmt(ctx->err, GA_INVALID_ERROR,
                      "Invalid reduction: source nd = %u, %u axes to reduce", s0->nd, reduxLen);
  const unsigned nd = s0->nd;
  std::vector<char> reduced(nd, 0);
  for (unsigned i = 0; i < reduxLen; i++) {
    const int ax = reduxList[i];
    if (ax < 0 || ax >= (int)nd || reduced[ax])
      return ga_err_fmt(ctx->err, GA_INVALID_ERROR, "Reduction axis %d is out of range or repeated", ax);
    reduced[ax] = 1;
  }
  if (s0->typecode != gr->src_tc)
    return ga_err_fmt(ctx->err, GA_VALUE_ERROR, "Source has typecode %d, operator was made for %d",
                      s0->typecode, gr->src_tc);
  if (GpuArray_context(s0) != ctx || (d0 && GpuArray_context(d0) != ctx) ||
      (d1 && GpuArray_context(d1) != ctx))
    return ga_err_set(ctx->err, GA_VALUE_ERROR, "Arrays belong to another context");

  // result types
  const rd_kind kind = info.kind;
  const bool minmax = kind == K_MIN || kind == K_MAX;
  int d0_tc = d0 ? d0->typecode : gr->src_tc, d1_tc = d1 ? d1->typecode : GA_LONG;
  if (d0) {
    if (!GpuArray_ISWRITEABLE(d0)) return ga_err_set(ctx->err, GA_VALUE_ERROR, "Destination not writeable");
    if (minmax && d0_tc != gr->src_tc)
      return ga_err_set(ctx->err, GA_VALUE_ERROR, "min/max results must have the source's type");
    if ((kind == K_AND || kind == K_OR || kind == K_XOR || kind == K_ALL || kind == K_ANY) &&
        !is_int_type(d0_tc))
      return ga_err_set(ctx->err, GA_VALUE_ERROR, "Result of a logical/bitwise reduction must be an integer type");
    if (!is_int_type(d0_tc) && !is_float_type(d0_tc))
      return ga_err_fmt(ctx->err, GA_UNSUPPORTED_ERROR, "Result typecode %d is not supported", d0_tc);
  }
  if (d1) {
    if (!GpuArray_ISWRITEABLE(d1)) return ga_err_set(ctx->err, GA_VALUE_ERROR, "Destination not writeable");
    if (d1_tc != GA_LONG && d1_tc != GA_ULONG)
      return ga_err_set(ctx->err, GA_VALUE_ERROR, "Index results must be GA_LONG or GA_ULONG");
  }

  // free axes in ascending order must match the destinations' shapes
  const unsigned nfree = nd - reduxLen;
  for (GpuArray *d : {d0, d1}) {
    if (d == nullptr) continue;
    if (d->nd != nfree)
      return ga_err_fmt(ctx->err, GA_VALUE_ERROR, "Destination has nd = %u, expected %u", d->nd, nfree);
    unsigned k = 0;
    for (unsigned ax = 0; ax < nd; ax++) {
      if (reduced[ax]) continue;
      if (d->dimensions[k] != s0->dimensions[ax])
        return ga_err_fmt(ctx->err, GA_VALUE_ERROR,
                          "Destination dimension %u is %zu, source axis %u is %zu", k,
                          d->dimensions[k], ax, s0->dimensions[ax]);
      k++;
    }
  }

  // dim lists
  std::vector<dimrec> fr, rd;
  int64_t nrows = 1, rtotal = 1;
  {
    unsigned k = 0;
    for (unsigned ax = 0; ax < nd; ax++) {
      if (reduced[ax]) continue;
      const int64_t dim = (int64_t)s0->dimensions[ax];
      nrows *= dim;
      if (dim != 1)
        fr.push_back({dim, (int64_t)s0->strides[ax], d0 ? (int64_t)d0->strides[k] : 0,
                      d1 ? (int64_t)d1->strides[k] : 0});
      k++;
    }
    int64_t mul = 1;
    for (unsigned i = reduxLen; i-- > 0;) {
      const int ax = reduxList[i];
      const int64_t dim = (int64_t)s0->dimensions[ax];
      rtotal *= dim;
      if (dim != 1) rd.insert(rd.begin(), {dim, (int64_t)s0->strides[ax], mul, 0});
      mul *= dim;
    }
  }
  if (nrows == 0) return GA_NO_ERROR;
  if (rtotal == 0 && minmax)
    return ga_err_set(ctx->err, GA_VALUE_ERROR, "min/max over an empty axis has no value");
  if (rtotal == 0) rd.clear();
  sort_and_fuse(fr, true);
  sort_and_fuse(rd, false);
  if (fr.size() > (size_t)RD_MAXD || rd.size() > (size_t)RD_MAXD)
    return ga_err_fmt(ctx->err, GA_UNSUPPORTED_ERROR,
                      "More than %d non-mergeable free or reduced dimensions", RD_MAXD);

  rd_plan p;
  memset(&p, 0, sizeof(p));
  p.nf = (int)fr.size();
  p.nr = (int)rd.size();
  for (int i = 0; i < p.nf; i++) {
    p.fdim[i] = fr[i].dim; p.fsstr[i] = fr[i].s; p.fd0str[i] = fr[i].a; p.fd1str[i] = fr[i].b;
  }
  for (int i = 0; i < p.nr; i++) {
    p.rdim[i] = rd[i].dim; p.rsstr[i] = rd[i].s; p.rmul[i] = rd[i].a;
  }
  p.nrows = nrows;
  p.rtotal = rtotal;
  p.nsplit = 1;

  const int64_t elsz = (int64_t)gpuarray_get_elsize(gr->src_tc);
  const int64_t ncu = (int64_t)ga_hip_numprocs(ctx);
  const int64_t rin = p.nr ? p.rdim[p.nr - 1] : 1;
  const int64_t rstr = p.nr ? iabs(p.rsstr[p.nr - 1]) : 0;
  const int64_t fstr = p.nf ? iabs(p.fsstr[p.nf - 1]) : INT64_MAX;

  // Lanes along the reduced run unless the free run is the one that is
  // contiguous in memory (or the reduced run is too short to feed a wavefront).
  bool use_row = p.nf == 0 || (rstr <= fstr && rin >= 32) || (rin >= 4096 && rstr <= 4 * elsz);
  if (rtotal == 0) use_row = true;
  {
    const char *force = getenv("GPUARRAY_REDUX_FAMILY");
    if (force && strcmp(force, "row") == 0) use_row = true;
    if (force && strcmp(force, "col") == 0 && p.nf > 0) use_row = false;
  }

  unsigned G = 256, V = 1, U = 4, ES = 1;
  bool wrows = false;
  size_t groups;
  if (use_row) {
    // Widest aligned load the layout allows.  The inner reduced dim may step
    // by ES = 1, 2 or 4 elements (a [::2] / [::4] view): a load then fetches
    // V*ES contiguous elements and uses every ES-th one.  Such a load reads up
    // to ES-1 elements past the last one used, so it must stay inside the
    // buffer.
    if (p.nr && rtotal > 0 && p.rsstr[p.nr - 1] > 0 && p.rsstr[p.nr - 1] % elsz == 0) {
      const int64_t es = p.rsstr[p.nr - 1] / elsz;
      if (es == 1 || es == 2 || es == 4) {
        unsigned v = (unsigned)(16 / (elsz * es));
        const uintptr_t base = (uintptr_t)s0->data->devptr + s0->offset;
        size_t bufsz = 0;
        gpudata_property(s0->data, GA_BUFFER_PROP_SIZE, &bufsz);
        int64_t last = (int64_t)s0->offset;   // byte offset of the farthest element
        for (int i = 0; i < p.nf; i++) if (p.fsstr[i] > 0) last += (p.fdim[i] - 1) * p.fsstr[i];
        for (int i = 0; i < p.nr; i++) if (p.rsstr[i] > 0) last += (p.rdim[i] - 1) * p.rsstr[i];
        const bool overread_ok = es == 1 || (size_t)(last + es * elsz) <= bufsz;
        while (v > 1) {
          const int64_t bytes = (int64_t)v * es * elsz;
          bool ok = overread_ok && rin % v == 0 && base % (uintptr_t)bytes == 0;
          for (int i = 0; ok && i < p.nf; i++) ok = p.fsstr[i] % bytes == 0;
          for (int i = 0; ok && i + 1 < p.nr; i++) ok = p.rsstr[i] % bytes == 0;
          if (ok) break;
          v /= 2;
        }
        V = v;
        if (V > 1) ES = (unsigned)es;
      }
    }
    // One wavefront per output when eight loads per lane cover the inner
    // reduced dim, four wavefronts otherwise.  Measured on MI355X: rows of
    // 8192 floats run at 6.7 TB/s with 256 lanes per row and 6.0 with 64;
    // rows of 512 stepped halves at 3.1 TB/s (useful) with 64 and 2.0 with 256.
    G = (rin <= (int64_t)64 * V * 8) ? 64 : 256;
    {
      const unsigned long force = env_ul("GPUARRAY_REDUX_G", 0);
      if (force == 64 || force == 256) G = (unsigned)force;
    }
    int64_t per_pass = (int64_t)G * V;
    U = (unsigned)env_ul("GPUARRAY_REDUX_U", 8);
    if (U != 1 && U != 2 && U != 4 && U != 8) U = 8;
    while (U > 1 && per_pass * (U / 2) >= rin) U /= 2;
    const int64_t seg = per_pass * U;
    p.nseg = rin > 0 ? (rin + seg - 1) / seg : 1;
    if (p.nseg < 1) p.nseg = 1;
    int64_t outer = 1;
    for (int i = 0; i + 1 < p.nr; i++) outer *= p.rdim[i];
    p.units = rtotal > 0 ? outer * p.nseg : 0;
    const int64_t rows_per_group = 256 / G;
    const int64_t rowgroups = (nrows + rows_per_group - 1) / rows_per_group;
    // too few groups to fill the chip: cut the rows
    int64_t nsplit = 1;
    // How many groups a compute unit needs depends on how many bytes each one
    // keeps in flight.  Measured on MI355X (full fp32 sum of 2^28 elements):
    // 2 groups of 256 lanes per unit, each lane with eight 16-byte streaming
    // loads outstanding (64 KB per unit), read at 6.9-7.1 TB/s; 16 such
    // groups per unit at 6.3, 64 at 5.8.  Narrow or strided loads carry fewer
    // bytes per lane, so they get proportionally more groups, up to 32.
    int64_t per_cu = (int64_t)env_ul("GPUARRAY_REDUX_GROUPS_PER_CU", 0);
    if (per_cu == 0) {
      const int64_t inflight = (int64_t)G * U * V * ES * elsz;   // bytes per group
      per_cu = (65536 + inflight - 1) / inflight;
      if (per_cu < 2) per_cu = 2;
      if (per_cu > 32) per_cu = 32;
    }
    const int64_t target = ncu * per_cu;
    if (rowgroups < target && p.units >= 8) {
      nsplit = (target + rowgroups - 1) / rowgroups;
      if (nsplit > p.units / 4) nsplit = p.units / 4;
      if (nsplit > 65536) nsplit = 65536;
      if (nsplit < 1) nsplit = 1;
    }
    p.upb = p.units > 0 ? (p.units + nsplit - 1) / nsplit : 0;
    if (p.upb > 0) nsplit = (p.units + p.upb - 1) / p.upb;
    p.nsplit = (int)nsplit;
    groups = (size_t)(rowgroups * nsplit);
    // Short rows, one wavefront each, take the kernel without the unit loop.
    // It can walk several rows per wavefront with the next row's loads in
    // flight, but on MI355X one row per wavefront measured best (65536 rows
    // of 1000 floats: 43 us with 1 row, 45 / 47 / 52 us with 2 / 4 / 8), so
    // that is the default.
    if (G == 64 && nsplit == 1 && p.units == 1 && p.nr <= 1 && env_ul("GPUARRAY_REDUX_WROWS", 1)) {
      wrows = true;
      int64_t rpw = (int64_t)env_ul("GPUARRAY_REDUX_RPW", 1);
      if (rpw < 1) rpw = 1;
      p.upb = rpw;
      const int64_t waves = (nrows + rpw - 1) / rpw;
      groups = (size_t)((waves + 3) / 4);
    }
  } else {
    const int64_t fin = p.fdim[p.nf - 1];
    p.gx = (fin + 63) / 64;
    const int64_t outer = nrows / fin;
    const int64_t base_groups = p.gx * outer;
    int64_t nsplit = 1;
    const int64_t target = ncu * (int64_t)env_ul("GPUARRAY_REDUX_GROUPS_PER_CU", 8);
    if (base_groups < target && rtotal >= 256) {
      nsplit = (target + base_groups - 1) / base_groups;
      if (nsplit > rtotal / 64) nsplit = rtotal / 64;
      if (nsplit > 4096) nsplit = 4096;
      if (nsplit < 1) nsplit = 1;
    }
    p.upb = (rtotal + nsplit - 1) / nsplit;
    if (p.upb > 0) nsplit = (rtotal + p.upb - 1) / p.upb;
    p.nsplit = (int)nsplit;
    groups = (size_t)(base_groups * nsplit);
    U = 4;
  }
  if (groups == 0 || groups > 0x7fffffffull)
    return ga_err_set(ctx->err, GA_XLARGE_ERROR, "Reduction needs more groups than one launch has");

  // bit 0: streaming loads; bit 1: interleaved splits (single reduced dim only)
  unsigned opts = env_ul("GPUARRAY_REDUX_NT", 1) ? 1u : 0u;
  if (use_row && p.nr == 1 && p.nsplit > 1 && env_ul("GPUARRAY_REDUX_INTERLEAVE", 1)) opts |= 2u;
  variant *var = nullptr;
  int err = get_variant(gr, d0_tc, d1_tc, use_row ? G : 256, use_row ? V : 1, U, opts,
                        use_row ? ES : 1, &var);
  if (err != GA_NO_ERROR) return err;

  // partials of a split reduction live in the context's scratch buffer:
  // values first, indices after, both 8-byte aligned
  const size_t accsz = (kind == K_ALL || kind == K_ANY) ? 4 : acc_size_for(minmax ? gr->src_tc : d0_tc);
  gpudata *scratch = ga_hip_scratch(ctx, 16);
  size_t pv_off = 0, pi_off = 0;
  if (p.nsplit > 1) {
    const size_t slots = (size_t)nrows * (size_t)p.nsplit;
    pi_off = (slots * accsz + 255) & ~(size_t)255;
    scratch = ga_hip_scratch(ctx, pi_off + slots * 8);
  }
  if (scratch == nullptr) return ctx->err->code;
  (void)pv_off;

  // A destination the operation does not write still needs a valid pointer.
  gpudata *d0b = d0 ? d0->data : scratch, *d1b = d1 ? d1->data : scratch;
  size_t s_off = s0->offset, d0_off = d0 ? d0->offset : 0, d1_off = d1 ? d1->offset : 0;

  // The two scratch views are passed as (buffer) arguments; the index part
  // starts pi_off bytes in, which the kernels receive through a second
  // gpudata wrapping the same memory.
  struct { void *devptr; gpucontext *ctx; } pi_view = {(char *)scratch->devptr + pi_off, ctx};
  void *args[9] = {s0->data, &s_off, d0b, &d0_off, d1b, &d1_off, scratch, &pi_view, &p};
  size_t ls = 256;
  GpuKernel *k1 = use_row ? (wrows ? &var->wrows : &var->row) : &var->col;
  if ((err = GpuKernel_call(k1, 1, &groups, &ls, 0, args)) != GA_NO_ERROR) return err;
  if (p.nsplit > 1) {
    size_t fg = (size_t)((nrows + 3) / 4);
    if ((err = GpuKernel_call(&var->fin, 1, &fg, &ls, 0, args)) != GA_NO_ERROR) return err;
  }
  return GA_NO_ERROR;
}

// Reference entry point (src/gpuarray_reduction.c:100-124).  The operator is
// cached per context and source type, so repeated calls compile nothing.
int GpuArray_maxandargmax(GpuArray *dstMax, GpuArray *dstArgmax, const GpuArray *src,
                          unsigned reduxLen, const unsigned *reduxList) {
  if (dstMax == nullptr || dstArgmax == nullptr || src == nullptr || src->nd == 0 ||
      reduxLen == 0 || reduxLen > src->nd || reduxList == nullptr)
    return GA_INVALID_ERROR;
  gpucontext *ctx = GpuArray_context(src);
  if (ctx == nullptr) return GA_INVALID_ERROR;
  typedef std::map<int, GpuReduction *> cache_t;
  void **slot = ga_hip_redux_cache_slot(ctx);
  if (*slot == nullptr) *slot = new cache_t();
  cache_t &cache = *(cache_t *)*slot;
  GpuReduction *gr = nullptr;
  auto it = cache.find(src->typecode);
  if (it != cache.end()) {
    gr = it->second;
  } else {
    int err = GpuReduction_new(&gr, ctx, GA_REDUCE_MAXANDARGMAX, src->nd - reduxLen, reduxLen,
                               src->typecode, 0);
    if (err != GA_NO_ERROR) return err;
    cache[src->typecode] = gr;
  }
  std::vector<int> axes(reduxList, reduxList + reduxLen);
  return GpuReduction_call(gr, dstMax, dstArgmax, src, reduxLen, axes.data(), 0);
}

}  // extern "C"

void ga_redux_cache_free(gpucontext *ctx) {
  typedef std::map<int, GpuReduction *> cache_t;
  void **slot = ga_hip_redux_cache_slot(ctx);
  if (*slot == nullptr) return;
  cache_t *cache = (cache_t *)*slot;
  *slot = nullptr;
  for (auto &kv : *cache) GpuReduction_free(kv.second);
  delete cache;
}
