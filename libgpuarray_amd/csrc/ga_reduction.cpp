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
#include <array>
#include <cctype>
#include <cmath>
#include <map>
#include <mutex>
#include <string>
#include <vector>

namespace {

constexpr int RD_MAXD = 8;

constexpr unsigned RD_MAXSRC = 8;

// Must match `struct rd_plan` in reduce_kernels.h: this fixed part, then the
// sources' free strides [nsrc][RD_MAXD] and reduced strides [nsrc][RD_MAXD].
struct rd_plan {
  int64_t fdim[RD_MAXD], fd0str[RD_MAXD], fd1str[RD_MAXD];
  int64_t rdim[RD_MAXD], rmul[RD_MAXD];
  int64_t nrows, rtotal, nseg, units, upb, gx, router;
  int32_t nf, nr, nsplit, split_major;
  int32_t rising, fused;
};

enum rd_kind { K_SUM, K_PROD, K_PRODNZ, K_MIN, K_MAX, K_AND, K_OR, K_XOR, K_ALL, K_ANY, K_CUSTOM };

bool is_float_type(int tc) { return tc == GA_FLOAT || tc == GA_DOUBLE || tc == GA_HALF; }
bool is_int_type(int tc) { return tc >= GA_BOOL && tc <= GA_ULONG; }


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
  case GA_REDUCE_CUSTOM: *o = {K_CUSTOM, true, false}; return true;
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
  case K_CUSTOM: break;
  }
  return "0";
}

struct variant {
  GpuKernel row = {nullptr, nullptr}, col = {nullptr, nullptr}, fin = {nullptr, nullptr},
            fin_cols = {nullptr, nullptr},   // second pass after redux_col
            wrows = {nullptr, nullptr},   // wrows only exists in 64-lane variants
            srows = {nullptr, nullptr},   // the only kernel of a short-rows variant (opts bit 3)
            trows = {nullptr, nullptr},   // the only kernel of a tiny-rows variant (opts bit 10)
            pcols = {nullptr, nullptr};   // the only kernel of a short-kept-rows variant (opts bit 11)
};

struct dimrec {
  int64_t dim, s[RD_MAXSRC], a, b;   // extent, source strides, (d0 stride | index multiplier), d1 stride
  int64_t smax;                      // largest |source stride|: the sort key
};

// What the launches of a planned call need besides the plan itself.
struct launch_rec {
  GpuKernel *k1 = nullptr, *k2 = nullptr;   // first launch; second pass of a split reduction, or NULL
  size_t groups = 0, fin_groups = 0, lds_bytes = 0;
  size_t pi_off = 0, need = 0;   // partials of a split reduction: offset of the indices, bytes in all
  bool fused = false;            // the first launch finishes the reduction itself (counters)
  bool remember = true;          // false: planned under a passing condition, plan again next time
};

// A planned call kept with its operator.  The key lists every input of the
// planners: extents, axes, the layout of every array (strides, offset,
// alignment of the base address, flags, type), the sizes of the sources'
// buffers, the tuning table's generation, the scratch arrangement.  A call
// whose key equals a kept one launches with the kept plan.
constexpr unsigned MEMO_KEYMAX = 160, MEMO_ENTRIES = 4;
struct call_memo {
  unsigned nkey = 0;
  int64_t key[MEMO_KEYMAX];
  std::vector<int64_t> plan;
  launch_rec rec;
};

struct rd_arg {
  std::string name;
  int tc;
  bool scalar;
};

inline int64_t iabs(int64_t v) { return v < 0 ? -v : v; }

}  // namespace

struct _GpuReduction {
  gpucontext *ctx;
  ga_reduce_op op;
  op_info info;
  // Arguments in the caller's order.  A plain reduction has one array
  // argument and the identity as its expression.
  std::vector<rd_arg> args;
  std::vector<unsigned> arrays, scalars;   // positions in args
  bool mapped = false;        // an expression feeds the reduction
  int acc_tc = -1;            // mapped: accumulator (= value result) type
  std::string map_expr, preamble, reduce_expr, neutral;
  std::map<std::array<unsigned, 14>, variant> variants;   // by the fields of a variant_spec
  // the same operation on the type of folded partial results (see fold_rows), made on first use
  GpuReduction *fold_op = nullptr;
  int fold_tc = -1;
  // (row count, row bytes, widest fold) -> rows per folded row, 0 = no fold
  std::map<std::array<size_t, 3>, size_t> fold_memo;
  // planned calls, and the entry the next new plan replaces once all are taken
  std::vector<call_memo> memo;
  unsigned memo_next = 0;
  int src_tc() const { return args[arrays[0]].tc; }
  unsigned nsrc() const { return (unsigned)arrays.size(); }
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

// What a variant of the kernels is specialised on besides the operator.
struct variant_spec {
  int d0_tc, d1_tc;
  unsigned G, V, U, opts, ES;
  unsigned vecmask;   // bit k: array source k is fetched with vector loads
  unsigned RB;        // redux_wrows: rows per batch of loads
  unsigned L;         // redux_wrows: lanes per row
  unsigned CV;        // redux_col: adjacent outputs per lane
  unsigned LO;        // redux_row: outer reduced coordinates side by side
  unsigned CY = 4;    // redux_col: lane rows of a group (1 to 16), 256 / CY lanes along the free dim
  unsigned TE = 0;    // redux_trows (opts bit 10): elements of a row
};

const char *load_type_name(int tc) {
  return tc == GA_HALF ? "ga_ushort" : gpuarray_get_type(tc)->cluda_name;
}
const char *value_type_name(int tc) {
  return tc == GA_HALF ? "ga_float" : gpuarray_get_type(tc)->cluda_name;
}

// Accumulator type of the operator for a value result of type d0_tc.
int acc_typecode(const GpuReduction *gr, int d0_tc) {
  const rd_kind kind = gr->info.kind;
  if (gr->mapped) return gr->acc_tc;
  // min/max compare in the source's type; everything else in the result's
  return (kind == K_MIN || kind == K_MAX) ? gr->src_tc() : d0_tc;
}

// One-byte elements of a vector-loaded source are kept packed in 32-bit words
// when a load holds whole words.
bool packed_bytes(int tc, const variant_spec &vs) {
  return gpuarray_get_elsize(tc) == 1 && (vs.V * vs.ES) % 4 == 0;
}

// The text that specialises reduce_kernels.h: `defs` goes in front of it,
// `gen` replaces its @RD_GENERATED@ mark.
int gen_variant_text(const GpuReduction *gr, const variant_spec &vs, std::string &defs,
                     std::string &gen, ga_errrec *errrec) {
  const ga_tuning *tn = ga_hip_tuning(gr->ctx);
  const op_info &info = gr->info;
  const rd_kind kind = info.kind;
  const bool minmax = kind == K_MIN || kind == K_MAX;
  const int acc_tc = acc_typecode(gr, vs.d0_tc);
  const char *acc_t;
  if (kind == K_ALL || kind == K_ANY) acc_t = "ga_uint";
  else if (kind == K_CUSTOM) acc_t = value_type_name(acc_tc);
  else acc_t = acc_type_for(acc_tc, kind);
  if (acc_t == nullptr)
    return ga_err_fmt(errrec, GA_UNSUPPORTED_ERROR, "No accumulator for typecode %d", acc_tc);
  const bool valf = is_float_type(acc_tc);
  // floating min/max track the index even when it is not returned: the
  // lowest-index rule is what makes -0.0 / +0.0 come out as in a sequential scan
  const bool arg = info.has_d1 || (minmax && valf);
  const unsigned K = gr->nsrc();
  char line[512];
#define DEF(...) do { snprintf(line, sizeof(line), __VA_ARGS__); defs += line; } while (0)
  DEF("#define RD_NSRC %u\n", K);
  DEF("#define RD_ACC_T %s\n", acc_t);
  DEF("#define RD_DST_T %s\n", info.has_d0 ? gpuarray_get_type(vs.d0_tc)->cluda_name : "ga_int");
  DEF("#define RD_DST_HALF %d\n", info.has_d0 && vs.d0_tc == GA_HALF ? 1 : 0);
  DEF("#define RD_IDX_T %s\n", info.has_d1 ? gpuarray_get_type(vs.d1_tc)->cluda_name : "ga_long");
  DEF("#define RD_KIND %d\n", (int)kind);
  DEF("#define RD_ARG %d\n", arg ? 1 : 0);
  DEF("#define RD_HAS_D0 %d\n#define RD_HAS_D1 %d\n", info.has_d0 ? 1 : 0, info.has_d1 ? 1 : 0);
  DEF("#define RD_FLT %d\n", valf ? 1 : 0);
  if (kind == K_CUSTOM) {
    defs += "#define RD_NEUTRAL ((RD_ACC_T)(" + gr->neutral + "))\n";
    defs += "#define RD_CUSTOM_OP(a, b) (" + gr->reduce_expr + ")\n";
  } else {
    DEF("#define RD_NEUTRAL ((RD_ACC_T)%s)\n",
        neutral_for(kind, kind == K_ALL || kind == K_ANY ? GA_UINT : acc_tc).c_str());
  }
  DEF("#define RD_G %u\n#define RD_VEC %u\n#define RD_U %u\n", vs.G, vs.V, vs.U);
  DEF("#define RD_NT %u\n#define RD_INTERLEAVE %u\n#define RD_ES %u\n#define RD_RB %u\n",
      vs.opts & 1u, (vs.opts >> 1) & 1u, vs.ES, vs.RB ? vs.RB : 1u);
  DEF("#define RD_L %u\n#define RD_CV %u\n#define RD_LO %u\n", vs.L ? vs.L : 64u,
      vs.CV ? vs.CV : 1u, vs.LO ? vs.LO : 1u);
  DEF("#define RD_TAIL %u\n#define RD_ELSZ0 %u\n", (vs.opts >> 2) & 1u,
      (unsigned)gpuarray_get_elsize(gr->args[gr->arrays[0]].tc));
  DEF("#define RD_SROWS %u\n", (vs.opts >> 3) & 1u);
  DEF("#define RD_PCOLS %u\n", (vs.opts >> 11) & 1u);
  DEF("#define RD_CLOOSE %u\n", (vs.opts >> 12) & 1u);
  DEF("#define RD_XCD %u\n", (vs.opts >> 13) & 1u);
  {
    // redux_trows: a lane's run of whole rows in whole 16-byte chunks
    const unsigned te = vs.TE ? vs.TE : 1;
    const unsigned rowb = te * (unsigned)gpuarray_get_elsize(gr->args[gr->arrays[0]].tc);
    unsigned g = rowb, h = 16;
    while (h) { const unsigned t = g % h; g = h; h = t; }
    DEF("#define RD_TROWS %u\n#define RD_TE %u\n#define RD_TC %u\n#define RD_TR %u\n", (vs.opts >> 10) & 1u,
        te, rowb / g, 16 / g);
  }
  // opts bits 4, 5: redux_row / redux_col; bit 7: redux_wrows in place of redux_row; bit 8: second pass
  DEF("#define RD_WANT %u\n", ((vs.opts & 128u) ? 4u : (vs.opts >> 4) & 1u) | ((vs.opts >> 4) & 2u) |
                                  ((vs.opts & 256u) ? 8u : 0u));
  DEF("#define RD_RISING %u\n", (vs.opts >> 6) & 1u);
  DEF("#define RD_IDX32 %u\n", (vs.opts >> 9) & 1u);
  DEF("#define RD_CY %u\n", vs.CY ? vs.CY : 4u);
  {
    // One-byte elements under sum / any / all with an integer accumulator:
    // the unit is combined four elements per 32-bit operation (RD_FAST8: 1
    // unsigned, 2 signed).  Needs the plain operator on one source fetched
    // with vector loads of whole 32-bit words.
    const int stc = gr->args[gr->arrays[0]].tc;
    const bool bytes = K == 1 && !gr->mapped && gpuarray_get_elsize(stc) == 1 && (vs.vecmask & 1u) &&
                       (vs.V * vs.ES) % 4 == 0 && (vs.ES == 1 || vs.ES == 2 || vs.ES == 4) &&
                       (kind == K_SUM || kind == K_ANY || kind == K_ALL) && !valf &&
                       TUNE(tn, REDUX_FAST8, 1);
    DEF("#define RD_FAST8 %d\n", bytes ? (stc == GA_BYTE ? 2 : 1) : 0);
    // redux_col, any / all over one-byte elements: the words of a lane's load
    // are or-ed whole (all: their zero-byte masks) and taken apart once at
    // the end.
    const unsigned cvn = vs.CV ? vs.CV : 1;
    const bool col_bytes = K == 1 && !gr->mapped && gpuarray_get_elsize(stc) == 1 && cvn % 4 == 0 &&
                           (kind == K_ANY || kind == K_ALL) && TUNE(tn, REDUX_FAST8, 1);
    DEF("#define RD_COL_FAST8 %d\n", col_bytes ? 1 : 0);
  }
  {
    // redux_row: an unconditional use after each unit's loads where the
    // combination puts every use under a branch (see rd_touch)
    bool half_src = false;
    for (unsigned k = 0; k < K; k++) half_src = half_src || gr->args[gr->arrays[k]].tc == GA_HALF;
    // Measured on MI355X, without / with: int32 -> int64 sum of 2^26 elements
    // 76.4 / 47.5 us, int16 rows 50.9 / 43.4, float, double, byte and xor
    // sums the same either way, the two-source dot product 162.5 / 168.7.
    bool touch = K == 1 || kind == K_MIN || kind == K_MAX || kind == K_PRODNZ ||
                 ((vs.opts >> 2) & 1u) || half_src;
    touch = TUNE(tn, REDUX_TOUCH, touch ? 1 : 0) != 0;
    DEF("#define RD_TOUCH_ROW %u\n", touch ? 1u : 0u);
  }
#undef DEF

#define GEN(...) do { snprintf(line, sizeof(line), __VA_ARGS__); gen += line; } while (0)
  // kernel parameters and base pointers of the sources
  gen += "#define RD_SRC_PARAMS ";
  for (unsigned k = 0; k < K; k++)
    GEN("%sconst char *__restrict__ rd_s%u, const ga_size rd_s%u_off", k ? ", " : "", k, k);
  gen += "\n#define RD_SRC_BASES(b) do {";
  for (unsigned k = 0; k < K; k++) GEN(" (b)[%u] = rd_s%u + rd_s%u_off;", k, k, k);
  gen += " } while (0)\n";
  // scalars of the expression
  std::string sp, sa;
  for (unsigned i : gr->scalars) {
    sp += std::string(", const ") + gpuarray_get_type(gr->args[i].tc)->cluda_name + " " + gr->args[i].name;
    sa += ", " + gr->args[i].name;
  }
  gen += "#define RD_SCALAR_PARAMS " + sp + "\n#define RD_SCALAR_FPARAMS " + sp +
         "\n#define RD_SCALAR_ARGS " + sa + "\n";
  // registers of one unit / one element
  std::string unit = "struct rd_unit {", one = "struct rd_one {";
  for (unsigned k = 0; k < K; k++) {
    const int tc = gr->args[gr->arrays[k]].tc;
    const char *lt = load_type_name(tc);
    if (((vs.vecmask >> k) & 1u) && packed_bytes(tc, vs)) {
      // One-byte elements stay packed in 32-bit words; an element is shifted
      // out where it is used.  A vector of bytes would be taken apart right
      // after each load, which makes every load wait for the one before it.
      GEN("typedef ga_uint rd_pvec%u_t __attribute__((ext_vector_type(RD_PV / 4)));\n", k);
      snprintf(line, sizeof(line), " rd_pvec%u_t x%u[RD_U];", k, k);
    } else if ((vs.vecmask >> k) & 1u) {
      GEN("typedef %s rd_pvec%u_t __attribute__((ext_vector_type(RD_PV)));\n", lt, k);
      snprintf(line, sizeof(line), " rd_pvec%u_t x%u[RD_U];", k, k);
    } else {
      snprintf(line, sizeof(line), " %s x%u[RD_U][RD_VEC];", lt, k);
    }
    unit += line;
    snprintf(line, sizeof(line), " %s x%u;", lt, k);
    one += line;
    // raw loaded bits -> the value the expression sees (half widens to float)
    if (tc == GA_HALF)
      GEN("static __device__ inline ga_float rd_w%u(const ga_ushort r) { ga_half h; h.data = r; "
          "return ga_half2float(h); }\n", k);
    else
      GEN("static __device__ inline %s rd_w%u(const %s r) { return r; }\n", lt, k, lt);
  }
  gen += unit + " };\n" + one + " };\n";
  // the expression
  if (!gr->preamble.empty()) gen += gr->preamble + "\n";
  gen += "static __device__ inline auto rd_map(";
  for (unsigned k = 0; k < K; k++) {
    const rd_arg &a = gr->args[gr->arrays[k]];
    GEN("%sconst %s %s", k ? ", " : "", value_type_name(a.tc), a.name.c_str());
  }
  gen += " RD_SCALAR_FPARAMS) { return (" + gr->map_expr + "); }\n";
  // loads
  gen += "template <int LN>\nstatic __device__ inline void rd_unit_load(rd_unit &u, const char *const *base, "
         "ga_long e0, ga_long rin, const ga_long *rstr) {\n"
         "_Pragma(\"unroll\")\n"
         "  for (int j = 0; j < RD_U; j++) {\n"
         "    const ga_long e = e0 + (ga_long)j * LN * RD_VEC;\n";
  gen += "    if (e < rin) {\n";
  for (unsigned k = 0; k < K; k++) {
    const char *lt = load_type_name(gr->args[gr->arrays[k]].tc);
    if ((vs.vecmask >> k) & 1u)
      GEN("      u.x%u[j] = RD_LOAD((const rd_pvec%u_t *)(base[%u] + e * rstr[%u]));\n", k, k, k, k);
    else
      GEN("_Pragma(\"unroll\")\n      for (int v = 0; v < RD_VEC; v++) u.x%u[j][v] = "
          "RD_LOAD((const %s *)(base[%u] + (e + v) * rstr[%u]));\n", k, lt, k, k);
  }
  gen += "    }\n  }\n}\n"
         // An unconditional use of every load of the unit, last one first.
         "static __device__ inline void rd_unit_touch(const rd_unit &u) {\n"
         "_Pragma(\"unroll\")\n"
         "  for (int j = RD_U - 1; j >= 0; j--) {\n";
  for (unsigned k = K; k-- > 0;) {
    if ((vs.vecmask >> k) & 1u) GEN("    rd_touch(u.x%u[j][0]);\n", k);
    else GEN("_Pragma(\"unroll\")\n    for (int v = RD_VEC - 1; v >= 0; v--) rd_touch(u.x%u[j][v]);\n", k);
  }
  gen += "  }\n}\n#define RD_UNIT_VAL(u, j, v) rd_map(";
  for (unsigned k = 0; k < K; k++) {
    const int tck = gr->args[gr->arrays[k]].tc;
    if (((vs.vecmask >> k) & 1u) && packed_bytes(tck, vs))
      GEN("%srd_w%u((%s)((u).x%u[j][((v) * RD_ES) / 4] >> (8 * (((v) * RD_ES) %% 4))))", k ? ", " : "", k,
          load_type_name(tck), k);
    else if ((vs.vecmask >> k) & 1u) GEN("%srd_w%u((u).x%u[j][(v) * RD_ES])", k ? ", " : "", k, k);
    else GEN("%srd_w%u((u).x%u[j][v])", k ? ", " : "", k, k);
  }
  gen += " RD_SCALAR_ARGS)\n"
         "static __device__ inline void rd_one_load(rd_one &o, const char *const *p) {\n";
  for (unsigned k = 0; k < K; k++)
    GEN("  o.x%u = RD_LOAD((const %s *)p[%u]);\n", k, load_type_name(gr->args[gr->arrays[k]].tc), k);
  gen += "}\n#define RD_ONE_VAL(o) rd_map(";
  for (unsigned k = 0; k < K; k++) GEN("%srd_w%u((o).x%u)", k ? ", " : "", k, k);
  gen += " RD_SCALAR_ARGS)\n";
  // RD_CV adjacent elements per source (redux_col)
  // One- and two-byte elements stay packed in 32-bit words here too (see the
  // unit registers above); `words` is 0 for a source kept as a vector of its
  // own element type.
  std::vector<unsigned> words(K, 0);
  const unsigned cvn = vs.CV ? vs.CV : 1;
  for (unsigned k = 0; k < K; k++) {
    const int tc = gr->args[gr->arrays[k]].tc;
    const unsigned es = (unsigned)gpuarray_get_elsize(tc);
    if ((es == 1 || es == 2) && (cvn * es) % 4 == 0) words[k] = cvn * es / 4;
    if (words[k] == 1) GEN("typedef ga_uint rd_cv%u_t;\n", k);
    else if (words[k] > 1) GEN("typedef ga_uint rd_cv%u_t __attribute__((ext_vector_type(%u)));\n", k, words[k]);
    else if ((vs.opts >> 12) & 1u)
      GEN("typedef %s rd_cv%u_t __attribute__((ext_vector_type(RD_CV), aligned(%u)));\n", load_type_name(tc), k, es);
    else GEN("typedef %s rd_cv%u_t __attribute__((ext_vector_type(RD_CV)));\n", load_type_name(tc), k);
  }
  gen += "struct rd_cvec {";
  for (unsigned k = 0; k < K; k++) GEN(" rd_cv%u_t x%u;", k, k);
  gen += " };\nstatic __device__ inline void rd_cvec_load(rd_cvec &o, const char *const *p, const int nv) {\n";
  if ((vs.opts >> 12) & 1u) {
    // (the lane at the end of the inner free dim: only its nv first elements exist)
    gen += "  if (nv == RD_CV) {\n";
    for (unsigned k = 0; k < K; k++)
      GEN("    o.x%u = RD_LOAD((const rd_cv%u_t *)p[%u]);\n", k, k, k);
    gen += "  } else {\n#pragma unroll\n    for (int c = 0; c < RD_CV; c++) {\n";
    for (unsigned k = 0; k < K; k++) {
      const char *t = load_type_name(gr->args[gr->arrays[k]].tc);
      GEN("      o.x%u[c] = c < nv ? RD_LOAD((const %s *)p[%u] + c) : (%s)0;\n", k, t, k, t);
    }
    gen += "    }\n  }\n";
  } else {
    gen += "  (void)nv;\n";
    for (unsigned k = 0; k < K; k++)
      GEN("  o.x%u = RD_LOAD((const rd_cv%u_t *)p[%u]);\n", k, k, k);
  }
  gen += "}\n#define RD_CVEC_VAL(o, c) rd_map(";
  for (unsigned k = 0; k < K; k++) {
    const int tc = gr->args[gr->arrays[k]].tc;
    const unsigned es = (unsigned)gpuarray_get_elsize(tc), per = 4 / (es ? es : 4);
    if (words[k] == 1)
      GEN("%srd_w%u((%s)((o).x%u >> (%u * ((c) %% %u))))", k ? ", " : "", k, load_type_name(tc), k,
          8 * es, per);
    else if (words[k] > 1)
      GEN("%srd_w%u((%s)((o).x%u[(c) / %u] >> (%u * ((c) %% %u))))", k ? ", " : "", k,
          load_type_name(tc), k, per, 8 * es, per);
    else
      GEN("%srd_w%u((o).x%u[c])", k ? ", " : "", k, k);
  }
  gen += " RD_SCALAR_ARGS)\n";
  // word d of the first source's packed load (one- and two-byte elements)
  if (words[0] == 1) gen += "#define RD_CVEC_WORD(o, d) ((o).x0)\n";
  else if (words[0] > 1) gen += "#define RD_CVEC_WORD(o, d) ((o).x0[d])\n";
#undef GEN
  return GA_NO_ERROR;
}

// Whole kernel text of a variant.
int variant_source(const GpuReduction *gr, const variant_spec &vs, std::string &out,
                   ga_errrec *errrec) {
  std::string defs, gen;
  int err = gen_variant_text(gr, vs, defs, gen, errrec);
  if (err != GA_NO_ERROR) return err;
  static const char mark[] = "/*@RD_GENERATED@*/";
  const char *at = strstr(ga_reduce_kernels_src, mark);
  if (at == nullptr) return ga_err_set(errrec, GA_IMPL_ERROR, "reduction kernel text has no insertion mark");
  out = defs;
  out.append(ga_reduce_kernels_src, (size_t)(at - ga_reduce_kernels_src));
  out += gen;
  out += at + sizeof(mark) - 1;
  return GA_NO_ERROR;
}

size_t plan_bytes(unsigned nsrc) { return sizeof(rd_plan) + (size_t)nsrc * 2 * RD_MAXD * sizeof(int64_t); }

// `may_build` false: only a variant whose kernels are loaded already will do
// (building one loads a code object, and that allocates device memory).
int get_variant(GpuReduction *gr, const variant_spec &vs, variant **out, bool may_build = true) {
  gpucontext *ctx = gr->ctx;
  const std::array<unsigned, 14> key = {(unsigned)vs.d0_tc, (unsigned)vs.d1_tc, vs.G, vs.V, vs.U,
                                        vs.opts, vs.ES, vs.vecmask, vs.RB, vs.L, vs.CV, vs.LO, vs.CY, vs.TE};
  auto it = gr->variants.find(key);
  if (it != gr->variants.end()) {
    *out = &it->second;
    return GA_NO_ERROR;
  }
  if (!may_build)
    return ga_err_set(ctx->err, GA_UNSUPPORTED_ERROR,
                      "GpuReduction_call_noalloc: the kernels for arrays of this layout are not "
                      "built yet, and building them allocates; run GpuReduction_call once on "
                      "arrays of this layout first");
  std::string s;
  int err = variant_source(gr, vs, s, ctx->err);
  if (err != GA_NO_ERROR) return err;
  const char *strs[1] = {s.c_str()};
  size_t lens[1] = {s.size()};
  // sources (buffer, offset) ..., d0, d0_off, d1, d1_off, part_v, part_i, done, plan, scalars ...
  std::vector<int> types;
  std::vector<int> flag_types;
  for (unsigned k = 0; k < gr->nsrc(); k++) {
    types.push_back(GA_BUFFER);
    types.push_back(GA_SIZE);
    flag_types.push_back(gr->args[gr->arrays[k]].tc);
  }
  for (int t : {GA_BUFFER, GA_SIZE, GA_BUFFER, GA_SIZE, GA_BUFFER, GA_BUFFER, GA_BUFFER}) types.push_back(t);
  types.push_back(ga_plan_typecode(plan_bytes(gr->nsrc())));
  for (unsigned i : gr->scalars) {
    types.push_back(gr->args[i].tc);
    flag_types.push_back(gr->args[i].tc);
  }
  flag_types.push_back(vs.d0_tc);
  if (gr->mapped) flag_types.push_back(gr->acc_tc);
  int kflags = 0;
  for (int t : flag_types) kflags |= gpuarray_type_flags(t, -1);
  const unsigned na = (unsigned)types.size();
  variant v;
  // the text holds only the kernels its calls launch (opts bits 4, 5, 7, 8):
  // a variant is compiled when its first call needs it, and that call waits
  const char *names[6];
  GpuKernel *ks[6];
  int nk = 0;
  auto want = [&](const char *name, GpuKernel *k) { names[nk] = name; ks[nk++] = k; };
  if (vs.opts & 8u) want("redux_srows", &v.srows);
  if (vs.opts & 1024u) want("redux_trows", &v.trows);
  if (vs.opts & 2048u) want("redux_pcols", &v.pcols);
  if (vs.opts & 16u) {
    if (vs.opts & 128u) want("redux_wrows", &v.wrows);
    else want("redux_row", &v.row);
  }
  if (vs.opts & 32u) {
    want("redux_col", &v.col);
    if (vs.opts & 256u) want("redux_final_cols", &v.fin_cols);
  }
  if ((vs.opts & 48u) && (vs.opts & 256u)) want("redux_final", &v.fin);
  for (int i = 0; i < nk; i++) {
    err = GpuKernel_init(ks[i], ctx, 1, strs, lens, names[i], na, types.data(), kflags, nullptr);
    if (err != GA_NO_ERROR) {
      for (int j = 0; j < i; j++) GpuKernel_clear(ks[j]);
      return err;
    }
  }
  *out = &gr->variants.emplace(key, v).first->second;
  return GA_NO_ERROR;
}

// Sort slowest-stride first, then fuse neighbours that every listed stride
// walks as one run.
void sort_and_fuse(std::vector<dimrec> &v, unsigned nsrc, bool use_b) {
  for (dimrec &d : v) {
    d.smax = 0;
    for (unsigned k = 0; k < nsrc; k++) d.smax = std::max(d.smax, iabs(d.s[k]));
  }
  std::stable_sort(v.begin(), v.end(), [](const dimrec &x, const dimrec &y) { return x.smax > y.smax; });
  for (size_t i = v.size(); i-- > 1;) {
    const dimrec &in = v[i];
    dimrec &out = v[i - 1];
    bool ok = out.a == in.dim * in.a && (!use_b || out.b == in.dim * in.b);
    for (unsigned k = 0; ok && k < nsrc; k++) ok = out.s[k] == in.dim * in.s[k];
    if (ok) {
      out.dim *= in.dim;
      for (unsigned k = 0; k < nsrc; k++) out.s[k] = in.s[k];
      out.a = in.a;
      out.b = in.b;
      out.smax = in.smax;
      v.erase(v.begin() + (long)i);
    }
  }
}

bool valid_identifier(const char *s) {
  if (s == nullptr || !(isalpha((unsigned char)*s) || *s == '_')) return false;
  for (const char *c = s; *c; c++)
    if (!(isalnum((unsigned char)*c) || *c == '_')) return false;
  return true;
}

// Builds an operator without touching a device (shared by the constructors and
// by the source generators used for build-time checks).
int make_operator(GpuReduction **grp, gpucontext *ctx, ga_errrec *errrec, ga_reduce_op op,
                  const char *reduce_expr, const char *neutral, int acc_tc, const char *preamble,
                  const char *map_expr, unsigned n, const gpuelemwise_arg *args) {
  op_info info;
  if (!op_lookup(op, &info))
    return ga_err_fmt(errrec, GA_INVALID_ERROR, "Unknown reduction operation %d", (int)op);
  if (info.kind == K_CUSTOM && (reduce_expr == nullptr || neutral == nullptr || *reduce_expr == 0 || *neutral == 0))
    return ga_err_set(errrec, GA_INVALID_ERROR, "A custom reduction needs a combining expression and a neutral element");
  if (map_expr == nullptr || *map_expr == 0 || n == 0 || args == nullptr)
    return ga_err_set(errrec, GA_INVALID_ERROR, "A mapped reduction needs an expression and arguments");
  if (!is_int_type(acc_tc) && !is_float_type(acc_tc))
    return ga_err_fmt(errrec, GA_UNSUPPORTED_ERROR, "Accumulator typecode %d is not supported", acc_tc);
  if ((info.kind == K_AND || info.kind == K_OR || info.kind == K_XOR) && !is_int_type(acc_tc))
    return ga_err_set(errrec, GA_UNSUPPORTED_ERROR, "Bitwise reductions need an integer accumulator");
  GpuReduction *gr = new (std::nothrow) GpuReduction();
  if (gr == nullptr) return ga_err_set(errrec, GA_MEMORY_ERROR, "Out of memory");
  gr->ctx = ctx;
  gr->op = op;
  gr->info = info;
  gr->mapped = true;
  gr->acc_tc = acc_tc;
  gr->map_expr = map_expr;
  gr->preamble = preamble ? preamble : "";
  gr->reduce_expr = reduce_expr ? reduce_expr : "";
  gr->neutral = neutral ? neutral : "";
  int err = GA_NO_ERROR;
  for (unsigned i = 0; i < n && err == GA_NO_ERROR; i++) {
    const gpuelemwise_arg &a = args[i];
    const bool scalar = (a.flags & GE_SCALAR) != 0;
    if (!valid_identifier(a.name))
      err = ga_err_fmt(errrec, GA_VALUE_ERROR, "Argument %u has no valid name", i);
    else if (a.flags & GE_WRITE)
      err = ga_err_fmt(errrec, GA_VALUE_ERROR, "Argument %s: a reduction only reads its arguments", a.name);
    else if (!is_int_type(a.typecode) && !is_float_type(a.typecode))
      err = ga_err_fmt(errrec, GA_UNSUPPORTED_ERROR, "Argument %s: typecode %d is not supported", a.name, a.typecode);
    else if (scalar && a.typecode == GA_HALF)
      err = ga_err_fmt(errrec, GA_UNSUPPORTED_ERROR, "Argument %s: half scalars are not supported", a.name);
    for (unsigned j = 0; j < i && err == GA_NO_ERROR; j++)
      if (gr->args[j].name == a.name)
        err = ga_err_fmt(errrec, GA_VALUE_ERROR, "Argument name %s is used twice", a.name);
    if (err != GA_NO_ERROR) break;
    gr->args.push_back({a.name, a.typecode, scalar});
    (scalar ? gr->scalars : gr->arrays).push_back(i);
  }
  if (err == GA_NO_ERROR && gr->arrays.empty())
    err = ga_err_set(errrec, GA_VALUE_ERROR, "A reduction needs at least one array argument");
  if (err == GA_NO_ERROR && gr->arrays.size() > RD_MAXSRC)
    err = ga_err_fmt(errrec, GA_UNSUPPORTED_ERROR, "More than %u array arguments", RD_MAXSRC);
  if (err != GA_NO_ERROR) {
    delete gr;
    return err;
  }
  *grp = gr;
  return GA_NO_ERROR;
}

int make_plain_operator(GpuReduction **grp, gpucontext *ctx, ga_errrec *errrec, ga_reduce_op op,
                        int s0Typecode) {
  op_info info;
  if (!op_lookup(op, &info) || info.kind == K_CUSTOM)
    return ga_err_fmt(errrec, GA_INVALID_ERROR, "Unknown reduction operation %d", (int)op);
  if (!is_int_type(s0Typecode) && !is_float_type(s0Typecode))
    return ga_err_fmt(errrec, GA_UNSUPPORTED_ERROR, "Reductions over typecode %d are not supported",
                      s0Typecode);
  if ((info.kind == K_AND || info.kind == K_OR || info.kind == K_XOR) && !is_int_type(s0Typecode))
    return ga_err_set(errrec, GA_UNSUPPORTED_ERROR, "Bitwise reductions need an integer source");
  GpuReduction *gr = new (std::nothrow) GpuReduction();
  if (gr == nullptr) return ga_err_set(errrec, GA_MEMORY_ERROR, "Out of memory");
  gr->ctx = ctx;
  gr->op = op;
  gr->info = info;
  gr->args.push_back({"x", s0Typecode, false});
  gr->arrays.push_back(0);
  gr->map_expr = "x";
  *grp = gr;
  return GA_NO_ERROR;
}

// The launch: checks, plan, kernels.  `srcs` are the array arguments with the
// strides to use (broadcast dims already have stride 0) over the common
// extents `dims`; `scalars` point at host values of the declared types.
struct src_view {
  const GpuArray *a;
  const int64_t *strides;   // nd byte strides (an array's own, or 0 where it is broadcast)
};
static_assert(sizeof(ssize_t) == sizeof(int64_t), "strides are read through int64_t pointers");

int issue_launches(gpucontext *ctx, const launch_rec &rec, const void *plan, unsigned K, const src_view *srcs,
                   GpuArray *d0, GpuArray *d1, void *const *scalars, unsigned nscalars, bool noalloc,
                   size_t scratch_skip);

// One call of an operator: argument checks, the dim lists and the plan the
// kernels read, the choice of kernel family and lane geometry, the launch.
class reduction_call {
 public:
  reduction_call(GpuReduction *gr_, GpuArray *d0_, GpuArray *d1_, unsigned nd_, const size_t *dims_,
                 const src_view *srcs_, void *const *scalars_, unsigned nscalars_,
                 unsigned reduxLen_, const int *reduxList_, bool noalloc_ = false, size_t scratch_skip_ = 0)
      : noalloc(noalloc_), scratch_skip(scratch_skip_), gr(gr_), ctx(gr_->ctx), tn(ga_hip_tuning(gr_->ctx)), info(gr_->info), K(gr_->nsrc()), d0(d0_), d1(d1_), nd(nd_),
        dims(dims_), srcs(srcs_), scalars(scalars_), nscalars(nscalars_), reduxLen(reduxLen_), reduxList(reduxList_),
        kind(info.kind), minmax(kind == K_MIN || kind == K_MAX),
        logical(kind == K_ALL || kind == K_ANY),
        planbuf(plan_bytes(K) / sizeof(int64_t), 0),
        p(*reinterpret_cast<rd_plan *>(planbuf.data())),
        fsstr(planbuf.data() + sizeof(rd_plan) / sizeof(int64_t)),
        rsstr(fsstr + (size_t)K * RD_MAXD),
        vecmask((1u << K) - 1) {}

  int run() {
    int err;
    if ((err = check_arguments()) != GA_NO_ERROR) return err;
    if ((err = build_dims()) != GA_NO_ERROR || nrows == 0) return err;
    fill_plan();
    choose_family();
    if (use_row) {
      choose_row_loads();
      row_geometry();
      wrows_geometry();
      srows_geometry();
      trows_geometry();
    } else {
      col_geometry();
    }
    if ((err = pick_variant()) != GA_NO_ERROR) return err;
    if ((err = prepare_launch()) != GA_NO_ERROR) return err;
    planned = true;
    if (plan_only) return GA_NO_ERROR;
    return issue_launches(ctx, rec, planbuf.data(), K, srcs, d0, d1, scalars, nscalars, noalloc, scratch_skip);
  }

  // what the planning left (valid when `planned`: arguments fine, something to launch)
  bool plan_only = false, planned = false;
  launch_rec rec;
  const std::vector<int64_t> &plan() const { return planbuf; }

 private:
  // true: partials go to the device's static scratch array, kernels must be
  // loaded already, and nothing on the way allocates device memory
  const bool noalloc;
  // bytes at the start of the context's scratch buffer that belong to the
  // caller (fold_rows keeps its folded partial results there)
  const size_t scratch_skip;
  GpuReduction *gr;
  gpucontext *ctx;
  const ga_tuning *tn;
  const op_info &info;
  const unsigned K;                 // number of array sources
  GpuArray *d0, *d1;
  const unsigned nd;
  const size_t *dims;
  const src_view *srcs;             // K of them
  void *const *scalars;             // nscalars host values, in the operator's order
  const unsigned nscalars;
  const unsigned reduxLen;
  const int *reduxList;
  const rd_kind kind;
  const bool minmax, logical;
  int d0_tc = -1, d1_tc = GA_LONG;
  std::vector<char> reduced;        // per source axis
  std::vector<dimrec> fr, rd;       // free and reduced dims, slowest first, fused
  int64_t nrows = 1, rtotal = 1;    // outputs, elements per output
  // plan = fixed part + per-source stride tables
  std::vector<int64_t> planbuf;
  rd_plan &p;
  int64_t *fsstr, *rsstr;           // [K][RD_MAXD] each
  std::vector<int64_t> elsz;
  int64_t elsz_max = 0, elsz_sum = 0, ncu = 1;
  int64_t rin = 1, rstr = 0, fstr = 0;   // inner reduced extent and stride, inner free stride
  int64_t rin_sz = 1;               // rin plus what a shifted row can gain
  // kernel family and lane geometry
  bool use_row = true, wrows = false, tail = false, srows = false, trows = false;
  unsigned G = 256, V = 1, U = 4, ES = 1, vecmask, RB = 1, L = 64, CV = 1, LO = 1, CY = 4;
  bool cloose = false;   // redux_col: four outputs per lane on any alignment and extent (four-byte elements)
  size_t groups = 0, lds_bytes = 0;
  variant *var = nullptr;

  int check_arguments() {
    if ((info.has_d0 && d0 == nullptr) || (info.has_d1 && d1 == nullptr))
      return ga_err_set(ctx->err, GA_INVALID_ERROR, "A destination array required by the operation is NULL");
    if (!info.has_d0) d0 = nullptr;
    if (!info.has_d1) d1 = nullptr;
    if (nd == 0 || reduxLen == 0 || reduxLen > nd || reduxList == nullptr)
      return ga_err_fmt(ctx->err, GA_INVALID_ERROR,
                        "Invalid reduction: source nd = %u, %u axes to reduce", nd, reduxLen);
    reduced.assign(nd, 0);
    for (unsigned i = 0; i < reduxLen; i++) {
      const int ax = reduxList[i];
      if (ax < 0 || ax >= (int)nd || reduced[ax])
        return ga_err_fmt(ctx->err, GA_INVALID_ERROR, "Reduction axis %d is out of range or repeated", ax);
      reduced[ax] = 1;
    }
    for (const GpuArray *d : {(const GpuArray *)d0, (const GpuArray *)d1})
      if (d != nullptr && d->data == nullptr)
        return ga_err_set(ctx->err, GA_INVALID_ERROR, "A destination array has no buffer");
    for (unsigned k = 0; k < K; k++) {
      const GpuArray *s = srcs[k].a;
      if (s->data == nullptr)
        return ga_err_set(ctx->err, GA_INVALID_ERROR, "A source array has no buffer");
      const int want = gr->args[gr->arrays[k]].tc;
      if (s->typecode != want)
        return ga_err_fmt(ctx->err, GA_VALUE_ERROR, "Source has typecode %d, operator was made for %d",
                          s->typecode, want);
      if (GpuArray_context(s) != ctx)
        return ga_err_set(ctx->err, GA_VALUE_ERROR, "Arrays belong to another context");
    }
    if ((d0 && GpuArray_context(d0) != ctx) || (d1 && GpuArray_context(d1) != ctx))
      return ga_err_set(ctx->err, GA_VALUE_ERROR, "Arrays belong to another context");

    // result types
    d0_tc = d0 ? d0->typecode : (gr->mapped ? gr->acc_tc : gr->src_tc());
    d1_tc = d1 ? d1->typecode : GA_LONG;
    if (d0) {
      if (!GpuArray_ISWRITEABLE(d0)) return ga_err_set(ctx->err, GA_VALUE_ERROR, "Destination not writeable");
      if (gr->mapped && !logical && d0_tc != gr->acc_tc)
        return ga_err_fmt(ctx->err, GA_VALUE_ERROR,
                          "Result has typecode %d, the operator accumulates in %d", d0_tc, gr->acc_tc);
      if (!gr->mapped && minmax && d0_tc != gr->src_tc())
        return ga_err_set(ctx->err, GA_VALUE_ERROR, "min/max results must have the source's type");
      if ((kind == K_AND || kind == K_OR || kind == K_XOR || logical) && !is_int_type(d0_tc))
        return ga_err_set(ctx->err, GA_VALUE_ERROR,
                          "Result of a logical/bitwise reduction must be an integer type");
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
        if (d->dimensions[k] != dims[ax])
          return ga_err_fmt(ctx->err, GA_VALUE_ERROR,
                            "Destination dimension %u is %zu, source axis %u is %zu", k,
                            d->dimensions[k], ax, dims[ax]);
        k++;
      }
    }
    return GA_NO_ERROR;
  }

  // Free and reduced dim lists (extent-1 dims dropped, sorted, fused).
  int build_dims() {
    // dim lists
    nrows = 1;
    rtotal = 1;
    {
      unsigned k = 0;
      for (unsigned ax = 0; ax < nd; ax++) {
        if (reduced[ax]) continue;
        const int64_t dim = (int64_t)dims[ax];
        nrows *= dim;
        if (dim != 1) {
          dimrec r;
          memset(&r, 0, sizeof(r));
          r.dim = dim;
          for (unsigned q = 0; q < K; q++) r.s[q] = srcs[q].strides[ax];
          r.a = d0 ? (int64_t)d0->strides[k] : 0;
          r.b = d1 ? (int64_t)d1->strides[k] : 0;
          fr.push_back(r);
        }
        k++;
      }
      int64_t mul = 1;
      for (unsigned i = reduxLen; i-- > 0;) {
        const int ax = reduxList[i];
        const int64_t dim = (int64_t)dims[ax];
        rtotal *= dim;
        if (dim != 1) {
          dimrec r;
          memset(&r, 0, sizeof(r));
          r.dim = dim;
          for (unsigned q = 0; q < K; q++) r.s[q] = srcs[q].strides[ax];
          r.a = mul;
          rd.insert(rd.begin(), r);
        }
        mul *= dim;
      }
    }
    if (nrows == 0) return GA_NO_ERROR;   // (run() sees nrows == 0 and stops)
    if (rtotal == 0 && minmax)
      return ga_err_set(ctx->err, GA_VALUE_ERROR, "min/max over an empty axis has no value");
    if (rtotal == 0) rd.clear();
    sort_and_fuse(fr, K, true);
    sort_and_fuse(rd, K, false);
    if (fr.size() > (size_t)RD_MAXD || rd.size() > (size_t)RD_MAXD)
      return ga_err_fmt(ctx->err, GA_UNSUPPORTED_ERROR,
                        "More than %d non-mergeable free or reduced dimensions", RD_MAXD);
    return GA_NO_ERROR;
  }

  void fill_plan() {
    // plan = fixed part + per-source stride tables
    p.nf = (int)fr.size();
    p.nr = (int)rd.size();
    for (int i = 0; i < p.nf; i++) {
      p.fdim[i] = fr[i].dim; p.fd0str[i] = fr[i].a; p.fd1str[i] = fr[i].b;
      for (unsigned q = 0; q < K; q++) fsstr[q * RD_MAXD + i] = fr[i].s[q];
    }
    for (int i = 0; i < p.nr; i++) {
      p.rdim[i] = rd[i].dim; p.rmul[i] = rd[i].a;
      for (unsigned q = 0; q < K; q++) rsstr[q * RD_MAXD + i] = rd[i].s[q];
    }
    p.nrows = nrows;
    p.rtotal = rtotal;
    p.nsplit = 1;
    // Does the flattened index grow with the position in the reduced range
    // (dims slowest first)?  Then a scan in that order meets equal values
    // lowest index first.
    p.rising = rtotal < 0x7fffffff ? 1 : 0;
    for (int i = 0; i + 1 < p.nr; i++)
      if (p.rmul[i] < p.rdim[i + 1] * p.rmul[i + 1]) p.rising = 0;
    for (int i = 0; i < p.nr; i++)
      if (p.rmul[i] <= 0) p.rising = 0;
    p.fused = 0;

    elsz_max = elsz_sum = 0;
    elsz.assign(K, 0);
    for (unsigned q = 0; q < K; q++) {
      elsz[q] = (int64_t)gpuarray_get_elsize(gr->args[gr->arrays[q]].tc);
      elsz_max = std::max(elsz_max, elsz[q]);
      elsz_sum += elsz[q];
    }
    ncu = (int64_t)ga_hip_numprocs(ctx);
    rin = p.nr ? p.rdim[p.nr - 1] : 1;
    rstr = p.nr ? rd[p.nr - 1].smax : 0;
    fstr = p.nf ? fr[p.nf - 1].smax : INT64_MAX;
  }

  void choose_family() {
    // Lanes along the reduced run unless the free run is the one that is
    // contiguous in memory (or the reduced run is too short to feed a wavefront).
    // Short reduced runs are fine when they are the only reduced dim: several
    // rows then share a wavefront (redux_wrows).
    use_row = p.nf == 0 || (rstr <= fstr && (rin >= 32 || p.nr <= 1)) ||
                   (rin >= 4096 && rstr <= 4 * elsz_max);
    if (rtotal == 0) use_row = true;
    // (A handful of outputs over a small array - the sum over axis 0 of
    // (8192, 10) floats - looks faster with lanes along the reduced run when the
    // array is still in the cache from the call before, 7.9 -> 4.8 us; read
    // after another kernel wrote it, as the second call of folded rows does, it
    // is slower, 7.6 -> 10.2 us.  Not taken.)
    {
      const char *force = tn->redux_family;
      if (strcmp(force, "row") == 0) use_row = true;
      if (strcmp(force, "col") == 0 && p.nf > 0) use_row = false;
    }
  }

  // redux_row / redux_wrows: elements per load, element step, which sources
  // take vector loads, shifted rows.
  void choose_row_loads() {
    // Widest aligned load the layout allows, for a source whose inner reduced
    // stride is its element size: v elements, v*elsz bytes, everything the
    // lane's address is built from a multiple of that.
    auto fits = [&](unsigned q, unsigned v, int64_t es) {
      const GpuArray *s0 = srcs[q].a;
      const int64_t bytes = (int64_t)v * es * elsz[q];
      const uintptr_t base = (uintptr_t)s0->data->devptr + s0->offset;
      bool ok = rin % v == 0 && base % (uintptr_t)bytes == 0;
      for (int i = 0; ok && i < p.nf; i++) ok = fsstr[q * RD_MAXD + i] % bytes == 0;
      for (int i = 0; ok && i + 1 < p.nr; i++) ok = rsstr[q * RD_MAXD + i] % bytes == 0;
      return ok;
    };
    if (K == 1 && p.nr && rtotal > 0 && rsstr[p.nr - 1] > 0 && rsstr[p.nr - 1] % elsz[0] == 0) {
      // One source: its inner reduced dim may also step by ES = 2 or 4
      // elements (a [::2] / [::4] view): a load then fetches V*ES contiguous
      // elements and uses every ES-th one.  Such a load reads up to ES-1
      // elements past the last one used, so it must stay inside the buffer.
      const GpuArray *s0 = srcs[0].a;
      const int64_t es = rsstr[p.nr - 1] / elsz[0];
      if (es == 1 || es == 2 || es == 4) {
        unsigned v = (unsigned)(16 / (elsz[0] * es));
        if (v < 1) v = 1;   // 8-byte elements four apart: no load holds two of them
        size_t bufsz = 0;
        gpudata_property(s0->data, GA_BUFFER_PROP_SIZE, &bufsz);
        int64_t last = (int64_t)s0->offset;   // byte offset of the farthest element
        for (int i = 0; i < p.nf; i++) if (fsstr[i] > 0) last += (p.fdim[i] - 1) * fsstr[i];
        for (int i = 0; i < p.nr; i++) if (rsstr[i] > 0) last += (p.rdim[i] - 1) * rsstr[i];
        const bool overread_ok = es == 1 || (size_t)(last + es * elsz[0]) <= bufsz;
        const unsigned vmax = v;
        while (v > 1 && !(overread_ok && fits(0, v, es))) v /= 2;
        V = v;
        if (V > 1) ES = (unsigned)es;
        // A contiguous row that is misaligned, or whose length is not a
        // multiple of the load, still takes full-width aligned loads: a row
        // is read from the 16-byte boundary at or below its start, and the
        // elements before its first and after its last are masked out.  The
        // loads stay inside the buffer's allocation.  Measured on MI355X:
        // sums over 65536 rows of 1023 floats 65 us with 4-byte loads, 41 us
        // for rows of 1024; element-aligned (misaligned) 16-byte loads were
        // tried first and ran slower than 4-byte loads on long rows.
        if (es == 1 && V < vmax && rin >= (int64_t)vmax && GpuArray_ISALIGNED(s0) &&
            TUNE(tn, REDUX_TAIL, 1)) {
          const size_t readable = ga_hip_readable_bytes(s0->data);
          const size_t end = ((size_t)last + (size_t)elsz[0] + 15) & ~(size_t)15;
          bool nonneg = true;   // the lowest address is the array's own start
          for (int i = 0; i < p.nf; i++) nonneg = nonneg && fsstr[i] >= 0;
          for (int i = 0; i < p.nr; i++) nonneg = nonneg && rsstr[i] >= 0;
          if ((uintptr_t)s0->data->devptr % 16 == 0 && end <= readable && nonneg) {
            V = vmax;
            ES = 1;
            tail = true;
          }
        }
      }
    } else if (K > 1 && p.nr && rtotal > 0) {
      // Several sources: the widest type gets 16-byte loads when every source
      // that is contiguous along the inner reduced dim is aligned for its
      // share; sources with another stride there (0 for a broadcast one) are
      // fetched element by element.
      unsigned v = (unsigned)(16 / elsz_max), unit_mask = 0;
      for (unsigned q = 0; q < K; q++)
        if (rsstr[q * RD_MAXD + p.nr - 1] == elsz[q]) unit_mask |= 1u << q;
      if (unit_mask != 0) {
        for (unsigned q = 0; q < K; q++)
          while (v > 1 && ((unit_mask >> q) & 1u) && !fits(q, v, 1)) v /= 2;
        V = v;
        if (V > 1) vecmask = unit_mask;
      }
    }
  }

  // redux_row: lanes per output, loads in flight, outer coordinates side by
  // side, units and splits.
  void row_geometry() {
    // One wavefront per output when eight loads per lane cover the inner
    // reduced dim, four wavefronts otherwise.  Measured on MI355X: rows of
    // 8192 floats run at 6.7 TB/s with 256 lanes per row and 6.0 with 64;
    // rows of 512 stepped halves at 3.1 TB/s (useful) with 64 and 2.0 with 256.
    // a shifted row can be up to V-1 elements longer than its extent
    rin_sz = rin + (tail ? (int64_t)V - 1 : 0);
    G = (rin_sz <= (int64_t)64 * V * 8) ? 64 : 256;
    {
      const unsigned long force = TUNE(tn, REDUX_G, 0);
      if (force == 64 || force == 256) G = (unsigned)force;
    }
    int64_t per_pass = (int64_t)G * V;
    U = (unsigned)TUNE(tn, REDUX_U, 8);
    if (U != 1 && U != 2 && U != 4 && U != 8) U = 8;
    // Bytes a lane keeps in flight over all sources.  Measured on MI355X
    // (dot product of two 2^27-float vectors): 64 bytes per lane with 4 groups
    // per compute unit 162 us, 128 bytes with 2 groups 179 us; one source
    // keeps the 128 bytes its sweep found best.
    const int64_t lane_bytes = (int64_t)TUNE(tn, REDUX_LANE_BYTES, K > 1 ? 64 : 128);
    while (U > 1 && (int64_t)U * V * ES * elsz_sum > lane_bytes) U /= 2;
    while (U > 1 && per_pass * (U / 2) >= rin_sz) U /= 2;
    int64_t outer = 1;
    for (int i = 0; i + 1 < p.nr; i++) outer *= p.rdim[i];
    // A few rows of moderate length are a matter of latency, not of bandwidth:
    // with eight loads per lane and unit such a row is cut into a handful of
    // pieces, and each lane then walks a long chain of dependent operations
    // (for min/max a compare and two selects per element).  Fewer loads per
    // unit give more units, hence more pieces.  Measured on MI355X, one row of
    // 2^16 / 2^18 floats, kernel time with 8 / 4 / 2 loads per unit: max 6.8 /
    // 5.8 / 5.5 and 6.8 / 6.0 / 5.5 us, sum 4.4 / 4.0 / 4.0 and 4.3 / 4.1 / 4.1;
    // 2^20 floats 7.4 / 7.3 / 7.9 (enough pieces as it is), 2^14 floats 4.7 / 5.0
    // / 5.5 (too short to be worth cutting at all).
    if (TUNE(tn, REDUX_U, 0) == 0 && rtotal >= 49152) {
      const int64_t rowgroups_now = (nrows + 256 / G - 1) / (256 / G);
      auto pieces = [&](unsigned u) {
        const int64_t units_u = outer * ((rin_sz + per_pass * u - 1) / (per_pass * u));
        return rowgroups_now * (units_u / 2);
      };
      while (U > 2 && pieces(U) < 64) U /= 2;
    }
    // Several reduced dims with a short inner one (statistics over the batch
    // and a small spatial extent, say): the lanes a row does not need take
    // further outer reduced coordinates.  LI lanes cover the inner dim with up
    // to four loads each, LO = G / LI outer coordinates sit side by side.
    // Only when one load per lane would leave half the wavefront idle: rows
    // of 512 stepped halves ran at 45.4 us with 64 lanes and two loads each,
    // 47.4 us with 32 lanes and two outer coordinates side by side.
    if (p.nr >= 2 && rtotal > 0 && G == 64 && rin_sz <= (int64_t)32 * V &&
        TUNE(tn, REDUX_LO, 1)) {
      const int64_t need = (rin_sz + (int64_t)V * 4 - 1) / ((int64_t)V * 4);
      unsigned LI = 1;
      while (LI < 64 && (int64_t)LI < need) LI *= 2;
      if (LI < 64) {
        LO = 64 / LI;
        U = 1;
        while (U < 8 && (int64_t)LI * V * U < rin_sz) U *= 2;
        per_pass = (int64_t)LI * V;
      }
    }
    const int64_t seg = per_pass * U;
    p.nseg = rin > 0 ? (rin_sz + seg - 1) / seg : 1;
    if (p.nseg < 1) p.nseg = 1;
    p.router = outer;
    p.units = rtotal > 0 ? (LO > 1 ? (outer + LO - 1) / LO : outer * p.nseg) : 0;
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
    int64_t per_cu = (int64_t)TUNE(tn, REDUX_GROUPS_PER_CU, 0);
    if (per_cu == 0) {
      const int64_t inflight = (int64_t)G * U * V * ES * elsz_sum;   // bytes per group
      // A kernel that does next to nothing per element - one source of floats
      // or doubles, summed or multiplied in its own type, whole aligned loads -
      // is best with ONE such group per unit, which also keeps it within the
      // single launch: full fp32 sum of 2^28 153.4 -> 147.3 us (7.3 TB/s), of
      // 2^24 16.0 -> 14.7, rows of (16, 2^22) 42.8 -> 39.6.  Everything else
      // needs the second group to overlap its arithmetic with the loads:
      // max of 2^26 floats 43 us with two groups against 57 with one (NaN and
      // tie rules per element), sum of 2^27 halves 40 / 44.5 (a conversion per
      // element), int32 into int64 39.8 / 42.7, a ragged row (masked ends)
      // 40.2 / 48.6, the dot product of two arrays 156 / 180.
      const int stc0 = gr->args[gr->arrays[0]].tc;
      bool light = K == 1 && !gr->mapped && !tail && !info.has_d1 &&
                   (info.kind == K_SUM || info.kind == K_PROD) &&
                   (stc0 == GA_FLOAT || stc0 == GA_DOUBLE) && acc_typecode(gr, d0_tc) == stc0;
      if (!TUNE(tn, REDUX_LIGHT, 1)) light = false;
      const int64_t want = (int64_t)TUNE(tn, REDUX_INFLIGHT, light ? 32768 : 65536);
      const int64_t least = (int64_t)TUNE(tn, REDUX_MIN_PER_CU, light ? 1 : 2);
      per_cu = (want + inflight - 1) / inflight;
      if (per_cu < least) per_cu = least;
      if (per_cu > 32) per_cu = 32;
    }
    const int64_t target = ncu * per_cu;
    if (rowgroups < target && p.units >= 8) {
      nsplit = (target + rowgroups - 1) / rowgroups;
      const int64_t min_units = (int64_t)TUNE(tn, REDUX_MIN_UNITS, 2);
      if (nsplit > p.units / min_units) nsplit = p.units / min_units;
      if (nsplit > 65536) nsplit = 65536;
      if (nsplit < 1) nsplit = 1;
    }
    // Groups that all fit on the chip at once start together, and the compute
    // units that hold one more than the others finish last, alone: 300 rows
    // leave 212 units with one group and 44 with two.  More pieces even that
    // out.  Measured on MI355X, sum over axis 1 of (300, 223696) floats: 51.0
    // us whole rows, 45.2 in pieces (two launches); (130, 500000) 50.6 -> 43.5,
    // (520, 129000) 50.8 -> 45.8, int32 (290, 230000) 50.8 -> 48.0.  Only for a
    // large excess: the pieces need a finish of their own, often a second
    // launch ((640, 104857), a fifth too many on some units, 46.5 whole and
    // 47.3 in pieces; (1000, 65536), 3.9 groups per unit, 40.4 whole).
    if (TUNE(tn, REDUX_BALANCE, 1) && p.units >= 8 && rowgroups > 0) {
      const auto excess = [&](int64_t ns) {
        const int64_t g = rowgroups * ns;
        return (double)((g + ncu - 1) / ncu * ncu) / (double)g;
      };
      const int64_t resident = ncu * 8;
      int64_t cap = p.units / (int64_t)TUNE(tn, REDUX_MIN_UNITS, 2);
      if (cap > 65536) cap = 65536;
      if (nsplit > 1 && rowgroups * nsplit >= ncu) {
        // Rows already in pieces: another count costs nothing, so the nearest
        // one that fills the units more evenly is taken, below the target as
        // well as above (10 rows in 52 pieces are 520 groups on 256 units, in
        // 51 pieces 510).  Sum over axis 1, floats: (10, 6710886) 47.3 -> 43.7 us,
        // (24, 2796202) 47.8 -> 43.3, (48, 1398101) 48.8 -> 42.9 (two launches ->
        // one), (3, 22369621) 46.4 -> 42.7, maximum of int32 (10, 6710886) 45.9 ->
        // 43.7.  The search stops at the first count within 7 % of even: one further
        // away may cut the pieces too short to end in the same launch.
        const int64_t lo = std::max<int64_t>(1, (target - ncu) / rowgroups);
        int64_t best = nsplit;
        double be = excess(nsplit);
        for (int64_t d = 1; be > 1.07 && (nsplit - d >= lo || (nsplit + d <= cap && rowgroups * (nsplit + d) <= 2 * resident)); d++)
          for (const int64_t ns : {nsplit - d, nsplit + d})
            if (ns >= lo && ns <= cap && rowgroups * ns >= ncu && rowgroups * ns <= 2 * resident &&
                excess(ns) + 0.02 < be) {
              best = ns;
              be = excess(ns);
            }
        nsplit = best;
      } else if (rowgroups * nsplit < resident && excess(nsplit) > 1.25) {
        int64_t best = nsplit;
        for (int64_t ns = nsplit + 1; ns <= cap && rowgroups * ns <= 2 * resident; ns++) {
          if (excess(ns) < excess(best) - 0.02) best = ns;
          if (excess(best) <= 1.03) break;
        }
        nsplit = best;
      }
    }
    p.upb = p.units > 0 ? (p.units + nsplit - 1) / nsplit : 0;
    if (p.upb > 0) nsplit = (p.units + p.upb - 1) / p.upb;
    p.nsplit = (int)nsplit;
    groups = (size_t)(rowgroups * nsplit);
  }

  void wrows_geometry() {
    // Short rows, one wavefront each, take the kernel without the unit loop.
    // A wavefront takes RB rows at a time and issues their loads together:
    // a row that is a single load per lane would otherwise leave the
    // wavefront with one load in flight.
    if (G == 64 && p.nsplit == 1 && p.units == 1 && p.nr <= 1 && TUNE(tn, REDUX_WROWS, 1)) {
      wrows = true;
      // Measured on MI355X: any() over 131072 rows of 512 stepped bytes 29.8 us
      // one row at a time, 24.8 us with batches of 4 and 8 rows per wavefront;
      // rows of 1000 floats (four loads per lane already) 45 us one at a time,
      // 66 / 92 us in batches of 2 / 4.
      // A row much shorter than a wavefront's reach gets L < 64 lanes and
      // 64 / L rows share the wavefront: L is the smallest power of two that
      // covers the row with four loads per lane.
      {
        const int64_t need = (rin_sz + (int64_t)V * 4 - 1) / ((int64_t)V * 4);
        L = 1;
        while (L < 64 && (int64_t)L < need) L *= 2;
        // Up to 32 lanes, one load per lane and more lanes per row do better
        // than four loads on few lanes (the batches keep the loads in flight):
        // sums over rows of 32 floats 79.6 us with 2 lanes x 4 loads, 45.7 with
        // 8 x 1; rows of 100: 42.0 with 8 x 4, 34.6 with 32 x 1; rows of 17:
        // 76.9 -> 59.6.  Min/max carry an index through every cross-lane
        // step, so they keep two loads per lane (rows of 64: 80 us with 16
        // lanes, 67 with 8).
        // (vector loads only: rows of 3 floats, element loads, 60 us with one
        // lane per row and 74 with four).
        // Below 8 lanes a row of four-byte or wider elements does better
        // with one load per lane again (maximum over rows of 32 floats: 50.3 us
        // with 4 lanes x 2 loads, 44.3 with 8 x 1; of 24: 53.1 / 50.9).
        if (V > 1) {
          const auto lanes_for = [&](int64_t per_lane) {
            const int64_t n = (rin_sz + per_lane - 1) / per_lane;
            unsigned l = 1;
            while (l < 64 && (int64_t)l < n) l *= 2;
            return l;
          };
          unsigned l1 = lanes_for((int64_t)V * (minmax ? 2 : 1));
          if (minmax && elsz[0] >= 4 && l1 < 8 && nrows >= 65536) {   // (a thousand rows of 17: 4.6 us with 4 lanes, 7.3 with 8)
            const unsigned single = lanes_for((int64_t)V);
            l1 = single < 8 ? single : 8;
          }
          if (l1 <= 32) L = l1;
        }
        const unsigned long force = TUNE(tn, REDUX_L, 0);
        if (force >= 1 && force <= 64 && (force & (force - 1)) == 0 &&
            (int64_t)force * V * 8 >= rin_sz)
          L = (unsigned)force;
        if (L < 64) {
          U = 1;
          while (U < 8 && (int64_t)L * V * U < rin_sz) U *= 2;
        }
      }
      RB = (unsigned)TUNE(tn, REDUX_RB, L < 64 ? (U >= 4 ? 1 : 4 / U) : (U == 1 ? 4 : 1));
      if (RB != 1 && RB != 2 && RB != 4 && RB != 8) RB = 1;
      const int64_t per_batch = (int64_t)(64 / L) * RB;
      int64_t rpw = (int64_t)TUNE(tn, REDUX_RPW, (RB == 1 && L == 64) ? 1 : 2 * per_batch);
      if (rpw < 1) rpw = 1;
      p.upb = rpw;
      const int64_t waves = (nrows + rpw - 1) / rpw;
      groups = (size_t)((waves + 3) / 4);
    }
  }

  void srows_geometry() {
    // Rows of a few dozen elements that follow one another in memory: a group
    // stages the bytes of up to 256 rows in LDS and every lane walks one row
    // (redux_srows).  Measured on MI355X, 2^26 floats in rows of 8 / 17 / 33 /
    // 64: sum 63 / 72 / 68 / 48 us with redux_wrows, 51 / 48 / 46 / 45 us
    // staged; maxandargmax 73 / 76 / 78 / 56 against 59 / 53 / 53 / 72 us
    // (its walk costs more per element, and 64 KiB of LDS per group leaves
    // two groups per compute unit), hence the lower limit for min/max.  Rows
    // whose pitch is no multiple of 16 bytes cost redux_wrows a shifted,
    // masked load pattern per row and stay here longer: 33 doubles (264
    // bytes) sum / max 118 / 145 us there, 91 / 91 us staged; 40 doubles (320
    // bytes, aligned) 89 / 100 against 95 / 121 us.  Rows of whole 16-byte
    // pieces leave at 128 bytes (96 for min/max): 2^26 floats in rows of 24 /
    // 32 / 48 / 64, staged against redux_wrows: sum 44.0 / 43.3 / 42.9 / 43.0
    // against 44.4 / 42.7 / 41.0 / 40.5 us, maximum 44.7 / 48.9 / 57.8 / 63.9
    // against 50.9 / 44.3 / 44.0 / 41.7; maximum of 2^26 halves in rows of 48 /
    // 64: 30.6 / 35.4 against 26.6 / 25.8.  Bytes that are summed or tested
    // (four to an operation in redux_wrows, one by one in a staged walk) leave
    // at 32: 2^28 bytes in rows of 48 / 64 / 96 / 128, sum 60.3 / 58.1 / 54.7 /
    // 68.0 against 50.9 / 48.8 / 48.2 / 47.5 us, any 53.1 / 48.6 / 49.9 / 70.4
    // against 41.6 / 41.2 / 40.0 / 40.6; their maximum stays to 96 (47.8 / 46.5 /
    // 43.5 against 76.0 / 65.5 / 74.7).
    if (K == 1 && p.nr == 1 && p.nf == 1 && rtotal > 0 && rsstr[0] == elsz[0] &&
        fsstr[0] == rin * elsz[0] && rin >= 2 &&
        rin * elsz[0] <= (int64_t)TUNE(tn, REDUX_SROWS_MAX_BYTES, (rin * elsz[0]) % 16 != 0 ? 384 : (minmax ? 96 : (elsz[0] == 1 ? 32 : 128))) &&
        rin * elsz[0] > (int64_t)TUNE(tn, REDUX_SROWS_MIN_BYTES, 16) &&
        nrows >= (int64_t)TUNE(tn, REDUX_SROWS_MIN_ROWS, 512) * ncu &&
        GpuArray_ISALIGNED(srcs[0].a) && TUNE(tn, REDUX_SROWS, 1)) {
      const GpuArray *s0 = srcs[0].a;
      const size_t readable = ga_hip_readable_bytes(s0->data);
      const size_t end = ((size_t)s0->offset + (size_t)(nrows * rin * elsz[0]) + 15) & ~(size_t)15;
      if ((uintptr_t)s0->data->devptr % 16 == 0 && end <= readable) {
        int64_t per_group = (65536 - 16) / (rin * elsz[0]);
        if (per_group > 256) per_group = 256;
        per_group &= ~(int64_t)63;   // whole wavefronts
        if (per_group >= 64) {
          srows = true;
          wrows = false;
          p.nsplit = 1;
          p.upb = per_group;
          groups = (size_t)((nrows + per_group - 1) / per_group);
          lds_bytes = (size_t)(per_group * rin * elsz[0] + 16 + 15) & ~(size_t)15;
        }
      }
    }
  }

  void trows_geometry() {
    // Rows of at most 32 bytes that follow one another in memory, the first
    // on a 16-byte boundary: a lane takes the least run of whole rows that is
    // whole 16-byte chunks into registers and walks its rows there
    // (redux_trows).  redux_wrows is bound by its instructions per row on
    // these.  Measured on MI355X, 2^26 floats in rows of 3 / 5 / 6 / 7: sum
    // 75.4 / 62.6 / 56.9 / 51.7 us there, 50.9 / 49.6 / 48.4 / 48.5 here,
    // argmax 86.7 / 65.9 / 64.0 / 54.4 against 58.3 / - / 51.1 / -; 2^24 rows
    // of 6 halves 71.5 -> 36.9 us, of 12 bytes (summed into 64-bit integers)
    // 74.9 -> 48.5.  Rows of more than 32 bytes gain nothing (10 floats 44.9
    // there, 47.4 here; 16 floats 45 staged in LDS, 43 here).
    const int64_t rowb = rin * elsz[0];
    if (K == 1 && p.nr == 1 && p.nf == 1 && rtotal > 0 && rsstr[0] == elsz[0] && fsstr[0] == rowb &&
        rin >= 2 && elsz[0] <= 8 && rowb <= (int64_t)TUNE(tn, REDUX_TROWS_MAX_BYTES, 32) &&
        nrows >= (int64_t)TUNE(tn, REDUX_TROWS_MIN_ROWS, 16384) && TUNE(tn, REDUX_TROWS, 1)) {
      const GpuArray *s0 = srcs[0].a;
      const size_t readable = ga_hip_readable_bytes(s0->data);
      const size_t end = ((size_t)s0->offset + (size_t)(nrows * rowb) + 15) & ~(size_t)15;
      int64_t g = rowb, h = 16;
      while (h) { const int64_t t = g % h; g = h; h = t; }
      const int64_t per_lane = 16 / g, chunks = rowb / g;   // a lane's rows, in as many chunks
      // Rows of 2, 4, 8, 16 or 32 bytes need no hand-out (one or two chunks
      // per lane), and there redux_wrows keeps up: it stays for four- and
      // eight-byte elements (2^26 floats in rows of 2 / 4 / 8: 55.5 / 52.2 /
      // 49.3 us against 57.1 / 54.6 / 51.6 here) and for rows of 16 bytes
      // (2^27 bytes, any: 21.3 against 24.7 us); one- and two-byte elements
      // in rows of 2, 4, 8 or 32 bytes come here (2^27 bytes in rows of 2 /
      // 4 / 32, max: 104.6 / 39.9 / 28.2 us there, 29.3 / 28.4 / 21.9 here).
      const unsigned long direct = TUNE(tn, REDUX_TROWS_DIRECT, 1);
      // more than two chunks per lane are handed out through LDS, 4 KiB per chunk
      if (((uintptr_t)s0->data->devptr + (size_t)s0->offset) % 16 == 0 && end <= readable &&
          chunks <= (int64_t)TUNE(tn, REDUX_TROWS_MAX_CHUNKS, 7) &&
          (chunks > 2 || direct == 2 || (direct == 1 && elsz[0] <= 2 && rowb != 16))) {
        trows = true;
        srows = wrows = false;
        lds_bytes = 0;
        p.nsplit = 1;
        // bit 0 / 1: the values / indices of a lane's rows lie side by side
        // in memory and start on the boundary of one store
        auto side_by_side = [&](const GpuArray *d, int64_t stride) {
          if (d == nullptr) return false;
          const int64_t es = (int64_t)gpuarray_get_elsize(d->typecode);
          const int64_t run = std::min<int64_t>(es * per_lane, 16);
          return stride == es && ((uintptr_t)d->data->devptr + (size_t)d->offset) % (size_t)run == 0;
        };
        p.upb = (side_by_side(d0, p.fd0str[0]) ? 1 : 0) | (side_by_side(d1, p.fd1str[0]) ? 2 : 0);
        const int64_t lanes = (nrows + per_lane - 1) / per_lane;
        groups = (size_t)((lanes + 255) / 256);
      }
    }
  }

  void col_geometry() {
    const int64_t fin = p.fdim[p.nf - 1];
    const unsigned long cy_forced = TUNE(tn, REDUX_COL_ROWS, 0);
    // Lane rows of a group: 8 (32 lanes along the free dim) when the reduced
    // range is long, else 4.  Measured on MI355X with 4 / 8 / 16: per-channel
    // sum of (64, 56, 56, 256) floats 45.2 / 40.9 / 39.7 us, max over the
    // channels of (64, 256, 56, 56) 49.7 / 44.1 / 47.1, sum over axis 0 of
    // 8192 x 8192 50.9 / 49.4 / 51.4, over the middle axis of 256 x 512 x 512
    // 47.0 / 43.8 / 47.5; but 8 x 2^23 over axis 0 49.3 / 72.4 / 121 and
    // 256 x 2^18 45.8 / 48.2 / 47.2.
    // Also 8 when successive elements of the reduced range lie 12 KiB or more
    // apart (a middle axis over long inner rows) and there are 32 of them or
    // more.  Sum over the middle axis, 4 / 8 lane rows: (128, 128, 4096) floats
    // 59.7 / 41.0 us, (64, 128, 8192) 50.3 / 40.7, (128, 128, 3072) 31.5 /
    // 29.8, (32, 128, 12288) 34.4 / 29.3, (128, 32, 16384) 48.4 / 40.0,
    // (64, 256, 4096) 46.2 / 42.8, halves (128, 128, 8192) 60.0 / 41.7; but
    // (256, 128, 2048), 8 KiB apart, 42.8 / 44.7 and (512, 128, 1024) 40.5 / 44.2.
    int64_t rpitch = 0;
    for (unsigned q = 0; q < K && p.nr > 0; q++) rpitch = std::max(rpitch, iabs(rsstr[q * RD_MAXD + p.nr - 1]));
    const bool far_apart = rpitch >= (int64_t)TUNE(tn, REDUX_COL_FAR, 12288) && rtotal >= 32;
    CY = (cy_forced == 1 || cy_forced == 2 || cy_forced == 4 || cy_forced == 8 || cy_forced == 16)
             ? (unsigned)cy_forced : (rtotal >= 512 || far_apart ? 8 : 4);
    int64_t CX = 256 / CY;   // lanes along the free dim
    // Adjacent outputs per lane: as many as one 16-byte load of the widest
    // source holds, when the inner free dim is contiguous in every source and
    // every address a lane forms is a multiple of its load.
    {
      unsigned cv = (unsigned)(16 / elsz_max);
      if (info.has_d1 && cv > 8) cv = 8;   // (value, index) pairs meet in LDS: 32 KiB per group at 8
      if (cv > (unsigned)TUNE(tn, REDUX_COL_CVMAX, 16)) cv = (unsigned)TUNE(tn, REDUX_COL_CVMAX, 16);
      for (unsigned q = 0; q < K; q++)
        if (fsstr[q * RD_MAXD + p.nf - 1] != elsz[q]) cv = 1;
      while (cv > 1) {
        bool ok = fin % cv == 0;
        for (unsigned q = 0; ok && q < K; q++) {
          const int64_t bytes = (int64_t)cv * elsz[q];
          const uintptr_t base = (uintptr_t)srcs[q].a->data->devptr + srcs[q].a->offset;
          ok = base % (uintptr_t)bytes == 0;
          for (int i = 0; ok && i + 1 < p.nf; i++) ok = fsstr[q * RD_MAXD + i] % bytes == 0;
          for (int i = 0; ok && i < p.nr; i++) ok = rsstr[q * RD_MAXD + i] % bytes == 0;
        }
        if (ok) break;
        cv /= 2;
      }
      // Four-byte elements that fail the above - an inner free dim that is no
      // multiple of four, rows that start off the 16-byte boundaries - still
      // go four to a lane: a load that assumes four-byte boundaries only, and
      // the lane at the end of the dim fetches what exists of its four one by
      // one.  Measured on MI355X, sums, one output per lane against this:
      // over axis 0 of (8192, 8192)[:, 1:] floats 75.6 / 51.3 us (44 -> 65 % of
      // peak), of (8192, 8192)[:, :8191] 53.2 / 49.0, of (8192, 8190) 63.4 /
      // 50.5, over the middle axis of (64, 1001, 1001) 77.9 / 56.8.  Such loads
      // run at about six sevenths of the rate of aligned ones ((8192, 8188):
      // 44.2 us), and folded rows, where they apply, stay ahead ((20000, 3001)
      // 40.2 us folded, 57.0 this way).  Not for scans that carry a position:
      // maximum over axis 0 of (8192, 8191) 57.0 / 63.8.
      cloose = false;
      const bool carries_position = info.has_d1 || (minmax && is_float_type(acc_typecode(gr, d0_tc)));
      // (nor for small inputs, which want lanes, not wide loads: the (128, 1001)
      // partial rows of a folded (65536, 1001) took 2.5 us longer this way, sums
      // over axis 0 of 16 MB, (4097, 1023) and (513, 8191), 13 and 23 % longer;
      // 36 MB, (3000, 3001), 20 % shorter)
      if (cv < 4 && elsz_max == 4 && !carries_position && TUNE(tn, REDUX_COL_LOOSE, 1) != 0 && fin >= 4 &&
          (double)nrows * (double)rtotal * 4.0 >= (double)TUNE(tn, REDUX_COL_LOOSE_MIN_BYTES, 32u << 20)) {
        bool ok = true;
        for (unsigned q = 0; ok && q < K; q++) {
          ok = elsz[q] == 4 && fsstr[q * RD_MAXD + p.nf - 1] == 4 && GpuArray_ISALIGNED(srcs[q].a);
        }
        if (ok) { cv = 4; cloose = true; }
      }
      if (!TUNE(tn, REDUX_COLVEC, 1)) { cv = 1; cloose = false; }
      // Splitting the reduced range costs a second pass (sum over the middle
      // axis of 256x512x512 floats: 54 us unsplit with one output per lane,
      // 64 us split in two with four), so when the widest load leaves too
      // few groups, take the widest one that still fills the chip unsplit.
      {
        const int64_t want = ncu * 4, outer_f = nrows / fin;
        auto groups_at = [&](unsigned c) { return ((fin + CX * c - 1) / (CX * c)) * outer_f; };
        // ... but not with less than 256 contiguous bytes per row and group:
        // sums over axis 0 of 4096 x 65536 bytes ran at 108 us with two
        // columns per lane (64 bytes per row and group).
        if (groups_at(cv) < want)
          for (unsigned c = cv / 2; c >= 1 && (int64_t)c * elsz_max * CX >= 256; c /= 2)
            if (groups_at(c) >= want) { cv = c; break; }
      }
      CV = cv;
    }
    // A short inner free dim (channels last, a few dozen of them) leaves most
    // of 64 lanes idle: fewer lanes along it and more lane rows, which then
    // take adjacent reduced coordinates.  Measured on MI355X, sum over the two
    // middle axes of (32, 128, 128, 64) floats: 48.3 us with 64 lanes along
    // the 64 channels (16 of them busy).
    if (cy_forced == 0)
      while (CY < 16 && fin <= (int64_t)(256 / (CY * 2)) * CV) CY *= 2;
    CX = 256 / CY;
    p.gx = (fin + CX * CV - 1) / (CX * CV);
    const int64_t outer = nrows / fin;
    const int64_t base_groups = p.gx * outer;
    int64_t nsplit = 1;
    // Measured on MI355X (sums over axis 0 of 8192x8192, 256x262144, 65536x1000
    // and 8x2^23 floats): one output per lane 63.6 / 55.2 / 58.5 / 134 us with
    // 8 groups per compute unit; four outputs per lane 50.1 / 45.8 / 50.5 /
    // 49.6 us with 3-4 groups, and 60 / 84 / 61 / 51 us with 8 (the second
    // shape then splits its 256 rows for nothing).
    // Three against four groups per unit, later, with eight lane rows: bytes
    // 16384 x 16384 54.3 -> 49.5 us, floats 65536 x 1000 48.6 -> 46.3,
    // 8192 x 8192 49.3 -> 48.1, halves 2048 x 65536 48.2 -> 46.1; two groups
    // were faster still for 2- and 4-byte elements and slower for bytes (59.5).
    // Float sums and products (next to nothing per element), two against three:
    // over axis 0 of (1024, 16384) 17.0 -> 14.8 us, (65536, 1024) 44.6 -> 43.6,
    // (2^20, 64) 45.1 -> 44.0, (16384, 4096) 45.4 -> 45.0; maximum of the same
    // 49.0 -> 51.2, sum of bytes 47.7 -> 58.0, of halves 46.0 -> 49.4.
    const int stc0 = gr->args[gr->arrays[0]].tc;
    const bool light = K == 1 && !gr->mapped && !info.has_d1 && (info.kind == K_SUM || info.kind == K_PROD) &&
                       (stc0 == GA_FLOAT || stc0 == GA_DOUBLE) && acc_typecode(gr, d0_tc) == stc0 &&
                       TUNE(tn, REDUX_LIGHT, 1) != 0 &&
                       scratch_skip == 0;   // folded rows measured better with three: (2^24, 3) 38.8 against 43.4 us
    // Lanes past the end of the inner free dim idle (160 kept floats under tiles
    // of 256: 5 lanes of 8), and a group then has fewer bytes in flight: such
    // float sums get the third group per unit as well.  Sums over axis 0, two /
    // three groups: (419430, 160) floats 51.6 -> 44.6 us (65 -> 75 % of peak),
    // (209715, 320) 47.6 -> 44.1, (174762, 384) 48.4 -> 44.9; over the middle
    // axis of (64, 4096, 320) 58.6 -> 52.0 (71 -> 81 %), of (64, 4096, 160)
    // 39.4 -> 29.1, of (64, 8192, 72) 32.0 -> 28.4.  Up to 80 % of the lanes
    // busy; at 78 % the shapes disagree: over axis 0 of (223696, 300), 300 kept
    // floats of 384, three groups 74 % of peak and two 66, of (335544, 200), 200
    // of 256, three 62 and two 68; with 192 of 256 the two are even.
    const double lanes_used = (double)fin / (double)(p.gx * (int64_t)(CX * CV));
    const bool idle_lanes = light && CV > 1 && lanes_used <= 0.8 && TUNE(tn, REDUX_COL_IDLE, 1) != 0;
    const int64_t target = ncu * (int64_t)TUNE(tn, REDUX_GROUPS_PER_CU, CV > 1 ? (light && !idle_lanes ? 2 : 3) : 8);
    if (base_groups < target && rtotal >= 256) {
      nsplit = (target + base_groups - 1) / base_groups;
      // Groups are dealt out to the compute units in turn: a few more than a
      // whole number per unit leave some units with one group more than the
      // rest (3 tiles of outputs in 171 pieces: 513 groups on 256 units; 192
      // tiles in 3 pieces: 576).  Of the piece counts from the target down to
      // one group per unit less and up to one more, the nearest one that fills
      // the units more evenly is taken.  Sums of floats, before / after: over
      // axis 0 of (87381, 768) 51.4 -> 45.7 us (65 -> 74 % of peak), of
      // (104857, 640) 50.7 -> 45.6, of (20000, 3000) 61 -> 71 %, of (4096, 12000)
      // 70 -> 77 %; whole powers of two divide the target and are not touched.
      if (TUNE(tn, REDUX_COL_BALANCE, 1) != 0) {
        auto excess = [&](int64_t ns) {
          const double per = (double)(base_groups * ns) / (double)ncu;
          return std::ceil(per) / per;
        };
        int64_t cap = rtotal / 64 < 4096 ? rtotal / 64 : 4096;
        if (cap < 1) cap = 1;
        const int64_t lo = std::max<int64_t>(1, (target - ncu) / base_groups);
        const int64_t hi = std::min<int64_t>(cap, (target + ncu + base_groups - 1) / base_groups);
        if (nsplit <= cap && base_groups * nsplit >= ncu) {
          int64_t best = nsplit;
          double be = excess(nsplit);
          for (int64_t d = 1; nsplit - d >= lo || nsplit + d <= hi; d++)
            for (const int64_t ns : {nsplit - d, nsplit + d})
              if (ns >= lo && ns <= hi && base_groups * ns >= ncu && excess(ns) + 0.02 < be) {
                best = ns;
                be = excess(ns);
              }
          nsplit = best;
        }
      }
      if (nsplit > rtotal / 64) nsplit = rtotal / 64;
      if (nsplit > 4096) nsplit = 4096;
      if (nsplit < 1) nsplit = 1;
    }
    p.upb = (rtotal + nsplit - 1) / nsplit;
    if (p.upb > 0) nsplit = (rtotal + p.upb - 1) / p.upb;
    p.nsplit = (int)nsplit;
    // Partials of a split column reduction: with many outputs they are laid
    // out split-major, so that adjacent lanes write adjacent slots, and the
    // second pass runs with lanes along the outputs (sum over axis 0 of
    // 8192 x 8192 bytes 37.8 -> 32.8 us, of int16 41.0 -> 37.0); with few
    // outputs that second pass would have too few lanes (1000 outputs over
    // 256 splits: 51.6 -> 65.9 us), and they stay output-major for the
    // wavefront-per-output pass.
    const int64_t many = (int64_t)TUNE(tn, REDUX_SPLIT_MAJOR_MIN, 4096);
    p.split_major = (nsplit > 1 && nrows >= many) ? 1 : 0;
    groups = (size_t)(base_groups * nsplit);
    p.units = (int64_t)(groups / 8 * 8);   // for the order that keeps neighbours on one die
    U = (unsigned)TUNE(tn, REDUX_COL_U, 4);
    if (U != 1 && U != 2 && U != 4 && U != 8) U = 4;
  }

  int pick_variant() {
    if (groups == 0 || groups > 0x7fffffffull)
      return ga_err_set(ctx->err, GA_XLARGE_ERROR, "Reduction needs more groups than one launch has");

    // bit 0: streaming loads; bit 1: interleaved splits (single reduced dim only)
    unsigned opts = TUNE(tn, REDUX_NT, 1) ? 1u : 0u;
    if (use_row && p.nr == 1 && p.nsplit > 1 && TUNE(tn, REDUX_INTERLEAVE, 1)) opts |= 2u;
    if (use_row && tail) opts |= 4u;   // bit 2: element-aligned vector loads with a ragged end
    // Column kernel on rows that do not start on 128-byte lines: the pieces of a
    // row that neighbouring groups fetch share the lines they straddle.
    //  - Groups that follow one another in launch order run on different dies,
    //    each with its own cache, so such a line came from memory once per die:
    //    sum over the middle axis of (64, 1000, 1000) floats read 1.38 times the
    //    array.  bit 13: neighbours along the inner free dim follow one another
    //    on ONE die (see the kernel).  Measured on MI355X, sums of floats, plain
    //    order / this one: middle axis of (64, 1000, 1000) 52.5 -> 39.2 us (61 ->
    //    82 % of peak), of (64, 1001, 1001) 56.1 -> 43.1 us, of (64, 1000, 1008)
    //    66 -> 83 %, of (16, 2000, 2000) 69 -> 79 %, int32 maxima of the first
    //    61 -> 82 %, axis 0 of (1000, 50257) 42.7 -> 38.6 us, of (8192, 8191)
    //    54.2 -> 46.8 us.  On whole lines nothing is shared and the plain order
    //    stays: (256, 512, 512) over the middle axis 84.5 % plain, 79.1 this way.
    //  - A streamed line is fetched again by the neighbour, so the loads that
    //    assume four-byte boundaries only (cloose) stay cacheable there:
    //    (8192, 8192)[:, 1:] over axis 0 51.6 -> 48.7 us.  Aligned loads keep the
    //    hint on any pitch: (65536, 1000) over axis 0 72.8 % of peak streamed,
    //    66.9 cacheable, (8, 10000, 1000) over the middle axis 79.5 / 72.2.
    if (!use_row) {
      bool lines = true;
      for (unsigned q = 0; q < K && lines; q++) {
        lines = ((uintptr_t)srcs[q].a->data->devptr + srcs[q].a->offset) % 128 == 0;
        for (int i = 0; lines && i + 1 < p.nf; i++) lines = fsstr[q * RD_MAXD + i] % 128 == 0;
        for (int i = 0; lines && i < p.nr; i++) lines = rsstr[q * RD_MAXD + i] % 128 == 0;
      }
      const unsigned long xcd = TUNE(tn, REDUX_XCD, 1);
      // (fewer than 16 groups: the order would be the plain one, or nearly)
      if (xcd == 2 || (xcd == 1 && !lines && groups >= 16)) opts |= 8192u;
      if (!lines && cloose && CV > 1 && TUNE(tn, REDUX_NT_LINES, 1) != 0) opts &= ~1u;
    }
    variant_spec vs = {d0_tc, d1_tc, use_row ? G : 256, use_row ? V : 1, U, opts, use_row ? ES : 1,
                       use_row ? vecmask : (1u << K) - 1, wrows ? RB : 1, wrows ? L : 64, use_row ? 1 : CV,
                       (use_row && !wrows) ? LO : 1};
    if (!use_row) vs.CY = CY;
    vs.opts |= use_row ? 16u : 32u;   // bits 4, 5: the family of kernels the text holds
    if (wrows) vs.opts |= 128u;         // bit 7: redux_wrows, not redux_row
    // bit 9: the outputs, the reduced range and their product (the elements
    // visited) all count below 2^31, so the kernels' divisions are 32-bit ones
    if ((double)nrows * (double)rtotal < 2147483648.0 && groups < 0x7fffffffull) vs.opts |= 512u;
    // bit 8: the kernels of the second pass too.  Beside redux_col always: they
    // compile in a fraction of its time, and a split and an unsplit call then
    // share one text.
    if (p.nsplit > 1 || !use_row) vs.opts |= 256u;
    // bit 6: redux_col meets a lane's elements in rising index order (min, max and their arg forms)
    if (!use_row && p.rising && (gr->info.kind == K_MAX || gr->info.kind == K_MIN)) vs.opts |= 64u;
    if (!use_row && cloose && CV > 1) vs.opts |= 4096u;   // bit 12: redux_col's loads assume the elements' alignment only
    if (srows)   // one kernel, independent of the lane geometry
      vs = {d0_tc, d1_tc, 64, 1, 1, (opts & 1u) | 8u | (vs.opts & 512u), 1, 1, 1, 64, 1, 1};
    if (trows) {   // one kernel per row length
      vs = {d0_tc, d1_tc, 64, 1, 1, (opts & 1u) | 1024u | (vs.opts & 512u), 1, 1, 1, 64, 1, 1};
      vs.TE = (unsigned)rin;
    }
    return get_variant(gr, vs, &var, !noalloc);
  }

  // What is left of the plan once the kernels are chosen: which kernels, how
  // many groups, how the partials of a split reduction are laid out.
  int prepare_launch() {
    const int acc_tc = acc_typecode(gr, d0_tc);
    const size_t accsz = logical ? 4 : acc_size_for(acc_tc);
    // A split reduction of moderate size ends in the launch that started it:
    // its outputs (row kernel) or tiles of outputs (column kernel) have a
    // counter each, and the piece that counts in last combines the partials.
    // Measured on MI355X, one launch against two, calls timed one by one /
    // issued back to back: sum of 2^16 floats 6.4 / 5.2 us against 8.4 / 8.7,
    // of 2^20 7.0 / 5.3 against 8.4 / 8.6, of 2^22 (256 groups) 9.2 / 7.1
    // against 8.7 / 8.6; with one group or more per compute unit waiting for
    // its partial to be acknowledged before it counts in costs more than the
    // second launch (2^24, 512 groups: 17.5 against 14.8 us).
    // Calls on the static scratch array always take two launches: the second
    // reads only what the first has written, so nothing there has to start
    // at zero.
    rec.fused = false;
    if (p.nsplit > 1 && !noalloc) {
      const size_t counters = use_row ? (size_t)nrows : groups / (size_t)p.nsplit;
      const size_t fused_max = (size_t)ncu * TUNE(tn, REDUX_FUSED, 1);   // 0 turns it off
      // Beyond one group per compute unit the single launch pays again once a
      // piece is long: the wait for the acknowledgement is then a small part of
      // a group's life, and the second launch (3 to 4 us) is saved.  Measured,
      // two launches against one: full sum of 2^24 floats (512 pieces of 128 KiB)
      // 15.9 against 16.7 us, of 2^25 25.3 / 25.0, of 2^26 42.2 / 40.1, of 2^28
      // 156.0 / 152.9; sum over axis 1 of (64, 2^20) 43.2 / 40.6.  The column
      // kernel's last piece combines a tile's partials by itself, so it must
      // not have many: over axis 0 of (4096, 16384) 44.0 / 42.0 us, of
      // (16384, 4096) 44.3 / 43.8, of (65536, 1024) 44.0 / 51.9, of
      // (2^20, 64) 44.3 / 73.0.  With up to 16 pieces per tile they may be as
      // short as 32 KiB: sum over the middle axis of (128, 500, 128) floats,
      // two launches / one, 12.6 / 9.7 us, of (32, 2000, 256) 17.0 / 14.7, over
      // axis 0 of (4000, 4000) 16.3 / 15.4.
      bool fuse = groups <= fused_max;
      // (partials that carry an index cost the column kernel's last piece twice
      // the loads: maxandargmax over axis 0 of (8192, 8192) 47.8 / 50.5)
      const bool carries_index = info.has_d1 || (minmax && is_float_type(acc_tc));
      // The column kernel's last piece walks through a tile's partials with
      // one lane row per 1 / RD_CY of them: many pieces are better combined by
      // the second launch, whose every wavefront takes a share.  One launch
      // against the kernels of two, over axis 0: sum of (8192, 10) floats, 128
      // pieces, 5.6 / 8.0 us, of (4096, 256), 64 pieces, 7.0 / 8.2, of
      // (16384, 64), 256 pieces, 10.5 / 7.8; maximum of floats (value and
      // position) (4096, 256) 14.9 / 10.6, (16384, 64) 25.5 / 12.6, (1024, 1024)
      // 11.9 / 10.4.
      if (fuse && !use_row &&
          p.nsplit > (int)TUNE(tn, REDUX_FUSED_COL_FEW, carries_index ? 16 : 128))
        fuse = false;
      if (!fuse && fused_max > 0 && groups > fused_max) {
        const double piece_bytes = (double)nrows * (double)rtotal * (double)elsz_sum / (double)groups;
        // (rows in a few pieces each spread the counting over many counters and
        // the combining over many groups, and below 160 MB the second launch is
        // a larger share: there pieces from 64 KiB on.  Two launches / one:
        // maximum over axis 1 of (64, 262144) floats 18.8 / 16.5 us, of int32
        // (100, 100000) 13.1 / 10.0, sum of halves (50, 400000) 13.0 / 10.2, of
        // (100, 671088) 26.8 / 24.1, of floats (40, 200000) 11.7 / 8.8; one row
        // in 512 pieces stays with two: maximum of 2^24 floats 17.5 / 18.5, of
        // 2^23 13.0 / 14.6; 268 MB of 130 to 520 rows 43.4 / 44.7, 45.8 / 47.7)
        const bool few = p.nsplit <= (int)TUNE(tn, REDUX_FUSED_FEW, 64) &&
                         (double)nrows * (double)rtotal * (double)elsz_sum < 160.0 * 1048576.0;
        fuse = use_row ? piece_bytes >= (double)TUNE(tn, REDUX_FUSED_PIECE, few ? 64u << 10 : 384u << 10)
                       : (!carries_index && p.nsplit <= (int)TUNE(tn, REDUX_FUSED_COL_SPLITS, 16) &&
                          piece_bytes >= (double)TUNE(tn, REDUX_FUSED_COL_PIECE, 32u << 10));
      }
      if (fuse && counters <= ga_hip_redux_counters_max && (accsz == 4 || accsz == 8)) {
        if (ga_hip_redux_counters(ctx) != nullptr) {
          rec.fused = true;
          p.fused = 1;
          if (!use_row) p.split_major = 1;
        } else {
          // (no counters while the stream records a graph: two launches now,
          // and a later call should ask again rather than remember this plan)
          rec.remember = false;
        }
      }
    }
    rec.pi_off = rec.need = 0;
    if (p.nsplit > 1) {
      const size_t slots = (size_t)nrows * (size_t)p.nsplit;
      rec.pi_off = (slots * accsz + 255) & ~(size_t)255;
      rec.need = rec.pi_off + slots * 8;
      if (noalloc && scratch_skip + rec.need > ga_static_scratch_bytes)
        return ga_err_fmt(ctx->err, GA_XLARGE_ERROR,
                          "GpuReduction_call_noalloc: this reduction is split into %zu partial "
                          "results that take %zu bytes; the static scratch array holds %zu",
                          slots, scratch_skip + rec.need, (size_t)ga_static_scratch_bytes);
    }
    rec.k1 = trows ? &var->trows : srows ? &var->srows : use_row ? (wrows ? &var->wrows : &var->row) : &var->col;
    rec.k2 = nullptr;
    rec.groups = groups;
    rec.lds_bytes = lds_bytes;
    rec.fin_groups = 0;
    if (p.nsplit > 1 && !rec.fused) {
      rec.k2 = p.split_major ? &var->fin_cols : &var->fin;
      rec.fin_groups = (size_t)(p.split_major ? (nrows + 63) / 64 : (nrows + 3) / 4);
    }
    return GA_NO_ERROR;
  }
};

// The launches of a planned call.  `plan` is the kernels' by-value plan
// argument; partials of a split reduction live in the context's scratch buffer
// (in the device's static scratch array for a call that may not allocate):
// values first, indices after, both 8-byte aligned, `scratch_skip` bytes in.
int issue_launches(gpucontext *ctx, const launch_rec &rec, const void *plan, unsigned K, const src_view *srcs,
                   GpuArray *d0, GpuArray *d1, void *const *scalars, unsigned nscalars, bool noalloc,
                   size_t scratch_skip) {
  gpudata *scratch = nullptr;
  if (noalloc) {
    const char *why = "";
    scratch = ga_hip_static_scratch_buf(ctx, &why);
    if (scratch == nullptr)
      return ga_err_fmt(ctx->err, GA_IMPL_ERROR,
                        "GpuReduction_call_noalloc: the static scratch array was not found on "
                        "this device when the context was made (%s)", why);
  } else {
    scratch = ga_hip_scratch(ctx, scratch_skip + (rec.need > 16 ? rec.need : 16));
  }
  if (scratch == nullptr) return ctx->err->code;
  // the counters of a launch that finishes itself; a pointer the kernels take but do not use otherwise
  gpudata *done = rec.fused ? ga_hip_redux_counters(ctx) : scratch;
  if (done == nullptr) return ctx->err->code;

  // A destination the operation does not write still needs a valid pointer.
  gpudata *d0b = d0 ? d0->data : scratch, *d1b = d1 ? d1->data : scratch;
  size_t d0_off = d0 ? d0->offset : 0, d1_off = d1 ? d1->offset : 0;
  size_t s_off[RD_MAXSRC];
  // The two scratch views are passed as (buffer) arguments; the index part
  // starts pi_off bytes in, which the kernels receive through a second
  // gpudata wrapping the same memory (a kernel argument is only read through
  // the leading {device pointer, context} of a gpudata).
  struct { void *devptr; gpucontext *ctx; } pv_view = {(char *)scratch->devptr + scratch_skip, ctx};
  struct { void *devptr; gpucontext *ctx; } pi_view = {(char *)scratch->devptr + scratch_skip + rec.pi_off, ctx};
  constexpr unsigned MAXSCALARS = 32;
  void *fixed[2 * RD_MAXSRC + 8 + MAXSCALARS];
  std::vector<void *> many;
  void **args = fixed;
  if (nscalars > MAXSCALARS) {
    many.resize(2 * RD_MAXSRC + 8 + nscalars);
    args = many.data();
  }
  unsigned n = 0;
  for (unsigned q = 0; q < K; q++) {
    s_off[q] = srcs[q].a->offset;
    args[n++] = srcs[q].a->data;
    args[n++] = &s_off[q];
  }
  args[n++] = d0b;
  args[n++] = &d0_off;
  args[n++] = d1b;
  args[n++] = &d1_off;
  args[n++] = &pv_view;
  args[n++] = &pi_view;
  args[n++] = done;
  args[n++] = const_cast<void *>(plan);
  for (unsigned i = 0; i < nscalars; i++) args[n++] = scalars[i];
  size_t ls = 256, g1 = rec.groups, g2 = rec.fin_groups;
  int err;
  if ((err = GpuKernel_call(rec.k1, 1, &g1, &ls, rec.lds_bytes, args)) != GA_NO_ERROR) return err;
  if (rec.k2 != nullptr && (err = GpuKernel_call(rec.k2, 1, &g2, &ls, 0, args)) != GA_NO_ERROR) return err;
  return GA_NO_ERROR;
}

// The key of a call (see call_memo); 0 when the call is not one to remember:
// more dims or sources than the key has room for, or an argument that the
// checks of the planned path must report.
unsigned memo_key(GpuReduction *gr, const GpuArray *d0, const GpuArray *d1, unsigned nd, const size_t *dims,
                  const src_view *srcs, unsigned reduxLen, const int *reduxList, bool noalloc,
                  size_t scratch_skip, int64_t *key) {
  const unsigned K = gr->nsrc();
  if (nd == 0 || nd > 8 || K > 4 || reduxLen == 0 || reduxLen > nd || reduxList == nullptr) return 0;
  gpucontext *ctx = gr->ctx;
  unsigned n = 0;
  key[n++] = (int64_t)nd | ((int64_t)reduxLen << 8) | ((int64_t)K << 16) | ((int64_t)(noalloc ? 1 : 0) << 24) |
             ((int64_t)(d0 ? 1 : 0) << 25) | ((int64_t)(d1 ? 1 : 0) << 26);
  key[n++] = (int64_t)scratch_skip;
  key[n++] = (int64_t)ga_hip_tuning(ctx)->generation;
  for (unsigned i = 0; i < nd; i++) key[n++] = (int64_t)dims[i];
  for (unsigned i = 0; i < reduxLen; i++) key[n++] = reduxList[i];
  for (unsigned q = 0; q < K; q++) {
    const GpuArray *a = srcs[q].a;
    if (a == nullptr || a->data == nullptr || gpudata_context(a->data) != ctx) return 0;
    for (unsigned i = 0; i < nd; i++) key[n++] = srcs[q].strides[i];
    size_t sz = 0, readable = 0;
    uintptr_t base = 0;
    ga_hip_buf_info(a->data, &base, &sz, &readable);
    key[n++] = (int64_t)a->offset;
    key[n++] = (int64_t)(unsigned)a->flags | ((int64_t)a->typecode << 32);
    key[n++] = (int64_t)(base & 255u);
    key[n++] = (int64_t)sz;
    key[n++] = (int64_t)readable;
  }
  for (const GpuArray *d : {d0, d1}) {
    if (d == nullptr) continue;
    if (d->data == nullptr || gpudata_context(d->data) != ctx || d->nd > 8) return 0;
    key[n++] = (int64_t)d->nd | ((int64_t)d->typecode << 32);
    key[n++] = (int64_t)(unsigned)d->flags;
    for (unsigned i = 0; i < d->nd; i++) {
      key[n++] = (int64_t)d->dimensions[i];
      key[n++] = (int64_t)d->strides[i];
    }
    size_t sz = 0, readable = 0;
    uintptr_t base = 0;
    ga_hip_buf_info(d->data, &base, &sz, &readable);
    key[n++] = (int64_t)d->offset;
    key[n++] = (int64_t)(base & 255u);
  }
  return n;   // at most 3 + 8 + 8 + 4 * (8 + 5) + 2 * (2 + 16 + 2) = 111
}

int reduce_launch(GpuReduction *gr, GpuArray *d0, GpuArray *d1, unsigned nd, const size_t *dims,
                  const src_view *srcs, void *const *scalars, unsigned nscalars,
                  unsigned reduxLen, const int *reduxList, bool noalloc = false, size_t scratch_skip = 0) {
  gpucontext *ctx = gr->ctx;
  // REDUX_MEMO: 0 plans every call anew; 2 plans every call anew and compares
  // with the kept plan where there is one (a difference is a planner input
  // missing from the key: the process stops)
  const unsigned long mode = TUNE(ga_hip_tuning(ctx), REDUX_MEMO, 1);
  if (!gr->info.has_d0) d0 = nullptr;
  if (!gr->info.has_d1) d1 = nullptr;
  int64_t key[MEMO_KEYMAX];
  const unsigned nkey = mode ? memo_key(gr, d0, d1, nd, dims, srcs, reduxLen, reduxList, noalloc,
                                        scratch_skip, key) : 0;
  call_memo *hit = nullptr;
  if (nkey != 0) {
    for (size_t i = 0; i < gr->memo.size(); i++) {
      call_memo &m = gr->memo[i];
      if (m.nkey == nkey && memcmp(m.key, key, nkey * sizeof(int64_t)) == 0) {
        hit = &m;
        break;
      }
    }
  }
  if (hit != nullptr && mode != 2)
    return issue_launches(ctx, hit->rec, hit->plan.data(), gr->nsrc(), srcs, d0, d1, scalars, nscalars,
                          noalloc, scratch_skip);
  reduction_call call(gr, d0, d1, nd, dims, srcs, scalars, nscalars, reduxLen, reduxList, noalloc, scratch_skip);
  call.plan_only = true;
  int err = call.run();
  if (err != GA_NO_ERROR || !call.planned) {
    if (hit != nullptr) {
      fprintf(stderr, "libgpuarray: a remembered reduction plan exists for a call that planning refuses (%d)\n", err);
      abort();
    }
    return err;
  }
  if (hit != nullptr) {
    const launch_rec &a = hit->rec, &b = call.rec;
    if (hit->plan != call.plan() || a.k1 != b.k1 || a.k2 != b.k2 || a.groups != b.groups ||
        a.fin_groups != b.fin_groups || a.lds_bytes != b.lds_bytes || a.pi_off != b.pi_off ||
        a.need != b.need || a.fused != b.fused) {
      fprintf(stderr, "libgpuarray: a remembered reduction plan differs from the plan made anew\n");
      abort();
    }
  } else if (nkey != 0 && call.rec.remember) {
    // a few entries, replaced in turn once all are taken
    const bool room = gr->memo.size() < MEMO_ENTRIES;
    if (room) gr->memo.emplace_back();
    call_memo &m = room ? gr->memo.back() : gr->memo[gr->memo_next++ % MEMO_ENTRIES];
    m.nkey = nkey;
    memcpy(m.key, key, nkey * sizeof(int64_t));
    m.plan = call.plan();
    m.rec = call.rec;
  }
  return issue_launches(ctx, call.rec, call.plan().data(), gr->nsrc(), srcs, d0, d1, scalars, nscalars,
                        noalloc, scratch_skip);
}

}  // namespace

extern "C" {

// Full kernel text of one variant, for checks that have no device.  The
// caller frees the result.
GPUARRAY_PUBLIC char *ga_reduction_gen_source(int op, int src_tc, int d0_tc, int d1_tc,
                                              unsigned int G, unsigned int V, unsigned int U) {
  GpuReduction *gr = nullptr;
  if (make_plain_operator(&gr, nullptr, ga_global_err, (ga_reduce_op)op, src_tc) != GA_NO_ERROR)
    return nullptr;
  // bits 8.. of V carry the element step of strided loads (0 means 1), bits
  // 8.. of U the rows per batch of redux_wrows (0 means 1), bits 16.. of G its
  // lanes per row (0 means 64), bits 16..23 of V the outputs per lane of
  // redux_col, bit 24 of V its order of groups that keeps neighbours on one die
  const unsigned ES = ((V >> 8) & 0xffu) ? ((V >> 8) & 0xffu) : 1;
  const unsigned cv_bits = (V >> 16) & 0xffu;
  const unsigned xcd_bit = (V >> 24) & 1u;
  V &= 0xffu;
  std::string s;
  variant_spec vs = {d0_tc, d1_tc, G & 0xffffu, V, U & 0xffu,
                     ((U >> 16) & 0xffu ? 1u : 3u) | (((U >> 24) & 1u) ? 4u : 0u) |
                         (((U >> 25) & 1u) ? 8u : 0u) | (((U >> 26) & 1u) ? 64u : 0u) |
                         (((U >> 27) & 1u) ? 128u : 0u) | (((U >> 28) & 1u) ? 512u : 0u) |
                         (((U >> 29) & 1u) ? 1024u : 0u) | (((U >> 30) & 1u) ? 2048u : 0u) |
                         (((U >> 31) & 1u) ? 4096u : 0u) | (xcd_bit ? 8192u : 0u) | 48u | 256u, ES, 1,
                     ((U >> 8) & 0xffu) ? ((U >> 8) & 0xffu) : 1,
                     (G >> 16) ? (G >> 16) : 64, cv_bits ? cv_bits : 1,
                     ((U >> 16) & 0xffu) ? ((U >> 16) & 0xffu) : 1};
  if ((U >> 29) & 1u) {   // redux_trows: V is the row length
    vs.TE = V;
    vs.V = 1;
  }
  const int err = variant_source(gr, vs, s, ga_global_err);
  delete gr;
  return err == GA_NO_ERROR ? strdup(s.c_str()) : nullptr;
}

// The same for an operator with an expression; vecmask as in variant_spec.
GPUARRAY_PUBLIC char *ga_mapreduce_gen_source(int op, const char *reduce_expr, const char *neutral,
                                              int acc_tc, const char *preamble, const char *map_expr,
                                              unsigned int n, const gpuelemwise_arg *args, int d0_tc,
                                              unsigned int G, unsigned int V, unsigned int U,
                                              unsigned int vecmask) {
  GpuReduction *gr = nullptr;
  if (make_operator(&gr, nullptr, ga_global_err, (ga_reduce_op)op, reduce_expr, neutral, acc_tc,
                    preamble, map_expr, n, args) != GA_NO_ERROR)
    return nullptr;
  std::string s;
  // bit 27 of U: redux_wrows in place of redux_row (G = 64 only)
  variant_spec vs = {d0_tc, GA_LONG, G, V, U & 0xffu, 3 | 48u | 256u | (((U >> 27) & 1u) ? 128u : 0u),
                     1, vecmask, 1, 64, 1, 1};
  const int err = variant_source(gr, vs, s, ga_global_err);
  delete gr;
  return err == GA_NO_ERROR ? strdup(s.c_str()) : nullptr;
}

int GpuReduction_new(GpuReduction **grp, gpucontext *ctx, ga_reduce_op op, unsigned ndf,
                     unsigned ndr, int s0Typecode, int flags) {
  (void)ndf; (void)ndr; (void)flags;
  if (grp == nullptr) return GA_INVALID_ERROR;
  *grp = nullptr;
  if (ctx == nullptr) return ga_err_set(ga_global_err, GA_INVALID_ERROR, "GpuReduction_new: no context");
  return make_plain_operator(grp, ctx, ctx->err, op, s0Typecode);
}

int GpuReduction_new_map(GpuReduction **grp, gpucontext *ctx, ga_reduce_op op,
                         const char *reduce_expr, const char *neutral, int accTypecode,
                         const char *preamble, const char *map_expr, unsigned int n,
                         const gpuelemwise_arg *args, int flags) {
  (void)flags;
  if (grp == nullptr) return GA_INVALID_ERROR;
  *grp = nullptr;
  if (ctx == nullptr)
    return ga_err_set(ga_global_err, GA_INVALID_ERROR, "GpuReduction_new_map: no context");
  return make_operator(grp, ctx, ctx->err, op, reduce_expr, neutral, accTypecode, preamble,
                       map_expr, n, args);
}

void GpuReduction_free(GpuReduction *gr) {
  if (gr == nullptr) return;
  GpuReduction_free(gr->fold_op);
  for (auto &kv : gr->variants) {
    GpuKernel_clear(&kv.second.row);
    GpuKernel_clear(&kv.second.col);
    GpuKernel_clear(&kv.second.fin);
    if (kv.second.fin_cols.k != nullptr) GpuKernel_clear(&kv.second.fin_cols);
    if (kv.second.wrows.k != nullptr) GpuKernel_clear(&kv.second.wrows);
    if (kv.second.srows.k != nullptr) GpuKernel_clear(&kv.second.srows);
    if (kv.second.trows.k != nullptr) GpuKernel_clear(&kv.second.trows);
    if (kv.second.pcols.k != nullptr) GpuKernel_clear(&kv.second.pcols);
  }
  delete gr;
}

// Reducing the leading dims of a dense array over short kept rows in one
// launch (redux_pcols): the array is walked as one run of 16-byte chunks by
// groups of L lanes, L chunks being a whole number of kept rows, so that a
// lane meets the same outputs at the same places of every chunk it loads; the
// groups' partial rows (a few hundred times F values) are combined by the
// group that finishes last.  Taken when such an L exists (F / gcd(F, elements
// per chunk) <= 256), the first element sits on a 16-byte boundary, the
// counters of single-launch reductions can be had and the caller may allocate;
// everything else is left to fold_rows below.  Measured on MI355X, kernel
// time, folded rows (two or three launches) against this, sums over axis 0:
// (2^22, 10) floats 31.0 -> 29.6 us, (2^24, 3) 35.7 -> 36.3, (2^20, 17) 17.6 ->
// 17.3, (2^20, 63) 47.3 -> 43.9, (2^22, 32) 81.5 -> 77.5 (87 % of peak),
// (2^24, 6) halves 40.0 -> 36.0, integer maximum of (2^22, 10) 30.6 -> 29.7;
// two groups per compute unit measured slower (31.7 us for the first shape).
static int pcols_call(GpuReduction *gr, GpuArray *d0, const GpuArray *s0, unsigned reduxLen,
                      const int *reduxList, bool *done, bool noalloc = false) {
  *done = false;
  gpucontext *ctx = gr->ctx;
  const ga_tuning *tn = ga_hip_tuning(ctx);
  // (REDUX_FUSED = 0 asks for reductions that do not end in their own launch)
  if (TUNE(tn, REDUX_PCOLS, 1) == 0 || TUNE(tn, REDUX_FUSED, 1) == 0 || gr->mapped || d0 == nullptr || s0->data == nullptr ||
      d0->data == nullptr || reduxLen == 0 || reduxLen >= s0->nd || !GpuArray_IS_C_CONTIGUOUS(s0) ||
      GpuArray_context(d0) != ctx || GpuArray_context(s0) != ctx || s0->typecode != gr->src_tc() ||
      !GpuArray_ISWRITEABLE(d0))
    return GA_NO_ERROR;
  const rd_kind kind = gr->info.kind;
  const int stc = s0->typecode;
  const bool regroupable = !gr->info.has_d1 &&
      (kind == K_SUM || kind == K_PROD || kind == K_AND || kind == K_OR || kind == K_XOR ||
       kind == K_ALL || kind == K_ANY || ((kind == K_MIN || kind == K_MAX) && is_int_type(stc)));
  if (!regroupable) return GA_NO_ERROR;
  // the reduced axes are one run of adjacent ones, [a0, a0 + reduxLen): the
  // leading dims (a0 = 0), or a middle run under O kept slabs
  std::array<char, 64> seen{};
  if (reduxLen > seen.size()) return GA_NO_ERROR;
  unsigned a0 = s0->nd;
  for (unsigned i = 0; i < reduxLen; i++) {
    if (reduxList[i] < 0 || (unsigned)reduxList[i] >= s0->nd) return GA_NO_ERROR;
    if ((unsigned)reduxList[i] < a0) a0 = (unsigned)reduxList[i];
  }
  if (a0 + reduxLen >= s0->nd) return GA_NO_ERROR;
  for (unsigned i = 0; i < reduxLen; i++) {
    const unsigned at = (unsigned)reduxList[i] - a0;
    if (at >= reduxLen || seen[at]) return GA_NO_ERROR;
    seen[at] = 1;
  }
  size_t O = 1, R = 1, F = 1;
  for (unsigned j = 0; j < s0->nd; j++) (j < a0 ? O : j < a0 + reduxLen ? R : F) *= s0->dimensions[j];
  const size_t es = gpuarray_get_elsize(stc), rowb = F * es;
  // (one kept element is a full reduction of a dense array: the planned path's ground)
  if (F < 2 || R < 2 || O == 0 || O * R * rowb < TUNE(tn, REDUX_FOLD_MIN_BYTES, 4u << 20)) return GA_NO_ERROR;
  // Slabs: one group each walks its slab as one run of chunks and writes the
  // slab's outputs itself - no partial results, no counter.  For slabs of whole
  // chunks that keep a group's lanes busy (4 KiB and more, up to 1 MiB), one
  // per compute unit and more - but not a few more than a whole number per
  // unit while that number is small: the stragglers then run alone ((524, 512,
  // 250) 67 % of peak this way, 69 with the column kernel; (262, 512, 500) 59 /
  // 69).  Measured on MI355X, sum over the middle axis of floats, column
  // kernel / this one: (10922, 512, 12) 67.1 -> 44.5 us (50 -> 75 % of peak),
  // (6553, 512, 20) 70 -> 80 %, (3971, 512, 33) 68 -> 80 %, (1008, 512, 130)
  // 67 -> 79 %, (655, 512, 200) 60 -> 77 %, (436, 512, 300) 65 -> 78 %,
  // (327, 512, 400) 68 -> 75 %.
  const size_t slabb = R * rowb;
  if (O > 1) {
    const size_t ncu = ga_hip_numprocs(ctx);
    const size_t rounds = O / ncu, over = O % ncu;
    if (TUNE(tn, REDUX_PSLABS, 1) == 0 || slabb % 16 != 0 || slabb < 4096 ||
        slabb > TUNE(tn, REDUX_PSLABS_MAX_BYTES, 1u << 20) ||
        O < TUNE(tn, REDUX_PSLABS_MIN_SLABS, ncu) || O > 0x7fffffffull ||
        (rounds <= 3 && over != 0 && over * 10 < ncu))
      return GA_NO_ERROR;
  }
  // The column kernel's own ground: kept rows of whole 16-byte pieces from 256
  // bytes on.  Between 256 and 512 bytes its second tile of 256 bytes is mostly
  // idle and this kernel is ahead (sums over axis 0, column kernel in two
  // launches / this one: (2^20, 72) floats 62.3 -> 52.0 us, 61 -> 73 % of peak,
  // (2^20, 36) doubles 62.0 -> 50.0, (2^18, 68) floats 20.9 -> 19.7; 19 MB of
  // rows of 72 floats 11.2 -> 11.7); rows of 256 bytes exactly are a tie.
  // (under slabs it has no second tile to spare: there every row length is taken)
  if (O == 1 && rowb % 16 == 0 && (rowb == 256 || rowb >= TUNE(tn, REDUX_PCOLS_COL_BYTES, 512))) return GA_NO_ERROR;
  if (es > 8 || 16 % es != 0 || d0->nd != s0->nd - reduxLen || d0->nd > (unsigned)RD_MAXD) return GA_NO_ERROR;
  for (unsigned j = 0; j < d0->nd; j++)
    if (d0->dimensions[j] != s0->dimensions[j < a0 ? j : reduxLen + j]) return GA_NO_ERROR;
  // the result's type must be one the operation accepts (the planned path reports what is wrong)
  const int d0_tc = d0->typecode;
  const bool logical = kind == K_ALL || kind == K_ANY, minmax = kind == K_MIN || kind == K_MAX;
  if ((minmax && d0_tc != stc) || ((kind == K_AND || kind == K_OR || kind == K_XOR || logical) && !is_int_type(d0_tc)) ||
      (!is_int_type(d0_tc) && !is_float_type(d0_tc)))
    return GA_NO_ERROR;
  const size_t accsz = logical ? 4 : acc_size_for(acc_typecode(gr, d0_tc));
  if (accsz != 4 && accsz != 8) return GA_NO_ERROR;
  // A lane keeps one accumulator per element of a chunk.  Up to 32 bytes of
  // them (four floats or doubles, four 64-bit sums of int32, eight float sums
  // of halves) this kernel wins; beyond, the elements are narrow and each is
  // taken out of its word and widened on its own, and the folded rows, whose
  // kernels take bytes four per instruction, are faster: 2^24 rows of 12 bytes
  // summed into 64-bit integers 68 us here against 43, of 6 int16 47 against 41.
  if (16 / es * accsz > 32) return GA_NO_ERROR;
  // L: the most lanes of 256 whose chunks are a whole number of kept rows
  const size_t pv = 16 / es;
  size_t g = F, h = pv;
  while (h) { const size_t t = g % h; g = h; h = t; }
  const size_t q = F / g;
  if (q > 256 || F > 65536) return GA_NO_ERROR;
  const size_t L = 256 / q * q;
  uintptr_t base = 0;
  size_t bufsz = 0, readable = 0;
  ga_hip_buf_info(s0->data, &base, &bufsz, &readable);
  const size_t bytes = R * rowb, chunks = (bytes + 15) / 16;   // of one slab
  if ((base + s0->offset) % 16 != 0 || s0->offset + O * chunks * 16 > readable) return GA_NO_ERROR;
  // (the counters are not to be had while the stream records a graph; a call
  // that may not allocate takes them only if an earlier call has made them)
  if (O == 1 && (noalloc ? !ga_hip_redux_counters_made(ctx) : ga_hip_redux_counters(ctx) == nullptr)) {
    if (noalloc)
      return ga_err_set(ctx->err, GA_UNSUPPORTED_ERROR,
                        "GpuReduction_call_noalloc: the kernels for arrays of this layout are not "
                        "built yet, and building them allocates; run GpuReduction_call once on "
                        "arrays of this layout first");
    return GA_NO_ERROR;
  }
  // groups: one per compute unit, each lane eight loads per batch
  const size_t ncu = ga_hip_numprocs(ctx), U = 8;
  size_t G = ncu * TUNE(tn, REDUX_PCOLS_PER_CU, 1);
  // The group that finishes last combines G partial rows by itself: that pays
  // while they are a few thousand values.
  // (256 groups, floats, one launch against folded rows in two: kept rows of 63,
  // 16 128 partial values, 43.9 against 47.3 us; of 250, 64 000 values, 52.8 against 46.7)
  if (O > 1) G = 1;   // a group per slab
  if (G * F > TUNE(tn, REDUX_PCOLS_MAX_PARTIALS, 20000)) return GA_NO_ERROR;
  size_t J = (chunks + G * L - 1) / (G * L);
  J = (J + U - 1) / U * U;
  if (O == 1) G = (chunks + L * J - 1) / (L * J);
  if (G < 1) G = 1;

  unsigned opts = TUNE(tn, REDUX_NT, 1) ? 1u : 0u;
  variant_spec vs = {d0_tc, GA_LONG, 64, 1, (unsigned)U, opts | 2048u, 1, 1, 1, 64, 1, 1};
  variant *var = nullptr;
  int err = get_variant(gr, vs, &var, !noalloc);
  if (err != GA_NO_ERROR) return err;
  std::vector<int64_t> planbuf(plan_bytes(1) / sizeof(int64_t), 0);
  rd_plan &p = *reinterpret_cast<rd_plan *>(planbuf.data());
  p.nf = (int)d0->nd;
  for (unsigned j = 0; j < d0->nd; j++) {
    p.fdim[j] = (int64_t)d0->dimensions[j];
    p.fd0str[j] = (int64_t)d0->strides[j];
  }
  if (p.nf == 0) {   // a 0-d result: one output
    p.nf = 1;
    p.fdim[0] = 1;
  }
  p.nrows = (int64_t)F;
  p.rtotal = (int64_t)R;
  p.upb = (int64_t)L;
  p.units = (int64_t)J;
  p.nsplit = (int)G;
  p.fused = 1;
  p.router = (int64_t)O;
  launch_rec rec;
  rec.k1 = &var->pcols;
  rec.groups = O * G;
  rec.fused = O == 1;
  rec.pi_off = O == 1 ? (G * F * accsz + 255) & ~(size_t)255 : 0;
  rec.need = O == 1 ? rec.pi_off + 16 : 0;
  const src_view src = {s0, (const int64_t *)s0->strides};
  if (noalloc && rec.need > ga_static_scratch_bytes)
    return ga_err_fmt(ctx->err, GA_XLARGE_ERROR,
                      "GpuReduction_call_noalloc: the partial results of this reduction take %zu "
                      "bytes; the static scratch array holds %zu", rec.need, (size_t)ga_static_scratch_bytes);
  err = issue_launches(ctx, rec, planbuf.data(), 1, &src, d0, nullptr, nullptr, 0, noalloc, 0);
  if (err == GA_NO_ERROR) *done = true;
  return err;
}

// Reducing the leading dims of a dense array whose trailing (kept) dims are
// short or leave rows off a 16-byte boundary - the sum over a batch of rows of
// 10 floats, say.  With lanes along the kept dims a load fetches a few
// elements, or one.  Every m rows are taken as one row of m F elements
// instead, with m F elements a multiple of the load and wide enough for a
// group: the column kernel then runs with full 16-byte loads over (R / m, m F),
// and a second, tiny call folds the m copies of every output.  For operations
// whose result does not depend on how the elements are grouped (sum, product,
// bitwise and logical ones, integer minimum and maximum) on arrays of 4 MiB
// and more, when a suitable m divides the row count.
// Measured on MI355X, kernel time of all launches: sum over axis 0 of
// (2^22, 10) floats 72 -> 37 us, of (2^24, 3) 92 -> 40, of (65536, 1001)
// 57 -> 49, over axes (0, 1) of (4096, 4096, 4) 148 -> 50.  The width of the
// folded rows hardly matters (2 KiB to 64 KiB: within 3 us of each other).
// Returns GA_NO_ERROR with *done = true when the reduction was carried out.
static int fold_rows(GpuReduction *gr, GpuArray *d0, const GpuArray *s0, unsigned reduxLen,
                     const int *reduxList, bool *done, bool noalloc = false) {
  *done = false;
  gpucontext *ctx = gr->ctx;
  const ga_tuning *tn = ga_hip_tuning(ctx);
  if (TUNE(tn, REDUX_FOLD, 1) == 0 || gr->mapped || d0 == nullptr || reduxLen == 0 ||
      reduxLen >= s0->nd || !GpuArray_IS_C_CONTIGUOUS(s0) || GpuArray_context(d0) != ctx)
    return GA_NO_ERROR;
  const rd_kind kind = gr->info.kind;
  const int stc = s0->typecode;
  const bool regroupable = !gr->info.has_d1 &&
      (kind == K_SUM || kind == K_PROD || kind == K_AND || kind == K_OR || kind == K_XOR ||
       kind == K_ALL || kind == K_ANY || ((kind == K_MIN || kind == K_MAX) && is_int_type(stc)));
  if (!regroupable) return GA_NO_ERROR;
  // the reduced axes are one run of adjacent ones, [a0, a0 + reduxLen), and
  // dims are kept behind it: O slabs (the dims in front of the run) of R rows
  // of F elements each
  unsigned a0 = s0->nd;
  for (unsigned i = 0; i < reduxLen; i++) {
    if (reduxList[i] < 0 || (unsigned)reduxList[i] >= s0->nd) return GA_NO_ERROR;
    if ((unsigned)reduxList[i] < a0) a0 = (unsigned)reduxList[i];
  }
  if (a0 + reduxLen >= s0->nd) return GA_NO_ERROR;
  std::vector<char> seen(reduxLen, 0);
  for (unsigned i = 0; i < reduxLen; i++) {
    const unsigned at = (unsigned)reduxList[i] - a0;
    if (at >= reduxLen || seen[at]) return GA_NO_ERROR;
    seen[at] = 1;
  }
  size_t O = 1, R = 1, F = 1;
  for (unsigned j = 0; j < s0->nd; j++) (j < a0 ? O : j < a0 + reduxLen ? R : F) *= s0->dimensions[j];
  if (a0 > 0 && TUNE(tn, REDUX_FOLD, 1) == 2) return GA_NO_ERROR;   // (2: leading axes only)
  // (slabs from 32 MiB on: (16, 16384, 42) floats, 42 MB, 18.6 -> 15.0 us, (8, 65536, 33) 25.7 -> 19.1;
  // below, (256, 1024, 30), 30 MB, 14.0 -> 14.3, (8, 8192, 33), 8 MB, 9.4 -> 12.0)
  if (a0 > 0 && O * R * F * gpuarray_get_elsize(stc) < TUNE(tn, REDUX_FOLD_SLAB_MIN_BYTES, 32u << 20))
    return GA_NO_ERROR;
  const size_t es = gpuarray_get_elsize(stc), rowb = F * es;
  if (O * R * rowb < TUNE(tn, REDUX_FOLD_MIN_BYTES, 4u << 20) || F == 0 || O == 0) return GA_NO_ERROR;
  if (rowb % 16 == 0 && rowb >= 256) return GA_NO_ERROR;
  // d0 must have the kept dims' shape (the launch below checks the rest)
  if (d0->nd != s0->nd - reduxLen) return GA_NO_ERROR;
  for (unsigned j = 0; j < d0->nd; j++)
    if (d0->dimensions[j] != s0->dimensions[j < a0 ? j : reduxLen + j]) return GA_NO_ERROR;
  // m: rows per folded row
  size_t g = rowb, h = 16;
  while (h) { size_t t = g % h; g = h; h = t; }      // g = gcd(rowb, 16)
  const size_t m0 = 16 / g;
  // Folded rows of 256 KiB where the row count allows it: the first call then
  // needs no split (or a few pieces that end in its own launch), and the second
  // combines a few thousand partial rows.  Narrower folds for smaller arrays.
  // Sum over axis 0, folds of 4 KiB / 256 KiB, all launches: (2^22, 10) floats
  // 35.5 / 31.6 us (three launches / two), (2^24, 3) 38.9 / 34.1, (65536, 1001)
  // 49.3 / 46.1, (4096, 4096, 4) over two axes 50.1 / 43.4, (2^20, 17) 20.2 / 16.9.
  // The search is remembered per (row count, row bytes, widest fold), "no
  // fold" included: a row count that no candidate divides (a prime one, say)
  // walks through every candidate, tens of thousands of them, which takes
  // longer than the kernels that follow; that is paid once per shape, not per
  // call.  (m0 must divide the row count for any candidate to.)
  size_t m = 0;
  const size_t widest = TUNE(tn, REDUX_FOLD_BYTES, 262144);
  const std::array<size_t, 3> memo_key = {R, rowb, widest};
  auto memo = gr->fold_memo.find(memo_key);
  if (memo != gr->fold_memo.end()) {
    m = memo->second;
  } else {
    if (R % m0 == 0)
      for (size_t width = widest; m == 0 && width >= 4096; width /= 8) {
        const size_t t0 = (width + m0 * rowb - 1) / (m0 * rowb);
        for (size_t t = t0; t * m0 <= 65536; t++)
          if (R % (t * m0) == 0 && R / (t * m0) >= 64) { m = t * m0; break; }
      }
    if (gr->fold_memo.size() >= 256) gr->fold_memo.clear();
    gr->fold_memo[memo_key] = m;
  }
  if (m <= 1) return GA_NO_ERROR;

  // type of the folded partial results: the accumulator's (a half result is summed in float)
  int tmp_tc = acc_typecode(gr, d0->typecode);
  if (tmp_tc == GA_HALF) tmp_tc = GA_FLOAT;
  if (noalloc && (gr->fold_op == nullptr || gr->fold_tc != tmp_tc))
    return ga_err_set(ctx->err, GA_UNSUPPORTED_ERROR,
                      "GpuReduction_call_noalloc: the kernels for arrays of this layout are not "
                      "built yet, and building them allocates; run GpuReduction_call once on "
                      "arrays of this layout first");
  if (gr->fold_op == nullptr || gr->fold_tc != tmp_tc) {
    GpuReduction_free(gr->fold_op);
    gr->fold_op = nullptr;
    int err = make_plain_operator(&gr->fold_op, ctx, ctx->err, gr->op, tmp_tc);
    if (err != GA_NO_ERROR) return err;
    gr->fold_tc = tmp_tc;
  }
  // The folded partial results take the start of the context's scratch
  // buffer (which is never handed to anybody else, also not after it has been
  // outgrown: a graph that recorded these launches may run them again); the
  // two calls below put their own partials behind them.
  const size_t tmp_len = O * m * F;
  const size_t skip = (tmp_len * gpuarray_get_elsize(tmp_tc) + 255) & ~(size_t)255;
  gpudata *scr = nullptr;
  if (noalloc) {
    const char *why = "";
    scr = ga_hip_static_scratch_buf(ctx, &why);
    if (scr == nullptr)
      return ga_err_fmt(ctx->err, GA_IMPL_ERROR,
                        "GpuReduction_call_noalloc: the static scratch array was not found on "
                        "this device when the context was made (%s)", why);
    if (skip + 16 > ga_static_scratch_bytes)
      return ga_err_fmt(ctx->err, GA_XLARGE_ERROR,
                        "GpuReduction_call_noalloc: the folded partial results of this reduction "
                        "take %zu bytes; the static scratch array holds %zu",
                        skip, (size_t)ga_static_scratch_bytes);
  } else {
    scr = ga_hip_scratch(ctx, skip + 16);
  }
  if (scr == nullptr) return ctx->err->code;
  GpuArray tmp;
  const ssize_t tmp_stride = (ssize_t)gpuarray_get_elsize(tmp_tc);
  int err = GpuArray_fromdata(&tmp, scr, 0, tmp_tc, 1, &tmp_len, &tmp_stride, 1);
  if (err != GA_NO_ERROR) return err;
  if (O == 1) {
    // first call: (R / m, m F) over axis 0 into tmp
    const size_t dims1[2] = {R / m, m * F};
    const int64_t str1[2] = {(int64_t)(m * rowb), (int64_t)es};
    const src_view src = {s0, str1};
    const int axis0 = 0;
    err = reduce_launch(gr, &tmp, nullptr, 2, dims1, &src, nullptr, 0, 1, &axis0, noalloc, skip);
  } else {
    // the same per slab: (O, R / m, m F) over axis 1 into tmp as (O, m F)
    GpuArray_clear(&tmp);
    const size_t tdims[2] = {O, m * F};
    const ssize_t tstr[2] = {(ssize_t)(m * F) * tmp_stride, tmp_stride};
    err = GpuArray_fromdata(&tmp, scr, 0, tmp_tc, 2, tdims, tstr, 1);
    if (err != GA_NO_ERROR) return err;
    const size_t dims1[3] = {O, R / m, m * F};
    const int64_t str1[3] = {(int64_t)(R * rowb), (int64_t)(m * rowb), (int64_t)es};
    const src_view src = {s0, str1};
    const int axis1 = 1;
    err = reduce_launch(gr, &tmp, nullptr, 3, dims1, &src, nullptr, 0, 1, &axis1, noalloc, skip);
  }
  if (err == GA_NO_ERROR) {
    // second call: tmp as (slab dims..., m, dims kept behind the run...) over
    // the axis of the m copies into d0
    std::vector<size_t> dims2(1 + d0->nd);
    std::vector<int64_t> str2(1 + d0->nd);
    const size_t tes = gpuarray_get_elsize(tmp_tc);
    size_t run = tes;
    for (unsigned j = d0->nd + 1; j-- > 0;) {
      dims2[j] = j < a0 ? d0->dimensions[j] : j == a0 ? m : d0->dimensions[j - 1];
      str2[j] = (int64_t)run;
      run *= dims2[j];
    }
    const src_view src = {&tmp, str2.data()};
    const int axis = (int)a0;
    err = reduce_launch(gr->fold_op, d0, nullptr, 1 + d0->nd, dims2.data(), &src, nullptr, 0, 1, &axis,
                        noalloc, skip);
  }
  GpuArray_clear(&tmp);
  if (err == GA_NO_ERROR) *done = true;
  return err;
}

// Reducing leading AND trailing dims of a dense array around kept ones when
// the trailing reduced run is short - per-channel sums over (batch, channel,
// a small height x width): the bias gradient of a convolution.  One kernel
// would walk reduced rows of a few dozen elements that lie a whole slab
// apart.  Done in two calls instead: the leading dims of (A, K B) go first,
// with the column kernel at full load width, into K B partial results, and
// the short trailing run of those (1 / A of the input) second.  For the
// operations that may be regrouped, on 4 MiB and more, when the trailing run
// has at most 4 KiB.  Measured on MI355X, sums of floats, kernel time of all
// launches, one call / two: (64, 52428, 20) over axes (0, 2) 215.5 -> 46.1 us
// (16 -> 73 % of peak), (64, 87381, 12) 147.6 -> 48.5, (256, 2048, 49) 34.6 ->
// 23.5, (64, 1024, 196) 21.1 -> 13.8, (64, 8065, 130) 75.7 -> 52.4, (64, 5242,
// 200) 53.7 -> 45.6, (64, 3495, 300) 52.3 -> 46.7, (16, 65536, 33) 40.4 ->
// 30.2; from 400 floats on the two are within 2 us of each other up to 8 KiB.
// Returns GA_NO_ERROR with *done = true when the reduction was carried out.
static int outer_then_inner(GpuReduction *gr, GpuArray *d0, const GpuArray *s0, unsigned reduxLen,
                            const int *reduxList, bool *done, bool noalloc = false) {
  *done = false;
  gpucontext *ctx = gr->ctx;
  const ga_tuning *tn = ga_hip_tuning(ctx);
  const size_t max_inner = TUNE(tn, REDUX_OUTER_FIRST, 4096);
  if (max_inner == 0 || gr->mapped || d0 == nullptr || reduxLen < 2 || reduxLen >= s0->nd ||
      s0->nd > 16 || !GpuArray_IS_C_CONTIGUOUS(s0) || GpuArray_context(d0) != ctx)
    return GA_NO_ERROR;
  const rd_kind kind = gr->info.kind;
  const int stc = s0->typecode;
  const bool regroupable = !gr->info.has_d1 &&
      (kind == K_SUM || kind == K_PROD || kind == K_AND || kind == K_OR || kind == K_XOR ||
       kind == K_ALL || kind == K_ANY || ((kind == K_MIN || kind == K_MAX) && is_int_type(stc)));
  if (!regroupable) return GA_NO_ERROR;
  // the reduced axes are a leading run [0, a) and a trailing run [b, nd), both non-empty
  bool reduced[16] = {};
  for (unsigned i = 0; i < reduxLen; i++) {
    if (reduxList[i] < 0 || (unsigned)reduxList[i] >= s0->nd || reduced[reduxList[i]]) return GA_NO_ERROR;
    reduced[reduxList[i]] = true;
  }
  unsigned a = 0, b = s0->nd;
  while (a < s0->nd && reduced[a]) a++;
  while (b > a && reduced[b - 1]) b--;
  if (a == 0 || b == s0->nd || a >= b || a + (s0->nd - b) != reduxLen) return GA_NO_ERROR;
  size_t A = 1, K = 1, B = 1;
  for (unsigned j = 0; j < s0->nd; j++) (j < a ? A : j < b ? K : B) *= s0->dimensions[j];
  const size_t es = gpuarray_get_elsize(stc);
  if (A < 2 || B < 2 || K == 0 || B * es > max_inner ||
      A * K * B * es < TUNE(tn, REDUX_FOLD_MIN_BYTES, 4u << 20))
    return GA_NO_ERROR;
  // d0 must have the kept dims' shape (the launch below checks the rest)
  if (d0->nd != b - a) return GA_NO_ERROR;
  for (unsigned j = 0; j < d0->nd; j++)
    if (d0->dimensions[j] != s0->dimensions[a + j]) return GA_NO_ERROR;

  // type of the partial results: the accumulator's (a half result is summed in float)
  int tmp_tc = acc_typecode(gr, d0->typecode);
  if (tmp_tc == GA_HALF) tmp_tc = GA_FLOAT;
  if (noalloc && (gr->fold_op == nullptr || gr->fold_tc != tmp_tc))
    return ga_err_set(ctx->err, GA_UNSUPPORTED_ERROR,
                      "GpuReduction_call_noalloc: the kernels for arrays of this layout are not "
                      "built yet, and building them allocates; run GpuReduction_call once on "
                      "arrays of this layout first");
  if (gr->fold_op == nullptr || gr->fold_tc != tmp_tc) {
    GpuReduction_free(gr->fold_op);
    gr->fold_op = nullptr;
    int err = make_plain_operator(&gr->fold_op, ctx, ctx->err, gr->op, tmp_tc);
    if (err != GA_NO_ERROR) return err;
    gr->fold_tc = tmp_tc;
  }
  // The partial results take the start of the context's scratch buffer (see
  // fold_rows); the two calls below put their own partials behind them.
  const size_t tes = gpuarray_get_elsize(tmp_tc);
  const size_t tmp_len = K * B;
  const size_t skip = (tmp_len * tes + 255) & ~(size_t)255;
  gpudata *scr = nullptr;
  if (noalloc) {
    const char *why = "";
    scr = ga_hip_static_scratch_buf(ctx, &why);
    if (scr == nullptr)
      return ga_err_fmt(ctx->err, GA_IMPL_ERROR,
                        "GpuReduction_call_noalloc: the static scratch array was not found on "
                        "this device when the context was made (%s)", why);
    if (skip + 16 > ga_static_scratch_bytes)
      return ga_err_fmt(ctx->err, GA_XLARGE_ERROR,
                        "GpuReduction_call_noalloc: the partial results of this reduction take "
                        "%zu bytes; the static scratch array holds %zu",
                        skip, (size_t)ga_static_scratch_bytes);
  } else {
    scr = ga_hip_scratch(ctx, skip + 16);
  }
  if (scr == nullptr) return ctx->err->code;
  GpuArray tmp;
  const ssize_t tmp_stride = (ssize_t)tes;
  int err = GpuArray_fromdata(&tmp, scr, 0, tmp_tc, 1, &tmp_len, &tmp_stride, 1);
  if (err != GA_NO_ERROR) return err;
  {
    // first call: (A, K B) over axis 0 into tmp
    const size_t dims1[2] = {A, K * B};
    const int64_t str1[2] = {(int64_t)(K * B * es), (int64_t)es};
    const src_view src = {s0, str1};
    const int axis0 = 0;
    err = reduce_launch(gr, &tmp, nullptr, 2, dims1, &src, nullptr, 0, 1, &axis0, noalloc, skip);
  }
  if (err == GA_NO_ERROR) {
    // second call: tmp as (kept dims..., B) over its last axis into d0
    std::vector<size_t> dims2(d0->nd + 1);
    std::vector<int64_t> str2(d0->nd + 1);
    size_t run = tes;
    for (unsigned j = d0->nd + 1; j-- > 0;) {
      dims2[j] = j == d0->nd ? B : d0->dimensions[j];
      str2[j] = (int64_t)run;
      run *= dims2[j];
    }
    const src_view src = {&tmp, str2.data()};
    const int axis = (int)d0->nd;
    err = reduce_launch(gr->fold_op, d0, nullptr, d0->nd + 1, dims2.data(), &src, nullptr, 0, 1, &axis,
                        noalloc, skip);
  }
  GpuArray_clear(&tmp);
  if (err == GA_NO_ERROR) *done = true;
  return err;
}

int GpuReduction_call(const GpuReduction *cgr, GpuArray *d0, GpuArray *d1, const GpuArray *s0,
                      unsigned reduxLen, const int *reduxList, int flags) {
  (void)flags;
  GpuReduction *gr = const_cast<GpuReduction *>(cgr);
  if (gr == nullptr || s0 == nullptr) return GA_INVALID_ERROR;
  if (gr->nsrc() != 1 || !gr->scalars.empty())
    return ga_err_set(gr->ctx->err, GA_INVALID_ERROR,
                      "This operator takes several arguments: use GpuReduction_call_map");
  {
    bool done = false;
    int err = pcols_call(gr, d0, s0, reduxLen, reduxList, &done);
    if (err != GA_NO_ERROR || done) return err;
    err = fold_rows(gr, d0, s0, reduxLen, reduxList, &done);
    if (err != GA_NO_ERROR || done) return err;
    err = outer_then_inner(gr, d0, s0, reduxLen, reduxList, &done);
    if (err != GA_NO_ERROR || done) return err;
  }
  const src_view src = {s0, (const int64_t *)s0->strides};
  return reduce_launch(gr, d0, d1, s0->nd, s0->dimensions, &src, nullptr, 0, reduxLen, reduxList);
}

int GpuReduction_call_noalloc(const GpuReduction *cgr, GpuArray *d0, GpuArray *d1,
                              const GpuArray *s0, unsigned reduxLen, const int *reduxList,
                              int flags) {
  (void)flags;
  GpuReduction *gr = const_cast<GpuReduction *>(cgr);
  if (gr == nullptr || s0 == nullptr) return GA_INVALID_ERROR;
  if (gr->nsrc() != 1 || !gr->scalars.empty())
    return ga_err_set(gr->ctx->err, GA_INVALID_ERROR,
                      "GpuReduction_call_noalloc takes operators made by GpuReduction_new");
  {
    // the same route as GpuReduction_call, so that the kernels its warm-up
    // call built are the ones asked for here
    bool done = false;
    int err = pcols_call(gr, d0, s0, reduxLen, reduxList, &done, true);
    if (err != GA_NO_ERROR || done) return err;
    err = fold_rows(gr, d0, s0, reduxLen, reduxList, &done, true);
    if (err != GA_NO_ERROR || done) return err;
    err = outer_then_inner(gr, d0, s0, reduxLen, reduxList, &done, true);
    if (err != GA_NO_ERROR || done) return err;
  }
  const src_view src = {s0, (const int64_t *)s0->strides};
  return reduce_launch(gr, d0, d1, s0->nd, s0->dimensions, &src, nullptr, 0, reduxLen, reduxList, true);
}

int GpuReduction_call_map(const GpuReduction *cgr, GpuArray *d0, GpuArray *d1, void **args,
                          unsigned reduxLen, const int *reduxList, int flags) {
  GpuReduction *gr = const_cast<GpuReduction *>(cgr);
  if (gr == nullptr || args == nullptr) return GA_INVALID_ERROR;
  gpucontext *ctx = gr->ctx;
  const unsigned K = gr->nsrc();
  std::vector<src_view> srcs(K);
  std::vector<void *> scalars;
  for (unsigned i : gr->scalars) {
    if (args[i] == nullptr) return ga_err_fmt(ctx->err, GA_INVALID_ERROR, "Argument %u is NULL", i);
    scalars.push_back(args[i]);
  }
  unsigned nd = 0;
  for (unsigned q = 0; q < K; q++) {
    const GpuArray *a = (const GpuArray *)args[gr->arrays[q]];
    if (a == nullptr) return ga_err_fmt(ctx->err, GA_INVALID_ERROR, "Argument %u is NULL", gr->arrays[q]);
    if (q == 0) nd = a->nd;
    else if (a->nd != nd)
      return ga_err_fmt(ctx->err, GA_VALUE_ERROR, "Argument %u has nd = %u, the first array %u",
                        gr->arrays[q], a->nd, nd);
    srcs[q].a = a;
  }
  // common extents; an extent of 1 stretches when broadcasting is allowed
  // (the rule of GpuElemwise_call, reference src/gpuarray_elemwise.c:272-383)
  std::vector<size_t> dims(nd ? nd : 1, 1);
  for (unsigned ax = 0; ax < nd; ax++) {
    size_t d = srcs[0].a->dimensions[ax];
    for (unsigned q = 1; q < K; q++) {
      const size_t dq = srcs[q].a->dimensions[ax];
      if (dq == d) continue;
      if ((flags & GE_BROADCAST) && d == 1) d = dq;
      else if (!((flags & GE_BROADCAST) && dq == 1))
        return ga_err_fmt(ctx->err, GA_VALUE_ERROR,
                          "Mismatched dimension %u: argument %u has %zu, expected %zu", ax,
                          gr->arrays[q], dq, d);
    }
    dims[ax] = d;
  }
  std::vector<int64_t> strides((size_t)K * (nd ? nd : 1));
  for (unsigned q = 0; q < K; q++) {
    const GpuArray *a = srcs[q].a;
    int64_t *st = strides.data() + (size_t)q * nd;
    for (unsigned ax = 0; ax < nd; ax++)
      st[ax] = a->dimensions[ax] == dims[ax] ? (int64_t)a->strides[ax] : 0;
    srcs[q].strides = st;
  }
  return reduce_launch(gr, d0, d1, nd, dims.data(), srcs.data(), scalars.data(), (unsigned)scalars.size(),
                       reduxLen, reduxList);
}

// Reference entry point (src/gpuarray_reduction.c:100-124).  The operator is
// cached per context and source type, so repeated calls compile nothing.
int GpuArray_maxandargmax(GpuArray *dstMax, GpuArray *dstArgmax, const GpuArray *src,
                          unsigned reduxLen, const unsigned *reduxList) {
  if (dstMax == nullptr || dstArgmax == nullptr || src == nullptr || src->nd == 0 ||
      reduxLen == 0 || reduxLen > src->nd || reduxList == nullptr)
    return GA_INVALID_ERROR;
  if (src->data == nullptr || dstMax->data == nullptr || dstArgmax->data == nullptr)
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
