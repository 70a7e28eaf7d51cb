// GpuElemwise: argument checking, iteration-space planning and kernel
// generation for one C-like expression over broadcastable strided arrays.
//
// The contract is the reference's (src/gpuarray_elemwise.c):
//   - GpuElemwise_new copies the descriptors and compiles the flat kernel at
//     once, so a bad expression fails here (:604-737);
//   - GpuElemwise_call first tries the flat path: every array has the first
//     array's exact shape and all are C- or all F-contiguous (:547-602);
//   - otherwise shapes are left-padded (GE_PADSHAPE), size-1 input dims are
//     stretched (GE_BROADCAST), outputs never stretch, the first GE_WRITE
//     array fixes the iteration space, and every mismatch is GA_VALUE_ERROR
//     (:272-383);
//   - n == 0 succeeds without a launch (:778,783).
//
// What is different is everything after the checks.  The reference unravels
// the flat index with one `%` and one `/` per dimension per ELEMENT
// (:198-209) and moves 4 bytes per lane.  Here:
//   - the order of an elementwise iteration space is free, so dims are sorted
//     by the output's stride before collapsing: an all-Fortran call, or a
//     transposed output, becomes a plain run;
//   - flat kernel: 256-lane groups, 16-byte loads and stores per lane, four
//     independent tiles of loads in flight before the first use;
//   - strided kernel: group index -> (row block, column block) with one
//     division per GROUP; a lane owns one row and walks the inner dim, so the
//     row is unravelled once per lane, never per element;
//   - an operand whose unit stride lies on another dim than the output's
//     (a transposed view) is staged through a padded 64x65 LDS tile so that
//     both its global access and the output's are coalesced.
#include "private.hpp"

#include <algorithm>
#include <array>
#include <map>
#include <string>
#include <vector>

namespace {

struct ge_arg {
  std::string name;
  int typecode;
  int flags;
  bool is_array() const { return !(flags & GE_SCALAR); }
  bool reads() const { return flags & GE_READ; }
  bool writes() const { return flags & GE_WRITE; }
};

// Flat kernel geometry: 256 lanes, each moving GE_U chunks of up to 16 bytes
// per array and tile.
constexpr unsigned GE_LANES = 256;

void appendf(std::string &s, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
void appendf(std::string &s, const char *fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  int n = vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  if (n < 0) return;
  if ((size_t)n < sizeof(buf)) {
    s.append(buf, (size_t)n);
    return;
  }
  std::vector<char> big((size_t)n + 1);
  va_start(ap, fmt);
  vsnprintf(big.data(), big.size(), fmt, ap);
  va_end(ap);
  s.append(big.data(), (size_t)n);
}

const char *ctype(int typecode) { return gpuarray_get_type(typecode)->cluda_name; }

const char *chunk_type(size_t bytes) {
  switch (bytes) {
  case 1: return "ga_ubyte";
  case 2: return "ga_ushort";
  case 4: return "ga_uint";
  case 8: return "ga_chunk8";
  case 32: return "ga_chunk32";
  default: return "ga_chunk16";
  }
}

}  // namespace

// One planned launch: the kernel, its geometry and where each of its
// arguments comes from - a value fixed by the plan, the buffer of an array
// argument of the call, or a scalar argument of the call.
struct ew_slot {
  enum : unsigned char { VALUE, ARRAY, SCALAR } kind;
  unsigned char arg;   // ARRAY / SCALAR: position among the call's arguments
  int64_t value;       // VALUE: the bytes of a 4- or 8-byte kernel argument
};
struct ew_launch {
  GpuKernel *k = nullptr;
  size_t gs = 0, ls = 0;
  std::vector<ew_slot> slots;
  bool valid = false;
  void value(const void *p, size_t bytes) {
    ew_slot s = {ew_slot::VALUE, 0, 0};
    memcpy(&s.value, p, bytes);
    slots.push_back(s);
  }
  template <class T> void value(const T &v) { static_assert(sizeof(T) <= 8, ""); value(&v, sizeof(T)); }
  void array(size_t arg) { slots.push_back(ew_slot{ew_slot::ARRAY, (unsigned char)arg, 0}); }
  void scalar(size_t arg) { slots.push_back(ew_slot{ew_slot::SCALAR, (unsigned char)arg, 0}); }
};
// A planned call kept with its operator.  The key lists every input of the
// planners: the call's flags, the tuning table's generation and, per array,
// rank, extents, strides, offset, flags and the alignment of the buffer's base.
constexpr unsigned EW_KEYMAX = 176, EW_ENTRIES = 4;
struct ew_memo {
  unsigned nkey = 0;
  int64_t key[EW_KEYMAX];
  ew_launch launch;
};

struct _GpuElemwise {
  gpucontext *ctx = nullptr;
  std::string expr, preamble;
  std::vector<ge_arg> args;
  unsigned int narray = 0;
  int flags = 0;
  int kflags = 0;           // GA_USE_* for the compiler
  unsigned int vec = 1;     // elements per chunk in the flat kernel
  unsigned int unroll = 1;  // chunks per lane and tile in the flat kernel
  bool narrow_side = false; // every input, or every output, is of narrower elements than the widest
  bool tile = false;        // a group's chunks are adjacent (tile) or a grid apart
  bool nontemporal = true;  // streaming hint on the flat kernel's loads and stores
  unsigned flat_nt_mask = ~0u;   // ... per array (bit k: array k)
  GpuKernel k_flat = {nullptr, nullptr};
  // the flat kernel with 2 or 4 adjacent chunks per lane, built on first use
  std::map<unsigned, GpuKernel> k_flat_tiled;
  // the flat kernel with some read-only operands addressed through the
  // coordinates of the flat index (broadcast operands), by (mask, dims)
  std::map<std::array<uint32_t, 4>, GpuKernel> k_flat_periodic;
  bool flat_forced = false;   // the environment fixed the flat kernel's shape
  // strided kernels by variant key: "<nd>:<idx64>:<transposed mask>"
  std::map<std::string, GpuKernel> k_strided;
  // planning scratch
  std::vector<size_t> dims;
  std::vector<std::vector<ssize_t>> strs;
  std::vector<ssize_t *> strp;
  ew_launch pending;             // what the planners leave for GpuElemwise_call to launch
  std::vector<ew_memo> memo;     // planned calls
  unsigned memo_next = 0;        // the entry the next new plan replaces once all are taken
};

namespace {

bool local_is_float(const GpuElemwise *ge, const ge_arg &a) {
  return (ge->flags & GE_CONVERT_F16) && a.typecode == GA_HALF;
}

// "T name;" plus the load, given an lvalue expression for the element.
void emit_load(const GpuElemwise *ge, std::string &s, const ge_arg &a, const std::string &src) {
  const bool cvt = local_is_float(ge, a);
  appendf(s, "%s %s;", cvt ? "ga_float" : ctype(a.typecode), a.name.c_str());
  if (a.reads()) {
    if (cvt) appendf(s, " %s = ga_half2float(%s);", a.name.c_str(), src.c_str());
    else appendf(s, " %s = %s;", a.name.c_str(), src.c_str());
  }
  s += "\n";
}

void emit_store(const GpuElemwise *ge, std::string &s, const ge_arg &a, const std::string &dst) {
  if (!a.writes()) return;
  if (local_is_float(ge, a)) appendf(s, "%s = ga_float2half(%s);\n", dst.c_str(), a.name.c_str());
  else appendf(s, "%s = %s;\n", dst.c_str(), a.name.c_str());
}

void emit_header(const GpuElemwise *ge, std::string &s) {
  s += "#include \"cluda.h\"\n";
  s += "typedef ga_uint __attribute__((ext_vector_type(2))) ga_chunk8;\n"
       "typedef ga_uint __attribute__((ext_vector_type(4))) ga_chunk16;\n"
       "typedef ga_uint __attribute__((ext_vector_type(8))) ga_chunk32;\n";
  s += ge->preamble;
  s += "\n";
}

// ---- flat kernel --------------------------------------------------------------
// elem(n, {data, byte offset | scalar}..., ga_vec)
//   ga_vec != 0: (ga_vec & 0xff) - 1 elements into every array a whole chunk of V
//   elements starts, except the arrays k with bit 8 + k set, which are moved
//   element by element
//   (16 bytes of the widest type).  Chunk c belongs to lane c % 256 of group
//   (c / 256) % G; a lane issues the loads of its next U chunks (G*256 chunks
//   apart, so every load instruction of a wavefront covers one contiguous
//   kilobyte) before the first use.  The elements before the first chunk and
//   after the last one, and the whole range when ga_vec == 0, run one element
//   per lane.
//
// pmask != 0 (bit k: array k): those read-only arrays are not walked as one
// dense run but addressed through the coordinates of the flat index in an
// iteration space of pnd (2 or 3) dims, (d0,) d1, d2: element i of the run is
// (c0, c1, c2) = (i / (d1 d2), i / d2 % d1, i % d2) and the operand's element
// is ps0 c0 + ps1 c1 + ps2 c2 bytes in.  That is how operands broadcast
// against dense arrays are read (a bias row, a per-row or per-channel factor)
// whatever the extents are: the dense arrays keep their 16-byte chunks.  The
// two divisions are multiplications by 2^k / d rounded up (n < 2^31), once
// per chunk; a lane steps the coordinates through its chunk's elements.
// Extra parameters, after ga_vec: d1, d2, the two multipliers and shifts,
// then ps0, ps1, ps2 per such array.  Arrays also in pvmask have unit stride
// along the inner dim and everything aligned to the chunk, and the caller
// passes no head: a chunk's elements are then one chunk of the operand too,
// fetched with one load.  Arrays in pumask (four-byte elements, four to a
// chunk, not in pvmask) fetch a chunk that lies inside one row of the inner
// dim with one load that assumes four-byte boundaries only, when their stride
// along that dim is the element's size; the chunks that straddle two rows
// stay element by element.
std::string gen_flat(const GpuElemwise *ge, std::vector<int> &ktypes, unsigned unroll = 0, int tiled = -1,
                     unsigned pmask = 0, unsigned pnd = 2, unsigned pvmask = 0, unsigned pumask = 0) {
  std::string s;
  const unsigned V = ge->vec, U = unroll ? unroll : ge->unroll;
  const bool tile = tiled < 0 ? ge->tile : tiled != 0;
  std::vector<int> aidx(ge->args.size(), -1);
  {
    int k = 0;
    for (size_t j = 0; j < ge->args.size(); j++)
      if (ge->args[j].is_array()) aidx[j] = k++;
  }
  auto is_p = [&](const ge_arg &a) {
    const size_t j = (size_t)(&a - ge->args.data());
    return aidx[j] >= 0 && ((pmask >> aidx[j]) & 1u);
  };
  auto is_pv = [&](const ge_arg &a) {
    const size_t j = (size_t)(&a - ge->args.data());
    return aidx[j] >= 0 && ((pmask & pvmask) >> aidx[j]) & 1u;
  };
  auto is_pu = [&](const ge_arg &a) {
    const size_t j = (size_t)(&a - ge->args.data());
    return aidx[j] >= 0 && ((pmask & ~pvmask & pumask) >> aidx[j]) & 1u && V == 4 &&
           gpuarray_get_elsize(a.typecode) == 4;
  };
  // lvalue of a periodic operand's element at coordinates named c0/c1/c2
  auto p_elem = [&](const ge_arg &a, const char *c0, const char *c1, const char *c2) {
    std::string e;
    appendf(e, "*(GLOBAL_MEM const %s *)((GLOBAL_MEM const char *)%s_p + (ga_ssize)%s * %s_ps0 + "
               "(ga_ssize)%s * %s_ps1 + (ga_ssize)%s * %s_ps2)",
            ctype(a.typecode), a.name.c_str(), c0, a.name.c_str(), c1, a.name.c_str(), c2, a.name.c_str());
    return e;
  };
  // coordinates of flat index `idx` into ga_p0, ga_p1, ga_p2
  auto p_coords = [&](const char *idx) {
    std::string e;
    appendf(e, "ga_uint ga_p0 = 0, ga_p1, ga_p2;\n{ const ga_uint ga_fi = (ga_uint)(%s);\n"
               "const ga_uint ga_q = (ga_uint)(((ga_ulong)ga_fi * ga_m2) >> ga_k2);\n"
               "ga_p2 = ga_fi - ga_q * ga_d2;\n", idx);
    if (pnd == 3)
      e += "ga_p0 = (ga_uint)(((ga_ulong)ga_q * ga_m1) >> ga_k1);\nga_p1 = ga_q - ga_p0 * ga_d1;\n}\n";
    else
      e += "ga_p1 = ga_q;\n}\n";
    return e;
  };
  emit_header(ge, s);
  {
    bool any_pu = false;
    for (const ge_arg &a : ge->args) any_pu = any_pu || is_pu(a);
    if (any_pu) s += "typedef ga_uint __attribute__((ext_vector_type(4), aligned(4))) ga_chunk16u;\n";
  }
  s += "KERNEL void __launch_bounds__(256) elem(const ga_size n";
  ktypes.push_back(GA_SIZE);
  for (const ge_arg &a : ge->args) {
    if (a.is_array()) {
      appendf(s, ", GLOBAL_MEM %s *%s_p, const ga_size %s_offset", ctype(a.typecode),
              a.name.c_str(), a.name.c_str());
      ktypes.push_back(GA_BUFFER);
      ktypes.push_back(GA_SIZE);
    } else {
      appendf(s, ", %s %s", ctype(a.typecode), a.name.c_str());
      ktypes.push_back(a.typecode);
    }
  }
  s += ", const ga_uint ga_vec";
  ktypes.push_back(GA_UINT);
  if (pmask) {
    s += ", const ga_uint ga_d1, const ga_uint ga_d2, const ga_ulong ga_m1, const ga_uint ga_k1, "
         "const ga_ulong ga_m2, const ga_uint ga_k2";
    for (int t : {GA_UINT, GA_UINT, GA_ULONG, GA_UINT, GA_ULONG, GA_UINT}) ktypes.push_back(t);
    for (const ge_arg &a : ge->args)
      if (is_p(a)) {
        appendf(s, ", const ga_ssize %s_ps0, const ga_ssize %s_ps1, const ga_ssize %s_ps2",
                a.name.c_str(), a.name.c_str(), a.name.c_str());
        for (int q = 0; q < 3; q++) ktypes.push_back(GA_SSIZE);
      }
  }
  s += ") {\n";
  if (pmask) s += "(void)ga_d1; (void)ga_m1; (void)ga_k1;\n";
  for (const ge_arg &a : ge->args)
    if (a.is_array())
      appendf(s, "%s_p = (GLOBAL_MEM %s *)((GLOBAL_MEM char *)%s_p + %s_offset);\n",
              a.name.c_str(), ctype(a.typecode), a.name.c_str(), a.name.c_str());
  s += "const ga_size ga_gtid = (ga_size)GID_0 * LDIM_0 + LID_0;\n"
       "const ga_size ga_nthr = (ga_size)GDIM_0 * LDIM_0;\n"
       "ga_size ga_done = 0; (void)ga_done;\n";
  if (V > 1 || U > 1) {
    // ga_vec - 1 leading elements come before the first whole chunk of every array
    // and bit 8 + k says that array k does not: it is then moved element by element
    s += "if (ga_vec) {\nconst ga_size ga_head = (ga_vec & 0xffu) - 1u;\nconst ga_uint ga_mis = ga_vec >> 8;\n";
    for (const ge_arg &a : ge->args)
      if (a.is_array() && !is_p(a)) appendf(s, "%s_p += ga_head;\n", a.name.c_str());
    appendf(s, "const ga_size ga_nchunks = (n - ga_head) / %uu;\n", V);
    if (tile) {
      appendf(s, "const ga_size ga_ustep = 256;\n"
                 "for (ga_size ga_c0 = (ga_size)GID_0 * %uu + LID_0; ga_c0 - LID_0 < ga_nchunks; "
                 "ga_c0 += (ga_size)GDIM_0 * %uu) {\n", 256 * U, 256 * U);
    } else {
      s += "const ga_size ga_ustep = ga_nthr;\n";
      appendf(s, "for (ga_size ga_c0 = ga_gtid; ga_c0 < ga_nchunks; ga_c0 += ga_nthr * %uu) {\n", U);
    }
    for (const ge_arg &a : ge->args) {
      if (!a.is_array()) continue;
      size_t cb = gpuarray_get_elsize(a.typecode) * V;
      appendf(s, "union { %s c; %s e[%u];%s } %s_u[%u];\n", chunk_type(cb), ctype(a.typecode), V,
              is_pu(a) ? " ga_chunk16u w;" : "", a.name.c_str(), U);
    }
    appendf(s, "#pragma unroll\nfor (int ga_u = 0; ga_u < %u; ga_u++) {\n", U);
    s += "const ga_size ga_c = ga_c0 + (ga_size)ga_u * ga_ustep;\nif (ga_c < ga_nchunks) {\n";
    if (pmask) {
      // the coordinates of the chunk's first element, then stepped through the chunk
      char idx[64];
      snprintf(idx, sizeof(idx), "ga_head + ga_c * %uu", V);
      s += "{\n" + p_coords(idx);
      for (const ge_arg &a : ge->args)
        if (is_pv(a)) {
          const size_t cb = gpuarray_get_elsize(a.typecode) * V;
          appendf(s, "%s_u[ga_u].c = *(GLOBAL_MEM const %s *)((GLOBAL_MEM const char *)%s_p + (ga_ssize)ga_p0 * %s_ps0 + "
                     "(ga_ssize)ga_p1 * %s_ps1 + (ga_ssize)ga_p2 * %s_ps2);\n",
                  a.name.c_str(), chunk_type(cb), a.name.c_str(), a.name.c_str(), a.name.c_str(), a.name.c_str());
        }
      for (const ge_arg &a : ge->args)
        if (is_pu(a))
          appendf(s, "const bool %s_w = %s_ps2 == 4 && ga_p2 + %uu <= ga_d2;\n"
                     "if (%s_w) %s_u[ga_u].w = *(GLOBAL_MEM const ga_chunk16u *)((GLOBAL_MEM const char *)%s_p + "
                     "(ga_ssize)ga_p0 * %s_ps0 + (ga_ssize)ga_p1 * %s_ps1 + (ga_ssize)ga_p2 * 4);\n",
                  a.name.c_str(), a.name.c_str(), V, a.name.c_str(), a.name.c_str(), a.name.c_str(),
                  a.name.c_str(), a.name.c_str());
      appendf(s, "#pragma unroll\nfor (int ga_v = 0; ga_v < %u; ga_v++) {\n", V);
      for (const ge_arg &a : ge->args)
        if (is_p(a) && !is_pv(a)) {
          if (is_pu(a)) appendf(s, "if (!%s_w) ", a.name.c_str());
          appendf(s, "%s_u[ga_u].e[ga_v] = %s;\n", a.name.c_str(), p_elem(a, "ga_p0", "ga_p1", "ga_p2").c_str());
        }
      s += "if (++ga_p2 == ga_d2) { ga_p2 = 0; ";
      s += pnd == 3 ? "if (++ga_p1 == ga_d1) { ga_p1 = 0; ga_p0++; } }\n" : "ga_p1++; }\n";
      s += "}\n}\n";
    }
    unsigned ak = 0;
    for (const ge_arg &a : ge->args) {
      if (!a.is_array()) continue;
      const unsigned bit = ak++;
      if (!a.reads() || is_p(a)) continue;
      size_t cb = gpuarray_get_elsize(a.typecode) * V;
      appendf(s, "if (ga_mis & %uu) {\n#pragma unroll\nfor (int ga_v = 0; ga_v < %u; ga_v++) "
                 "%s_u[ga_u].e[ga_v] = %s_p[ga_c * %uu + ga_v];\n} else {\n",
              1u << bit, V, a.name.c_str(), a.name.c_str(), V);
      if (ge->nontemporal && ((ge->flat_nt_mask >> bit) & 1u))
        appendf(s, "%s_u[ga_u].c = __builtin_nontemporal_load((const %s *)%s_p + ga_c);\n",
                a.name.c_str(), chunk_type(cb), a.name.c_str());
      else
        appendf(s, "%s_u[ga_u].c = ((const %s *)%s_p)[ga_c];\n", a.name.c_str(), chunk_type(cb),
                a.name.c_str());
      s += "}\n";
    }
    s += "}\n}\n";
    appendf(s, "#pragma unroll\nfor (int ga_u = 0; ga_u < %u; ga_u++) {\n", U);
    s += "const ga_size ga_c = ga_c0 + (ga_size)ga_u * ga_ustep;\nif (ga_c < ga_nchunks) {\n";
    appendf(s, "#pragma unroll\nfor (int ga_v = 0; ga_v < %u; ga_v++) {\n", V);
    appendf(s, "const ga_size i = ga_head + ga_c * %uu + ga_v; (void)i;\n{\n", V);
    for (const ge_arg &a : ge->args)
      if (a.is_array()) emit_load(ge, s, a, a.name + "_u[ga_u].e[ga_v]");
    s += ge->expr;
    s += ";\n";
    for (const ge_arg &a : ge->args)
      if (a.is_array()) emit_store(ge, s, a, a.name + "_u[ga_u].e[ga_v]");
    s += "}\n}\n";
    ak = 0;
    for (const ge_arg &a : ge->args) {
      if (!a.is_array()) continue;
      const unsigned bit = ak++;
      if (!a.writes()) continue;
      size_t cb = gpuarray_get_elsize(a.typecode) * V;
      appendf(s, "if (ga_mis & %uu) {\n#pragma unroll\nfor (int ga_v = 0; ga_v < %u; ga_v++) "
                 "%s_p[ga_c * %uu + ga_v] = %s_u[ga_u].e[ga_v];\n} else {\n",
              1u << bit, V, a.name.c_str(), V, a.name.c_str());
      if (ge->nontemporal && ((ge->flat_nt_mask >> bit) & 1u))
        appendf(s, "__builtin_nontemporal_store(%s_u[ga_u].c, (%s *)%s_p + ga_c);\n",
                a.name.c_str(), chunk_type(cb), a.name.c_str());
      else
        appendf(s, "((%s *)%s_p)[ga_c] = %s_u[ga_u].c;\n", chunk_type(cb), a.name.c_str(),
                a.name.c_str());
      s += "}\n";
    }
    s += "}\n}\n";
    s += "}\n";
    for (const ge_arg &a : ge->args)
      if (a.is_array() && !is_p(a)) appendf(s, "%s_p -= ga_head;\n", a.name.c_str());
    appendf(s, "ga_done = ga_nchunks * %uu;\n", V);
    // the elements before the first chunk and after the last one
    s += "const ga_size ga_rest = n - ga_done;\nfor (ga_size ga_t = ga_gtid; ga_t < ga_rest; ga_t += ga_nthr) {\n"
         "const ga_size i = ga_t < ga_head ? ga_t : ga_t + ga_done;\n";
    if (pmask) s += p_coords("i");
    for (const ge_arg &a : ge->args)
      if (a.is_array()) emit_load(ge, s, a, is_p(a) ? p_elem(a, "ga_p0", "ga_p1", "ga_p2") : a.name + "_p[i]");
    s += ge->expr;
    s += ";\n";
    for (const ge_arg &a : ge->args)
      if (a.is_array()) emit_store(ge, s, a, a.name + "_p[i]");
    s += "}\nreturn;\n}\n";
  }
  s += "for (ga_size i = ga_gtid; i < n; i += ga_nthr) {\n";
  if (pmask) s += p_coords("i");
  for (const ge_arg &a : ge->args)
    if (a.is_array()) emit_load(ge, s, a, is_p(a) ? p_elem(a, "ga_p0", "ga_p1", "ga_p2") : a.name + "_p[i]");
  s += ge->expr;
  s += ";\n";
  for (const ge_arg &a : ge->args)
    if (a.is_array()) emit_store(ge, s, a, a.name + "_p[i]");
  s += "}\n}\n";
  return s;
}

// ---- narrow planes in registers -------------------------------------------------
// Same parameters as the strided kernel with two or three dims (with three, the
// first counts planes, ga_gx groups each).  One of the last two dims is
// short (S, extent F <= 16, fixed in the text), the other long (L).  The
// arrays have elements of 1, 2, 4 or 8 bytes; es is the smallest size among
// them and E = 16 / es the elements of a chunk of that type (the text below
// says four).  A lane owns E adjacent positions along L and all F along S, a
// group 256 E positions along L; of an array of wider elements a lane's E
// positions of a row are several chunks, one after the other.
//  * The arrays in bmask have the short dim innermost: a lane's 4 F elements,
//    and a group's 4096 F, lie one after the other in memory (stride of S one
//    element, of L F elements: an (N, F) array taken as its transpose), on a
//    16-byte boundary.  Those also in smask pass through the LDS: the group
//    moves its piece of the array in 16-byte chunks, consecutive lanes on
//    consecutive chunks, and a lane exchanges its own F chunks with the LDS
//    (slots swizzled when F is a power of two: a lane's chunks are then a
//    multiple of 8 slots from its neighbours').  The others are fetched or
//    stored as the lane's own F chunks.
//  * The arrays in cmask run along L with unit stride and move as one 16-byte
//    chunk per position of S, side by side with the neighbouring lanes'; those
//    also in umask through accesses that assume four-byte boundaries only (the
//    element's own with two-byte elements).
//  * Operands constant along L (zmask): one element per position of S, once.
//  * Every other array one element at a time.
// The last lane of a row takes what exists of its positions one by one.
std::string gen_narrow_block(const GpuElemwise *ge, bool idx64, unsigned F, unsigned sd, unsigned bmask,
                             unsigned cmask, unsigned ntmask, std::vector<int> &ktypes, unsigned umask = 0,
                             unsigned smask = 0, unsigned nd = 2, unsigned es = 4, unsigned zmask = 0) {
  std::string s;
  const unsigned E = 16 / es;   // positions of a lane: the elements of a chunk of the smallest type (es bytes)
  // chunks that a lane's E positions of one row take in an array, and elements of a chunk of it
  auto cpr = [&](const ge_arg &a) { return (unsigned)(E * gpuarray_get_elsize(a.typecode) / 16); };
  auto epc = [&](const ge_arg &a) { return (unsigned)(16 / gpuarray_get_elsize(a.typecode)); };
  const char *I = idx64 ? "ga_ssize" : "ga_int";
  const char *N = idx64 ? "ga_size" : "ga_uint";
  const unsigned ld = sd == nd - 1 ? nd - 2 : nd - 1;
  emit_header(ge, s);
  if (umask)
    s += "typedef ga_uint __attribute__((ext_vector_type(4), aligned(4))) ga_chunk16u;\n"
         "typedef ga_uint __attribute__((ext_vector_type(4), aligned(2))) ga_chunk16u2;\n"
         "typedef ga_uint __attribute__((ext_vector_type(4), aligned(1))) ga_chunk16u1;\n";
  auto loose_type = [&](const ge_arg &a) {
    const size_t z = gpuarray_get_elsize(a.typecode);
    return z >= 4 ? "ga_chunk16u" : z == 2 ? "ga_chunk16u2" : "ga_chunk16u1";
  };
  if (smask) s += "#define GA_SLOTX(q) ((q) ^ (((q) >> 3) & 7u))\n#define GA_SLOTP(q) (q)\n";
  // (slots swizzled where a lane's chunks of the array are a power of two)
  auto slot = [&](const ge_arg &a) { const unsigned m = F * cpr(a); return (m & (m - 1)) == 0 ? "GA_SLOTX" : "GA_SLOTP"; };
  s += "KERNEL void __launch_bounds__(256) elem(const ga_size dim0";
  ktypes.push_back(GA_SIZE);
  for (unsigned d = 1; d < nd; d++) {
    appendf(s, ", const ga_size dim%u", d);
    ktypes.push_back(GA_SIZE);
  }
  std::vector<int> aidx(ge->args.size(), -1);
  {
    int k = 0;
    for (size_t j = 0; j < ge->args.size(); j++)
      if (ge->args[j].is_array()) aidx[j] = k++;
  }
  auto in = [&](unsigned mask, size_t j) { return aidx[j] >= 0 && ((mask >> aidx[j]) & 1u); };
  for (const ge_arg &a : ge->args) {
    if (a.is_array()) {
      appendf(s, ", GLOBAL_MEM %s *%s_data, const ga_size %s_offset", ctype(a.typecode), a.name.c_str(), a.name.c_str());
      ktypes.push_back(GA_BUFFER);
      ktypes.push_back(GA_SIZE);
      for (unsigned d = 0; d < nd; d++) {
        appendf(s, ", const ga_ssize %s_str_%u", a.name.c_str(), d);
        ktypes.push_back(GA_SSIZE);
      }
    } else {
      appendf(s, ", %s %s", ctype(a.typecode), a.name.c_str());
      ktypes.push_back(a.typecode);
    }
  }
  s += ", const ga_uint ga_gx, const ga_uint ga_ltx) {\n(void)ga_gx; (void)ga_ltx; (void)dim0; (void)dim1;\n";
  ktypes.push_back(GA_UINT);
  ktypes.push_back(GA_UINT);
  // three dims: planes one after the other, ga_gx groups each
  if (nd == 3) s += "const ga_uint ga_o = GID_0 / ga_gx;\nconst ga_uint ga_pc = GID_0 - ga_o * ga_gx;\n";
  else s += "const ga_uint ga_pc = GID_0;\n";
  for (size_t j = 0; j < ge->args.size(); j++) {
    const ge_arg &a = ge->args[j];
    if (!a.is_array()) continue;
    appendf(s, "GLOBAL_MEM char *%s_b = (GLOBAL_MEM char *)%s_data + %s_offset;\n", a.name.c_str(), a.name.c_str(),
            a.name.c_str());
    if (nd == 3) appendf(s, "%s_b += (%s)ga_o * (%s)%s_str_0;\n", a.name.c_str(), I, I, a.name.c_str());
    if (in(smask, j)) appendf(s, "LOCAL_MEM ga_chunk16 %s_s[%u];\n", a.name.c_str(), 256 * F * cpr(a));
  }
  appendf(s, "const %s ga_l0 = (%s)ga_pc * %uu;\n", N, N, 256 * E);
  appendf(s, "const %s ga_l4 = ga_l0 + LID_0 * %uu;\n", N, E);
  if (!smask) appendf(s, "if (ga_l4 >= (%s)dim%u) return;\n", N, ld);
  appendf(s, "const bool ga_full = ga_l4 + %uu < (%s)dim%u;\n", E - 1, N, ld);
  // the four-byte words of a staged array that the group's piece holds
  if (smask)
    appendf(s, "const ga_uint ga_cnt = (ga_uint)((%s)dim%u - ga_l0 < %uu ? (%s)dim%u - ga_l0 : %uu) * %uu;\n", N, ld, 256 * E,
            N, ld, 256 * E, F);
  // registers of the block arrays (element e * F + y: position e along L, y along S)
  // and of the chunked ones (element e of chunk y)
  for (size_t j = 0; j < ge->args.size(); j++) {
    const ge_arg &a = ge->args[j];
    if (in(bmask, j))
      appendf(s, "union { ga_chunk16 c[%u]; %s e[%u]; } %s_r;\n", F * cpr(a), ctype(a.typecode), E * F, a.name.c_str());
    else if (in(cmask, j))
      appendf(s, "union { ga_chunk16 c[%u]; %s e[%u]; } %s_r[%u];\n", cpr(a), ctype(a.typecode), E, a.name.c_str(), F);
  }
  auto elem_at = [&](const ge_arg &a, const std::string &y, const std::string &l) {
    std::string e;
    appendf(e, "*(GLOBAL_MEM %s *)(%s_b + ((%s)(%s) * (%s)%s_str_%u + (%s)(%s) * (%s)%s_str_%u))", ctype(a.typecode),
            a.name.c_str(), I, y.c_str(), I, a.name.c_str(), sd, I, l.c_str(), I, a.name.c_str(), ld);
    return e;
  };
  // byte address of the group's piece of a staged array, plus an expression in bytes
  auto piece_at = [&](const ge_arg &a, const char *cast, const std::string &bytes) {
    std::string e;
    appendf(e, "(GLOBAL_MEM %s *)(%s_b + (%s)ga_l0 * (%s)%s_str_%u + (%s))", cast, a.name.c_str(), I, I,
            a.name.c_str(), ld, bytes.c_str());
    return e;
  };
  // loads
  bool staged_in = false, staged_inout = false;
  for (size_t j = 0; j < ge->args.size(); j++) {
    const ge_arg &a = ge->args[j];
    if (!a.is_array() || !a.reads()) continue;
    const bool nt = (ntmask >> aidx[j]) & 1u;
    if (in(smask, j)) {
      staged_in = true;
      if (a.writes()) staged_inout = true;
      char eb[64];
      snprintf(eb, sizeof(eb), "(ga_q * %uu + ga_e) * %uu", epc(a), 16 / epc(a));
      for (unsigned h = 0; h < F * cpr(a); h++) {
        appendf(s, "{ const ga_uint ga_q = %uu + LID_0;\n", h * 256);
        const std::string ptr = piece_at(a, "const ga_chunk16", "ga_q * 16u");
        appendf(s, "if (ga_q * %uu + %uu < ga_cnt) %s_s[%s(ga_q)] = %s(%s);\n", epc(a), epc(a) - 1, a.name.c_str(), slot(a),
                nt ? "__builtin_nontemporal_load" : "*", ptr.c_str());
        appendf(s, "else for (ga_uint ga_e = 0; ga_e < %uu; ga_e++) if (ga_q * %uu + ga_e < ga_cnt) "
                   "((%s *)%s_s)[%s(ga_q) * %uu + ga_e] = *(%s);\n",
                epc(a), epc(a), ctype(a.typecode), a.name.c_str(), slot(a), epc(a), piece_at(a, ctype(a.typecode), eb).c_str());
        s += "}\n";
      }
    } else if (in(bmask, j)) {
      s += "if (ga_full) {\n";
      for (unsigned h = 0; h < F * cpr(a); h++) {
        std::string ptr;
        appendf(ptr, "(GLOBAL_MEM const ga_chunk16 *)(%s_b + (%s)ga_l4 * (%s)%s_str_%u) + %u", a.name.c_str(), I, I,
                a.name.c_str(), ld, h);
        appendf(s, "%s_r.c[%u] = %s(%s);\n", a.name.c_str(), h, nt ? "__builtin_nontemporal_load" : "*", ptr.c_str());
      }
      s += "} else {\n";
      for (unsigned e = 0; e < E; e++)
        for (unsigned y = 0; y < F; y++) {
          char l[32], yy[16];
          snprintf(l, sizeof(l), "ga_l4 + %uu", e);
          snprintf(yy, sizeof(yy), "%uu", y);
          appendf(s, "if (ga_l4 + %uu < (%s)dim%u) %s_r.e[%u] = %s;\n", e, N, ld, a.name.c_str(), e * F + y,
                  elem_at(a, yy, l).c_str());
        }
      s += "}\n";
    } else if (in(cmask, j)) {
      const char *ct = in(umask, j) ? loose_type(a) : "ga_chunk16";
      for (unsigned y = 0; y < F; y++) {
        char yy[16];
        snprintf(yy, sizeof(yy), "%uu", y);
        std::string ptr;
        appendf(ptr, "(GLOBAL_MEM const %s *)&%s", ct, elem_at(a, yy, "ga_l4").c_str());
        s += "if (ga_full) {";
        for (unsigned c = 0; c < cpr(a); c++)
          appendf(s, " %s_r[%u].c[%u] = %s((%s) + %u);", a.name.c_str(), y, c, nt ? "__builtin_nontemporal_load" : "*",
                  ptr.c_str(), c);
        s += " } else {\n";
        for (unsigned e = 0; e < E; e++) {
          char l[32];
          snprintf(l, sizeof(l), "ga_l4 + %uu", e);
          appendf(s, "if (ga_l4 + %uu < (%s)dim%u) %s_r[%u].e[%u] = %s;\n", e, N, ld, a.name.c_str(), y, e,
                  elem_at(a, yy, l).c_str());
        }
        s += "}\n";
      }
    }
  }
  if (staged_in) {
    s += "local_barrier();\n";
    for (size_t j = 0; j < ge->args.size(); j++) {
      const ge_arg &a = ge->args[j];
      if (!a.is_array() || !a.reads() || !in(smask, j)) continue;
      for (unsigned h = 0; h < F * cpr(a); h++)
        appendf(s, "%s_r.c[%u] = %s_s[%s(LID_0 * %uu + %uu)];\n", a.name.c_str(), h, a.name.c_str(), slot(a), F * cpr(a), h);
    }
  }
  // operands constant along L (in zmask, read only): one element per position of S, fetched once
  for (size_t j = 0; j < ge->args.size(); j++) {
    const ge_arg &a = ge->args[j];
    if (!in(zmask, j)) continue;
    appendf(s, "%s %s_z[%u];\n", ctype(a.typecode), a.name.c_str(), F);
    for (unsigned y = 0; y < F; y++) {
      char yy[16];
      snprintf(yy, sizeof(yy), "%uu", y);
      appendf(s, "%s_z[%u] = %s;\n", a.name.c_str(), y, elem_at(a, yy, "0u").c_str());
    }
  }
  // the expression, position by position
  for (unsigned y = 0; y < F; y++)
    for (unsigned e = 0; e < E; e++) {
      char l[32], yy[16];
      snprintf(l, sizeof(l), "ga_l4 + %uu", e);
      snprintf(yy, sizeof(yy), "%uu", y);
      appendf(s, "if (ga_l4 + %uu < (%s)dim%u) {\n", e, N, ld);
      for (size_t j = 0; j < ge->args.size(); j++) {
        const ge_arg &a = ge->args[j];
        if (!a.is_array()) continue;
        std::string src;
        if (in(bmask, j)) appendf(src, "%s_r.e[%u]", a.name.c_str(), e * F + y);
        else if (in(cmask, j)) appendf(src, "%s_r[%u].e[%u]", a.name.c_str(), y, e);
        else if (in(zmask, j)) appendf(src, "%s_z[%u]", a.name.c_str(), y);
        else src = elem_at(a, yy, l);
        emit_load(ge, s, a, src);
      }
      s += ge->expr;
      s += ";\n";
      for (size_t j = 0; j < ge->args.size(); j++) {
        const ge_arg &a = ge->args[j];
        if (!a.is_array() || !a.writes()) continue;
        std::string dst;
        if (in(bmask, j)) appendf(dst, "%s_r.e[%u]", a.name.c_str(), e * F + y);
        else if (in(cmask, j)) appendf(dst, "%s_r[%u].e[%u]", a.name.c_str(), y, e);
        else dst = elem_at(a, yy, l);
        emit_store(ge, s, a, dst);
      }
      s += "}\n";
    }
  // stores of the results kept in registers
  if (staged_inout) s += "local_barrier();\n";   // every lane has taken its chunks before the slots are written again
  bool staged_out = false;
  for (size_t j = 0; j < ge->args.size(); j++) {
    const ge_arg &a = ge->args[j];
    if (!a.is_array() || !a.writes() || !in(smask, j)) continue;
    staged_out = true;
    for (unsigned h = 0; h < F * cpr(a); h++)
      appendf(s, "%s_s[%s(LID_0 * %uu + %uu)] = %s_r.c[%u];\n", a.name.c_str(), slot(a), F * cpr(a), h, a.name.c_str(), h);
  }
  if (staged_out) s += "local_barrier();\n";
  for (size_t j = 0; j < ge->args.size(); j++) {
    const ge_arg &a = ge->args[j];
    if (!a.is_array() || !a.writes()) continue;
    const bool nt = (ntmask >> aidx[j]) & 1u;
    if (in(smask, j)) {
      char eb[64];
      snprintf(eb, sizeof(eb), "(ga_q * %uu + ga_e) * %uu", epc(a), 16 / epc(a));
      for (unsigned h = 0; h < F * cpr(a); h++) {
        appendf(s, "{ const ga_uint ga_q = %uu + LID_0;\n", h * 256);
        const std::string ptr = piece_at(a, "ga_chunk16", "ga_q * 16u");
        if (nt) appendf(s, "if (ga_q * %uu + %uu < ga_cnt) __builtin_nontemporal_store(%s_s[%s(ga_q)], %s);\n", epc(a),
                        epc(a) - 1, a.name.c_str(), slot(a), ptr.c_str());
        else appendf(s, "if (ga_q * %uu + %uu < ga_cnt) *(%s) = %s_s[%s(ga_q)];\n", epc(a), epc(a) - 1, ptr.c_str(),
                     a.name.c_str(), slot(a));
        appendf(s, "else for (ga_uint ga_e = 0; ga_e < %uu; ga_e++) if (ga_q * %uu + ga_e < ga_cnt) "
                   "*(%s) = ((%s *)%s_s)[%s(ga_q) * %uu + ga_e];\n",
                epc(a), epc(a), piece_at(a, ctype(a.typecode), eb).c_str(), ctype(a.typecode), a.name.c_str(), slot(a), epc(a));
        s += "}\n";
      }
    } else if (in(bmask, j)) {
      s += "if (ga_full) {\n";
      for (unsigned h = 0; h < F * cpr(a); h++) {
        std::string ptr;
        appendf(ptr, "(GLOBAL_MEM ga_chunk16 *)(%s_b + (%s)ga_l4 * (%s)%s_str_%u) + %u", a.name.c_str(), I, I,
                a.name.c_str(), ld, h);
        if (nt) appendf(s, "__builtin_nontemporal_store(%s_r.c[%u], %s);\n", a.name.c_str(), h, ptr.c_str());
        else appendf(s, "*(%s) = %s_r.c[%u];\n", ptr.c_str(), a.name.c_str(), h);
      }
      s += "} else {\n";
      for (unsigned e = 0; e < E; e++)
        for (unsigned y = 0; y < F; y++) {
          char l[32], yy[16];
          snprintf(l, sizeof(l), "ga_l4 + %uu", e);
          snprintf(yy, sizeof(yy), "%uu", y);
          appendf(s, "if (ga_l4 + %uu < (%s)dim%u) %s = %s_r.e[%u];\n", e, N, ld, elem_at(a, yy, l).c_str(),
                  a.name.c_str(), e * F + y);
        }
      s += "}\n";
    } else if (in(cmask, j)) {
      const char *ct = in(umask, j) ? loose_type(a) : "ga_chunk16";
      for (unsigned y = 0; y < F; y++) {
        char yy[16];
        snprintf(yy, sizeof(yy), "%uu", y);
        std::string ptr;
        appendf(ptr, "(GLOBAL_MEM %s *)&%s", ct, elem_at(a, yy, "ga_l4").c_str());
        s += "if (ga_full) {";
        for (unsigned c = 0; c < cpr(a); c++) {
          if (nt) appendf(s, " __builtin_nontemporal_store((%s)%s_r[%u].c[%u], (%s) + %u);", ct, a.name.c_str(), y, c, ptr.c_str(), c);
          else appendf(s, " *((%s) + %u) = %s_r[%u].c[%u];", ptr.c_str(), c, a.name.c_str(), y, c);
        }
        s += " } else {\n";
        for (unsigned e = 0; e < E; e++) {
          char l[32];
          snprintf(l, sizeof(l), "ga_l4 + %uu", e);
          appendf(s, "if (ga_l4 + %uu < (%s)dim%u) %s = %s_r[%u].e[%u];\n", e, N, ld, elem_at(a, yy, l).c_str(),
                  a.name.c_str(), y, e);
        }
        s += "}\n";
      }
    }
  }
  s += "}\n";
  return s;
}

// ---- narrow planes through the LDS ----------------------------------------------
// The same planes and parameters as gen_narrow_block for short extents F too
// large for a lane's registers (16 to 64).  A group owns 256 positions along L:
// the arrays in bmask (short dim innermost, the group's piece one contiguous
// run of 256 F elements on a 16-byte boundary) pass through the LDS whole, as
// consecutive 16-byte chunks on consecutive lanes; lane (lx, ly) = (LID_0 % 64,
// LID_0 / 64) then takes positions 4 lx .. 4 lx + 3 of the short dim's rows ly,
// ly + 4, ...: four words of the LDS per such array, one 16-byte chunk of the
// arrays in cmask (on four-byte boundaries for those in umask), single elements
// of the others.  In the LDS position l of the group and row y sit at word
// ((l % 4) * 65 + l / 4) * (F | 1) + y: the 64 lanes of a wavefront, on 64
// positions four apart and one row, then fall on 64 consecutive multiples of
// an odd pitch (no two on one bank beyond the two a bank serves anyway), and
// the words of the chunks that move between memory and the LDS, four rows
// apart on consecutive lanes, spread over the banks through the 65.
std::string gen_narrow_staged(const GpuElemwise *ge, bool idx64, unsigned F, unsigned sd, unsigned bmask,
                              unsigned cmask, unsigned ntmask, std::vector<int> &ktypes, unsigned umask,
                              unsigned nd) {
  std::string s;
  const char *I = idx64 ? "ga_ssize" : "ga_int";
  const char *N = idx64 ? "ga_size" : "ga_uint";
  const unsigned ld = sd == nd - 1 ? nd - 2 : nd - 1;
  const unsigned chunks = 64 * F;            // 16-byte chunks of a group's piece
  const unsigned Fp = F | 1;
  emit_header(ge, s);
  appendf(s, "#define GA_AT(l, y) ((((l) & 3u) * 65u + ((l) >> 2)) * %uu + (y))\n", Fp);
  if (umask) s += "typedef ga_uint __attribute__((ext_vector_type(4), aligned(4))) ga_chunk16u;\n";
  s += "KERNEL void __launch_bounds__(256) elem(const ga_size dim0";
  ktypes.push_back(GA_SIZE);
  for (unsigned d = 1; d < nd; d++) {
    appendf(s, ", const ga_size dim%u", d);
    ktypes.push_back(GA_SIZE);
  }
  std::vector<int> aidx(ge->args.size(), -1);
  {
    int k = 0;
    for (size_t j = 0; j < ge->args.size(); j++)
      if (ge->args[j].is_array()) aidx[j] = k++;
  }
  auto in = [&](unsigned mask, size_t j) { return aidx[j] >= 0 && ((mask >> aidx[j]) & 1u); };
  for (const ge_arg &a : ge->args) {
    if (a.is_array()) {
      appendf(s, ", GLOBAL_MEM %s *%s_data, const ga_size %s_offset", ctype(a.typecode), a.name.c_str(), a.name.c_str());
      ktypes.push_back(GA_BUFFER);
      ktypes.push_back(GA_SIZE);
      for (unsigned d = 0; d < nd; d++) {
        appendf(s, ", const ga_ssize %s_str_%u", a.name.c_str(), d);
        ktypes.push_back(GA_SSIZE);
      }
    } else {
      appendf(s, ", %s %s", ctype(a.typecode), a.name.c_str());
      ktypes.push_back(a.typecode);
    }
  }
  s += ", const ga_uint ga_gx, const ga_uint ga_ltx) {\n(void)ga_gx; (void)ga_ltx; (void)dim0; (void)dim1;\n";
  ktypes.push_back(GA_UINT);
  ktypes.push_back(GA_UINT);
  if (nd == 3) s += "const ga_uint ga_o = GID_0 / ga_gx;\nconst ga_uint ga_pc = GID_0 - ga_o * ga_gx;\n";
  else s += "const ga_uint ga_pc = GID_0;\n";
  for (size_t j = 0; j < ge->args.size(); j++) {
    const ge_arg &a = ge->args[j];
    if (!a.is_array()) continue;
    appendf(s, "GLOBAL_MEM char *%s_b = (GLOBAL_MEM char *)%s_data + %s_offset;\n", a.name.c_str(), a.name.c_str(),
            a.name.c_str());
    if (nd == 3) appendf(s, "%s_b += (%s)ga_o * (%s)%s_str_0;\n", a.name.c_str(), I, I, a.name.c_str());
    if (in(bmask, j)) appendf(s, "LOCAL_MEM %s %s_s[%u];\n", ctype(a.typecode), a.name.c_str(), 260 * Fp);
  }
  appendf(s, "const %s ga_l0 = (%s)ga_pc * 256u;\n", N, N);
  s += "const ga_uint ga_lx = LID_0 & 63u, ga_ly = LID_0 >> 6;\n";
  appendf(s, "const %s ga_l4 = ga_l0 + ga_lx * 4u;\n", N);
  appendf(s, "const bool ga_full = ga_l4 + 3u < (%s)dim%u;\n", N, ld);
  appendf(s, "const ga_uint ga_cnt = (ga_uint)((%s)dim%u - ga_l0 < 256u ? (%s)dim%u - ga_l0 : 256u) * %uu;\n", N, ld, N, ld, F);
  auto elem_at = [&](const ge_arg &a, const std::string &y, const std::string &l) {
    std::string e;
    appendf(e, "*(GLOBAL_MEM %s *)(%s_b + ((%s)(%s) * (%s)%s_str_%u + (%s)(%s) * (%s)%s_str_%u))", ctype(a.typecode),
            a.name.c_str(), I, y.c_str(), I, a.name.c_str(), sd, I, l.c_str(), I, a.name.c_str(), ld);
    return e;
  };
  auto piece_at = [&](const ge_arg &a, const char *cast, const std::string &bytes) {
    std::string e;
    appendf(e, "(GLOBAL_MEM %s *)(%s_b + (%s)ga_l0 * (%s)%s_str_%u + (%s))", cast, a.name.c_str(), I, I,
            a.name.c_str(), ld, bytes.c_str());
    return e;
  };
  bool staged_in = false, staged_out = false;
  for (size_t j = 0; j < ge->args.size(); j++) {
    const ge_arg &a = ge->args[j];
    if (!in(bmask, j)) continue;
    if (a.writes()) staged_out = true;
    if (!a.reads()) continue;
    staged_in = true;
    const bool nt = (ntmask >> aidx[j]) & 1u;
    appendf(s, "for (ga_uint ga_q = LID_0; ga_q < %uu; ga_q += 256u) {\n", chunks);
    appendf(s, "union { ga_chunk16 c; %s e[4]; } ga_v;\n", ctype(a.typecode));
    appendf(s, "if (ga_q * 4u + 3u < ga_cnt) ga_v.c = %s(%s);\n", nt ? "__builtin_nontemporal_load" : "*",
            piece_at(a, "const ga_chunk16", "ga_q * 16u").c_str());
    appendf(s, "else for (ga_uint ga_e = 0; ga_e < 4u; ga_e++) if (ga_q * 4u + ga_e < ga_cnt) ga_v.e[ga_e] = *(%s);\n",
            piece_at(a, ctype(a.typecode), "(ga_q * 4u + ga_e) * 4u").c_str());
    appendf(s, "for (ga_uint ga_e = 0; ga_e < 4u; ga_e++) { const ga_uint ga_w = ga_q * 4u + ga_e, ga_l = ga_w / %uu; "
               "%s_s[GA_AT(ga_l, ga_w - ga_l * %uu)] = ga_v.e[ga_e]; }\n", F, a.name.c_str(), F);
    s += "}\n";
  }
  if (staged_in) s += "local_barrier();\n";
  appendf(s, "for (ga_uint ga_y = ga_ly; ga_y < %uu; ga_y += 4u) {\n", F);
  // a lane's four values of the chunked arrays for this row
  for (size_t j = 0; j < ge->args.size(); j++) {
    const ge_arg &a = ge->args[j];
    if (!in(cmask, j)) continue;
    const char *ct = in(umask, j) ? "ga_chunk16u" : "ga_chunk16";
    const bool nt = (ntmask >> aidx[j]) & 1u;
    appendf(s, "union { ga_chunk16 c; %s e[4]; } %s_r;\n", ctype(a.typecode), a.name.c_str());
    if (!a.reads()) continue;
    std::string ptr;
    appendf(ptr, "(GLOBAL_MEM const %s *)&%s", ct, elem_at(a, "ga_y", "ga_l4").c_str());
    appendf(s, "if (ga_full) %s_r.c = %s(%s); else {\n", a.name.c_str(), nt ? "__builtin_nontemporal_load" : "*", ptr.c_str());
    for (unsigned e = 0; e < 4; e++) {
      char l[32];
      snprintf(l, sizeof(l), "ga_l4 + %uu", e);
      appendf(s, "if (ga_l4 + %uu < (%s)dim%u) %s_r.e[%u] = %s;\n", e, N, ld, a.name.c_str(), e, elem_at(a, "ga_y", l).c_str());
    }
    s += "}\n";
  }
  for (unsigned e = 0; e < 4; e++) {
    char l[32];
    snprintf(l, sizeof(l), "ga_l4 + %uu", e);
    appendf(s, "if (ga_l4 + %uu < (%s)dim%u) {\n", e, N, ld);
    auto place = [&](size_t j) {
      const ge_arg &a = ge->args[j];
      std::string x;
      if (in(bmask, j)) appendf(x, "%s_s[(%uu + ga_lx) * %uu + ga_y]", a.name.c_str(), e * 65, Fp);
      else if (in(cmask, j)) appendf(x, "%s_r.e[%u]", a.name.c_str(), e);
      else x = elem_at(a, "ga_y", l);
      return x;
    };
    for (size_t j = 0; j < ge->args.size(); j++)
      if (ge->args[j].is_array()) emit_load(ge, s, ge->args[j], place(j));
    s += ge->expr;
    s += ";\n";
    for (size_t j = 0; j < ge->args.size(); j++)
      if (ge->args[j].is_array() && ge->args[j].writes()) emit_store(ge, s, ge->args[j], place(j));
    s += "}\n";
  }
  for (size_t j = 0; j < ge->args.size(); j++) {
    const ge_arg &a = ge->args[j];
    if (!in(cmask, j) || !a.writes()) continue;
    const char *ct = in(umask, j) ? "ga_chunk16u" : "ga_chunk16";
    const bool nt = (ntmask >> aidx[j]) & 1u;
    std::string ptr;
    appendf(ptr, "(GLOBAL_MEM %s *)&%s", ct, elem_at(a, "ga_y", "ga_l4").c_str());
    if (nt) appendf(s, "if (ga_full) __builtin_nontemporal_store((%s)%s_r.c, %s); else {\n", ct, a.name.c_str(), ptr.c_str());
    else appendf(s, "if (ga_full) *(%s) = %s_r.c; else {\n", ptr.c_str(), a.name.c_str());
    for (unsigned e = 0; e < 4; e++) {
      char l[32];
      snprintf(l, sizeof(l), "ga_l4 + %uu", e);
      appendf(s, "if (ga_l4 + %uu < (%s)dim%u) %s = %s_r.e[%u];\n", e, N, ld, elem_at(a, "ga_y", l).c_str(), a.name.c_str(), e);
    }
    s += "}\n";
  }
  s += "}\n";
  if (staged_out) {
    s += "local_barrier();\n";
    for (size_t j = 0; j < ge->args.size(); j++) {
      const ge_arg &a = ge->args[j];
      if (!in(bmask, j) || !a.writes()) continue;
      const bool nt = (ntmask >> aidx[j]) & 1u;
      appendf(s, "for (ga_uint ga_q = LID_0; ga_q < %uu; ga_q += 256u) {\n", chunks);
      appendf(s, "union { ga_chunk16 c; %s e[4]; } ga_v;\n", ctype(a.typecode));
      appendf(s, "for (ga_uint ga_e = 0; ga_e < 4u; ga_e++) { const ga_uint ga_w = ga_q * 4u + ga_e, ga_l = ga_w / %uu; "
                 "ga_v.e[ga_e] = %s_s[GA_AT(ga_l, ga_w - ga_l * %uu)]; }\n", F, a.name.c_str(), F);
      const std::string ptr = piece_at(a, "ga_chunk16", "ga_q * 16u");
      if (nt) appendf(s, "if (ga_q * 4u + 3u < ga_cnt) __builtin_nontemporal_store(ga_v.c, %s);\n", ptr.c_str());
      else appendf(s, "if (ga_q * 4u + 3u < ga_cnt) *(%s) = ga_v.c;\n", ptr.c_str());
      appendf(s, "else for (ga_uint ga_e = 0; ga_e < 4u; ga_e++) if (ga_q * 4u + ga_e < ga_cnt) *(%s) = ga_v.e[ga_e];\n",
              piece_at(a, ctype(a.typecode), "(ga_q * 4u + ga_e) * 4u").c_str());
      s += "}\n";
    }
  }
  s += "}\n";
  return s;
}

// ---- tiles of short records -------------------------------------------------------
// Same parameters as the strided kernel with three or four dims: (planes,) Y, X
// and a short inner dim of F elements with unit stride in every array that has
// it - a record.  Every array has elements of es bytes (four in what follows;
// with others a lane's step is 16 / es elements and a block 64 / es).  The result and the arrays laid out like it have their
// records one after the other along X (stride of X = F elements); the arrays in
// tmask, read only, along Y (stride of Y = F elements): matrices of records taken
// as their transposes, (H, W, C) images turned, batch-major sequences of short
// feature vectors made time-major.  A group owns T x T records: of each array in
// tmask the T runs of T F contiguous elements (one per position of X) go to the
// LDS, four elements per lane through accesses that assume four-byte boundaries;
// then the lanes walk the T runs of the result (one per position of Y), four
// elements each, take the transposed arrays' elements out of the LDS and move
// the others directly.  ga_gx counts the tiles along X, ga_ltx those along Y.
// skew >= 0 (an array laid out like the result, normally the result): the window
// of a tile on a row is moved left by the 0 to 15 elements that put its first
// element on a 64-byte block of that array's row, so that a group stores whole
// blocks also where rows are no whole blocks long; the staged runs cover the
// records such a window can reach, and the grid has tiles for 15 more elements
// (T F must then be a multiple of 16: the windows of neighbouring tiles meet).
std::string gen_record_tiles(const GpuElemwise *ge, unsigned nd, bool idx64, unsigned F, unsigned T, unsigned tmask,
                             unsigned pmask, unsigned ntmask, std::vector<int> &ktypes, int skew = -1, unsigned es = 4,
                             bool ymajor = false) {
  std::string s;
  const char *I = idx64 ? "ga_ssize" : "ga_int";
  const unsigned R = T * F;          // elements of a run
  const unsigned V = 16 / es;        // elements per lane and step: a 16-byte chunk
  const unsigned B = 64 / es;        // elements of a 64-byte block
  const unsigned lg = es == 1 ? 0 : es == 2 ? 1 : es == 4 ? 2 : 3;
  const unsigned pitch = R + V;      // of a run in the LDS
  const unsigned extra = skew >= 0 ? (B - 1 + F - 1) / F + 1 : 0;   // records that a moved window can reach beyond the tile's
  const unsigned TS = T + extra;     // runs staged per transposed array
  const unsigned dy = nd - 3, dx = nd - 2, dc = nd - 1;
  emit_header(ge, s);
  appendf(s, "typedef ga_uint __attribute__((ext_vector_type(4), aligned(%u))) ga_chunk16u;\n", es < 4 ? es : 4);
  s += "KERNEL void __launch_bounds__(256) elem(const ga_size dim0";
  ktypes.push_back(GA_SIZE);
  for (unsigned d = 1; d < nd; d++) {
    appendf(s, ", const ga_size dim%u", d);
    ktypes.push_back(GA_SIZE);
  }
  std::vector<int> aidx(ge->args.size(), -1);
  int skew_j = -1;
  {
    int k = 0;
    for (size_t j = 0; j < ge->args.size(); j++)
      if (ge->args[j].is_array()) {
        if (k == skew) skew_j = (int)j;
        aidx[j] = k++;
      }
  }
  auto in = [&](unsigned mask, size_t j) { return aidx[j] >= 0 && ((mask >> aidx[j]) & 1u); };
  for (const ge_arg &a : ge->args) {
    if (a.is_array()) {
      appendf(s, ", GLOBAL_MEM %s *%s_data, const ga_size %s_offset", ctype(a.typecode), a.name.c_str(), a.name.c_str());
      ktypes.push_back(GA_BUFFER);
      ktypes.push_back(GA_SIZE);
      for (unsigned d = 0; d < nd; d++) {
        appendf(s, ", const ga_ssize %s_str_%u", a.name.c_str(), d);
        ktypes.push_back(GA_SSIZE);
      }
    } else {
      appendf(s, ", %s %s", ctype(a.typecode), a.name.c_str());
      ktypes.push_back(a.typecode);
    }
  }
  s += ", const ga_uint ga_gx, const ga_uint ga_ltx) {\n";
  ktypes.push_back(GA_UINT);
  ktypes.push_back(GA_UINT);
  if (ymajor)
    // tiles that follow one another along Y share the lines in which the transposed arrays' runs
    // begin and end: they get consecutive numbers, and consecutive numbers one die (group g runs
    // on die g % 8)
    s += "ga_uint ga_g = GID_0;\n{ const ga_uint ga_whole = GDIM_0 & ~7u; if (ga_g < ga_whole) ga_g = (ga_g % 8u) * (ga_whole / 8u) + ga_g / 8u; }\n"
         "const ga_uint ga_by = ga_g % ga_ltx; ga_g /= ga_ltx;\nconst ga_uint ga_bx = ga_g % ga_gx; ga_g /= ga_gx;\n";
  else
    s += "ga_uint ga_g = GID_0;\nconst ga_uint ga_bx = ga_g % ga_gx; ga_g /= ga_gx;\nconst ga_uint ga_by = ga_g % ga_ltx; ga_g /= ga_ltx;\n";
  // the tile: elements k0 .. k0 + R - 1 of the result's rows y0 .. y0 + T - 1; the transposed
  // arrays' records from xs on are staged
  appendf(s, "const ga_uint ga_k0 = ga_bx * %uu, ga_y0 = ga_by * %uu, ga_xf = (ga_uint)dim%u * %uu;\n", R, T, dx, F);
  if (skew >= 0) appendf(s, "const ga_uint ga_xs = ga_k0 >= %uu ? (ga_k0 - %uu) / %uu : 0u;\n", B - 1, B - 1, F);
  else appendf(s, "const ga_uint ga_xs = ga_bx * %uu;\n", T);
  appendf(s, "const ga_uint ga_ny = (ga_uint)dim%u - ga_y0 < %uu ? (ga_uint)dim%u - ga_y0 : %uu;\n", dy, T, dy, T);
  for (size_t j = 0; j < ge->args.size(); j++) {
    const ge_arg &a = ge->args[j];
    if (!a.is_array()) continue;
    appendf(s, "GLOBAL_MEM char *%s_b = (GLOBAL_MEM char *)%s_data + %s_offset + (%s)ga_y0 * (%s)%s_str_%u;\n", a.name.c_str(),
            a.name.c_str(), a.name.c_str(), I, I, a.name.c_str(), dy);
    if (nd == 4) appendf(s, "%s_b += (%s)ga_g * (%s)%s_str_0;\n", a.name.c_str(), I, I, a.name.c_str());
    if (in(tmask, j))
      appendf(s, "LOCAL_MEM %s %s_s[%u] __attribute__((aligned(16)));\n", ctype(a.typecode), a.name.c_str(), TS * pitch);
  }
  // the transposed arrays' runs into the LDS: run r (record xs + r along X), elements k .. k + 3 of it
  appendf(s, "for (ga_uint ga_i = LID_0 * %uu; ga_i < %uu; ga_i += %uu) {\n", V, TS * R, 256 * V);
  appendf(s, "const ga_uint ga_r = ga_i / %uu, ga_k = ga_i - ga_r * %uu;\n", R, R);
  appendf(s, "if (ga_xs + ga_r < (ga_uint)dim%u) {\n", dx);
  for (size_t j = 0; j < ge->args.size(); j++) {
    const ge_arg &a = ge->args[j];
    if (!in(tmask, j)) continue;
    const bool nt = (ntmask >> aidx[j]) & 1u;
    appendf(s, "{ GLOBAL_MEM const %s *ga_p = (GLOBAL_MEM const %s *)(%s_b + (%s)(ga_xs + ga_r) * (%s)%s_str_%u) + ga_k;\n",
            ctype(a.typecode), ctype(a.typecode), a.name.c_str(), I, I, a.name.c_str(), dx);
    appendf(s, "union { ga_chunk16u c; %s e[%u]; } ga_v;\n", ctype(a.typecode), V);
    appendf(s, "if (ga_k + %uu < ga_ny * %uu) ga_v.c = %s((GLOBAL_MEM const ga_chunk16u *)ga_p);\n", V - 1, F,
            nt ? "__builtin_nontemporal_load" : "*");
    appendf(s, "else for (ga_uint ga_e = 0; ga_e < %uu; ga_e++) if (ga_k + ga_e < ga_ny * %uu) ga_v.e[ga_e] = ga_p[ga_e];\n", V, F);
    appendf(s, "*(ga_chunk16u *)&%s_s[ga_r * %uu + ga_k] = ga_v.c; }\n", a.name.c_str(), pitch);
  }
  s += "}\n}\nlocal_barrier();\n";
  // the result's rows: row r (position y0 + r of Y), elements kk .. kk + 3 (record kk / F, element kk % F);
  // with moved windows a row's first element is the one on a 64-byte block of the array in skew at
  // or below element k0, and elements before the row wrap to huge indices that fail the extent test
  appendf(s, "for (ga_uint ga_i = LID_0 * %uu; ga_i < %uu; ga_i += %uu) {\n", V, T * R, 256 * V);
  appendf(s, "const ga_uint ga_r = ga_i / %uu, ga_k = ga_i - ga_r * %uu;\n", R, R);
  s += "if (ga_r >= ga_ny) continue;\n";
  if (skew_j >= 0) {
    const ge_arg &a = ge->args[skew_j];
    appendf(s, "const ga_uint ga_sh = (ga_uint)(((ga_size)(%s_b + (%s)ga_r * (%s)%s_str_%u) >> %u) + ga_k0) & %uu;\n",
            a.name.c_str(), I, I, a.name.c_str(), dy, lg, B - 1);
    s += "const ga_uint ga_kk = ga_k0 - ga_sh + ga_k;\n";
  } else {
    s += "const ga_uint ga_kk = ga_k0 + ga_k;\n";
  }
  appendf(s, "if (ga_kk >= ga_xf && ga_kk + %uu >= ga_xf) continue;\n", V - 1);
  appendf(s, "const bool ga_full = ga_kk < ga_xf && ga_kk + %uu < ga_xf;\n", V - 1);
  for (size_t j = 0; j < ge->args.size(); j++) {
    const ge_arg &a = ge->args[j];
    if (!in(pmask, j)) continue;
    const bool nt = (ntmask >> aidx[j]) & 1u;
    appendf(s, "GLOBAL_MEM %s *%s_p = (GLOBAL_MEM %s *)(%s_b + (%s)ga_r * (%s)%s_str_%u);\n", ctype(a.typecode),
            a.name.c_str(), ctype(a.typecode), a.name.c_str(), I, I, a.name.c_str(), dy);
    appendf(s, "union { ga_chunk16u c; %s e[%u]; } %s_v;\n", ctype(a.typecode), V, a.name.c_str());
    if (a.reads()) {
      appendf(s, "if (ga_full) %s_v.c = %s((GLOBAL_MEM const ga_chunk16u *)(%s_p + ga_kk));\n", a.name.c_str(),
              nt ? "__builtin_nontemporal_load" : "*", a.name.c_str());
      appendf(s, "else for (ga_uint ga_e = 0; ga_e < %uu; ga_e++) if ((ga_uint)(ga_kk + ga_e) < ga_xf) %s_v.e[ga_e] = %s_p[(ga_uint)(ga_kk + ga_e)];\n",
              V, a.name.c_str(), a.name.c_str());
    }
  }
  for (unsigned e = 0; e < V; e++) {
    appendf(s, "if ((ga_uint)(ga_kk + %uu) < ga_xf) {\n", e);
    appendf(s, "const ga_uint ga_x = (ga_uint)(ga_kk + %uu) / %uu, ga_c = (ga_uint)(ga_kk + %uu) - ga_x * %uu;\n", e, F, e, F);
    auto place = [&](size_t j) {
      const ge_arg &a = ge->args[j];
      std::string x;
      if (in(tmask, j)) appendf(x, "%s_s[(ga_x - ga_xs) * %uu + ga_r * %uu + ga_c]", a.name.c_str(), pitch, F);
      else if (in(pmask, j)) appendf(x, "%s_v.e[%u]", a.name.c_str(), e);
      else appendf(x, "*(GLOBAL_MEM %s *)(%s_b + (%s)ga_r * (%s)%s_str_%u + (%s)ga_x * (%s)%s_str_%u + (%s)ga_c * (%s)%s_str_%u)",
                   ctype(a.typecode), a.name.c_str(), I, I, a.name.c_str(), dy, I, I, a.name.c_str(), dx, I, I, a.name.c_str(), dc);
      return x;
    };
    for (size_t j = 0; j < ge->args.size(); j++)
      if (ge->args[j].is_array()) emit_load(ge, s, ge->args[j], place(j));
    s += ge->expr;
    s += ";\n";
    for (size_t j = 0; j < ge->args.size(); j++)
      if (ge->args[j].is_array() && ge->args[j].writes()) emit_store(ge, s, ge->args[j], place(j));
    s += "}\n";
  }
  for (size_t j = 0; j < ge->args.size(); j++) {
    const ge_arg &a = ge->args[j];
    if (!in(pmask, j) || !a.writes()) continue;
    const bool nt = (ntmask >> aidx[j]) & 1u;
    if (nt) appendf(s, "if (ga_full) __builtin_nontemporal_store(%s_v.c, (GLOBAL_MEM ga_chunk16u *)(%s_p + ga_kk));\n", a.name.c_str(), a.name.c_str());
    else appendf(s, "if (ga_full) *(GLOBAL_MEM ga_chunk16u *)(%s_p + ga_kk) = %s_v.c;\n", a.name.c_str(), a.name.c_str());
    appendf(s, "else for (ga_uint ga_e = 0; ga_e < %uu; ga_e++) if ((ga_uint)(ga_kk + ga_e) < ga_xf) %s_p[(ga_uint)(ga_kk + ga_e)] = %s_v.e[ga_e];\n",
            V, a.name.c_str(), a.name.c_str());
  }
  s += "}\n}\n";
  return s;
}

// ---- strided kernel -------------------------------------------------------------
// elem(dim0..dim{nd-1}, {data, byte offset, str_0..str_{nd-1} | scalar}...,
//      ga_gx, ga_ltx)
//
// Dims arrive sorted and collapsed; x = dim nd-1 is the output's fastest dim.
//
// Plain variant (no transposed operand): a group is TX x TY lanes (TX =
// 1 << ga_ltx, 256 lanes in all).  Lane (tx, ty) of group (bx, by) owns row
// by*TY + ty of the nd-1 outer dims and the columns (bx*4 + e)*TX + tx,
// e = 0..3.  The group id is split with one division; the row is unravelled
// once.
//
// Transposed variant: y = dim nd-2 is where the transposed operands have
// their small stride.  A group handles a 64 (y) x 64 (x) tile with 64 x 4
// lanes; transposed reads enter through LDS (lanes along y), the expression
// runs with lanes along x, transposed writes leave through LDS.
std::string gen_strided(const GpuElemwise *ge, unsigned nd, bool idx64, unsigned tmask,
                        std::vector<int> &ktypes) {
  std::string s;
  const char *I = idx64 ? "ga_ssize" : "ga_int";     // byte offsets
  const char *N = idx64 ? "ga_size" : "ga_uint";     // counts
  emit_header(ge, s);
  s += "KERNEL void __launch_bounds__(256) elem(";
  for (unsigned d = 0; d < nd; d++) {
    appendf(s, "%sconst ga_size dim%u", d ? ", " : "", d);
    ktypes.push_back(GA_SIZE);
  }
  for (const ge_arg &a : ge->args) {
    if (a.is_array()) {
      appendf(s, ", GLOBAL_MEM %s *%s_data, const ga_size %s_offset", ctype(a.typecode),
              a.name.c_str(), a.name.c_str());
      ktypes.push_back(GA_BUFFER);
      ktypes.push_back(GA_SIZE);
      for (unsigned d = 0; d < nd; d++) {
        appendf(s, ", const ga_ssize %s_str_%u", a.name.c_str(), d);
        ktypes.push_back(GA_SSIZE);
      }
    } else {
      appendf(s, ", %s %s", ctype(a.typecode), a.name.c_str());
      ktypes.push_back(a.typecode);
    }
  }
  s += ", const ga_uint ga_gx, const ga_uint ga_ltx) {\n";
  ktypes.push_back(GA_UINT);
  ktypes.push_back(GA_UINT);

  // array index among arrays, for the transposed mask
  std::vector<int> aidx(ge->args.size(), -1);
  {
    int k = 0;
    for (size_t j = 0; j < ge->args.size(); j++)
      if (ge->args[j].is_array()) aidx[j] = k++;
  }
  auto is_t = [&](size_t j) { return aidx[j] >= 0 && ((tmask >> aidx[j]) & 1u); };

  for (const ge_arg &a : ge->args)
    if (a.is_array())
      appendf(s, "GLOBAL_MEM char *%s_b = (GLOBAL_MEM char *)%s_data + %s_offset;\n",
              a.name.c_str(), a.name.c_str(), a.name.c_str());

  if (tmask == 0) {
    appendf(s, "const %s ga_tx = LID_0 & ((1u << ga_ltx) - 1u);\n", N);
    appendf(s, "const %s ga_ty = LID_0 >> ga_ltx;\n", N);
    appendf(s, "const %s ga_bx = GID_0 %% ga_gx;\n", N);
    appendf(s, "const %s ga_by = GID_0 / ga_gx;\n", N);
    appendf(s, "%s ga_rows = 1;\n", N);
    for (unsigned d = 0; d + 1 < nd; d++) appendf(s, "ga_rows *= (%s)dim%u;\n", N, d);
    appendf(s, "const %s ga_row = ga_by * (256u >> ga_ltx) + ga_ty;\n", N);
    s += "if (ga_row >= ga_rows) return;\n";
    // unravel the row over dims nd-2 .. 0
    for (const ge_arg &a : ge->args)
      if (a.is_array()) appendf(s, "%s %s_o = 0;\n", I, a.name.c_str());
    if (nd >= 2) {
      appendf(s, "{ %s ga_r = ga_row; %s ga_c;\n", N, N);
      for (unsigned d = nd - 1; d-- > 0;) {
        if (d > 0) appendf(s, "ga_c = ga_r %% (%s)dim%u; ga_r = ga_r / (%s)dim%u;\n", N, d, N, d);
        else s += "ga_c = ga_r;\n";
        for (const ge_arg &a : ge->args)
          if (a.is_array())
            appendf(s, "%s_o += (%s)ga_c * (%s)%s_str_%u;\n", a.name.c_str(), I, I,
                    a.name.c_str(), d);
      }
      s += "}\n";
    }
    const unsigned xd = nd - 1;
    appendf(s, "const %s ga_x0 = (ga_bx * 4u << ga_ltx) + ga_tx;\n", N);
    s += "#pragma unroll\nfor (int ga_e = 0; ga_e < 4; ga_e++) {\n";
    appendf(s, "const %s ga_x = ga_x0 + ((%s)ga_e << ga_ltx);\n", N, N);
    appendf(s, "if (ga_x < (%s)dim%u) {\n", N, xd);
    for (const ge_arg &a : ge->args) {
      if (!a.is_array()) continue;
      std::string at;
      appendf(at, "*(GLOBAL_MEM %s *)(%s_b + (%s_o + (%s)ga_x * (%s)%s_str_%u))", ctype(a.typecode),
              a.name.c_str(), a.name.c_str(), I, I, a.name.c_str(), xd);
      emit_load(ge, s, a, at);
    }
    s += ge->expr;
    s += ";\n";
    for (const ge_arg &a : ge->args) {
      if (!a.is_array()) continue;
      std::string at;
      appendf(at, "*(GLOBAL_MEM %s *)(%s_b + (%s_o + (%s)ga_x * (%s)%s_str_%u))", ctype(a.typecode),
              a.name.c_str(), a.name.c_str(), I, I, a.name.c_str(), xd);
      emit_store(ge, s, a, at);
    }
    s += "}\n}\n}\n";
    return s;
  }

  // transposed variant, nd >= 2
  const unsigned xd = nd - 1, yd = nd - 2;
  for (size_t j = 0; j < ge->args.size(); j++)
    if (is_t(j))
      appendf(s, "LOCAL_MEM %s %s_t[64 * 65];\n", ctype(ge->args[j].typecode),
              ge->args[j].name.c_str());
  appendf(s, "const %s ga_tx = LID_0 & 63u;\nconst %s ga_ty = LID_0 >> 6;\n", N, N);
  appendf(s, "const %s ga_gy = ((%s)dim%u + 63u) / 64u;\n", N, N, yd);
  appendf(s, "const %s ga_bx = GID_0 %% ga_gx;\n", N);
  appendf(s, "%s ga_r = GID_0 / ga_gx;\n", N);
  appendf(s, "const %s ga_by = ga_r %% ga_gy;\nga_r = ga_r / ga_gy;\n", N);
  for (const ge_arg &a : ge->args)
    if (a.is_array()) appendf(s, "%s %s_o = 0;\n", I, a.name.c_str());
  if (nd >= 3) {
    appendf(s, "{ %s ga_c;\n", N);
    for (unsigned d = nd - 2; d-- > 0;) {
      if (d > 0) appendf(s, "ga_c = ga_r %% (%s)dim%u; ga_r = ga_r / (%s)dim%u;\n", N, d, N, d);
      else s += "ga_c = ga_r;\n";
      for (const ge_arg &a : ge->args)
        if (a.is_array())
          appendf(s, "%s_o += (%s)ga_c * (%s)%s_str_%u;\n", a.name.c_str(), I, I, a.name.c_str(),
                  d);
    }
    s += "}\n";
  }
  appendf(s, "const %s ga_x0 = ga_bx * 64u;\nconst %s ga_y0 = ga_by * 64u;\n", N, N);
  auto gaddr = [&](const ge_arg &a, const char *y, const char *x) {
    std::string at;
    appendf(at, "*(GLOBAL_MEM %s *)(%s_b + (%s_o + (%s)(%s) * (%s)%s_str_%u + (%s)(%s) * (%s)%s_str_%u))",
            ctype(a.typecode), a.name.c_str(), a.name.c_str(), I, y, I, a.name.c_str(), yd, I, x,
            I, a.name.c_str(), xd);
    return at;
  };
  // phase 1: transposed reads, lanes along y
  bool any_tr = false, any_tw = false;
  for (size_t j = 0; j < ge->args.size(); j++) {
    if (!is_t(j)) continue;
    if (ge->args[j].reads()) any_tr = true;
    if (ge->args[j].writes()) any_tw = true;
  }
  // Every global load of a phase is issued into registers before its first
  // use, so a lane has 16 loads in flight instead of one.
  if (any_tr) {
    for (size_t j = 0; j < ge->args.size(); j++)
      if (is_t(j) && ge->args[j].reads())
        appendf(s, "%s %s_r[16];\n", ctype(ge->args[j].typecode), ge->args[j].name.c_str());
    s += "#pragma unroll\nfor (int ga_k = 0; ga_k < 16; ga_k++) {\n";
    appendf(s, "const %s ga_ly = ga_tx, ga_lx = ga_ty + 4u * (%s)ga_k;\n", N, N);
    appendf(s, "if (ga_y0 + ga_ly < (%s)dim%u && ga_x0 + ga_lx < (%s)dim%u) {\n", N, yd, N, xd);
    for (size_t j = 0; j < ge->args.size(); j++) {
      const ge_arg &a = ge->args[j];
      if (!is_t(j) || !a.reads()) continue;
      appendf(s, "%s_r[ga_k] = %s;\n", a.name.c_str(),
              gaddr(a, "ga_y0 + ga_ly", "ga_x0 + ga_lx").c_str());
    }
    s += "}\n}\n";
    s += "#pragma unroll\nfor (int ga_k = 0; ga_k < 16; ga_k++) {\n";
    appendf(s, "const %s ga_ly = ga_tx, ga_lx = ga_ty + 4u * (%s)ga_k;\n", N, N);
    appendf(s, "if (ga_y0 + ga_ly < (%s)dim%u && ga_x0 + ga_lx < (%s)dim%u) {\n", N, yd, N, xd);
    for (size_t j = 0; j < ge->args.size(); j++) {
      const ge_arg &a = ge->args[j];
      if (!is_t(j) || !a.reads()) continue;
      appendf(s, "%s_t[ga_lx * 65u + ga_ly] = %s_r[ga_k];\n", a.name.c_str(), a.name.c_str());
    }
    s += "}\n}\nlocal_barrier();\n";
  }
  // phase 2: expression, lanes along x
  for (size_t j = 0; j < ge->args.size(); j++) {
    const ge_arg &a = ge->args[j];
    if (a.is_array() && !is_t(j) && a.reads())
      appendf(s, "%s %s_g[16];\n", ctype(a.typecode), a.name.c_str());
  }
  s += "#pragma unroll\nfor (int ga_k = 0; ga_k < 16; ga_k++) {\n";
  appendf(s, "const %s ga_lx = ga_tx, ga_ly = ga_ty + 4u * (%s)ga_k;\n", N, N);
  appendf(s, "if (ga_y0 + ga_ly < (%s)dim%u && ga_x0 + ga_lx < (%s)dim%u) {\n", N, yd, N, xd);
  for (size_t j = 0; j < ge->args.size(); j++) {
    const ge_arg &a = ge->args[j];
    if (a.is_array() && !is_t(j) && a.reads())
      appendf(s, "%s_g[ga_k] = %s;\n", a.name.c_str(),
              gaddr(a, "ga_y0 + ga_ly", "ga_x0 + ga_lx").c_str());
  }
  s += "}\n}\n";
  s += "#pragma unroll\nfor (int ga_k = 0; ga_k < 16; ga_k++) {\n";
  appendf(s, "const %s ga_lx = ga_tx, ga_ly = ga_ty + 4u * (%s)ga_k;\n", N, N);
  appendf(s, "if (ga_y0 + ga_ly < (%s)dim%u && ga_x0 + ga_lx < (%s)dim%u) {\n", N, yd, N, xd);
  for (size_t j = 0; j < ge->args.size(); j++) {
    const ge_arg &a = ge->args[j];
    if (!a.is_array()) continue;
    if (is_t(j)) emit_load(ge, s, a, a.name + "_t[ga_lx * 65u + ga_ly]");
    else emit_load(ge, s, a, a.name + "_g[ga_k]");
  }
  s += ge->expr;
  s += ";\n";
  for (size_t j = 0; j < ge->args.size(); j++) {
    const ge_arg &a = ge->args[j];
    if (!a.is_array()) continue;
    if (is_t(j)) emit_store(ge, s, a, a.name + "_t[ga_lx * 65u + ga_ly]");
    else emit_store(ge, s, a, gaddr(a, "ga_y0 + ga_ly", "ga_x0 + ga_lx"));
  }
  s += "}\n}\n";
  // phase 3: transposed writes, lanes along y
  if (any_tw) {
    s += "local_barrier();\n#pragma unroll\nfor (int ga_k = 0; ga_k < 16; ga_k++) {\n";
    appendf(s, "const %s ga_ly = ga_tx, ga_lx = ga_ty + 4u * (%s)ga_k;\n", N, N);
    appendf(s, "if (ga_y0 + ga_ly < (%s)dim%u && ga_x0 + ga_lx < (%s)dim%u) {\n", N, yd, N, xd);
    for (size_t j = 0; j < ge->args.size(); j++) {
      const ge_arg &a = ge->args[j];
      if (!is_t(j) || !a.writes()) continue;
      appendf(s, "%s = %s_t[ga_lx * 65u + ga_ly];\n",
              gaddr(a, "ga_y0 + ga_ly", "ga_x0 + ga_lx").c_str(), a.name.c_str());
    }
    s += "}\n}\n";
  }
  s += "}\n";
  return s;
}


// ---- strided kernel, four elements per lane -------------------------------------
// Same arguments as the scalar strided kernel.  Preconditions checked by the
// caller: the x extent (and the y extent when operands are transposed) is a
// multiple of 4, element sizes are at most 8 bytes, and every array marked in
// `umask` (unit stride along x) or `tmask` (unit stride along y) has its base
// and all its other strides aligned to 4 elements, so that a lane can move 4
// consecutive elements with one access.  Arrays in neither mask (broadcast or
// oddly strided along x) are accessed element by element.
//
// Plain variant: a lane owns one row and 4 quads TX quads apart; all loads
// of the 16 elements are issued before the first use.
// Transposed variant: 64 x 64 tile.  Transposed reads: a lane loads 4
// consecutive y of one x column and scatters them into the padded tile;
// the expression runs on 4 consecutive x of one y row; transposed writes
// gather 4 consecutive y from the tile and store them with one access.
std::string gen_strided_vec(const GpuElemwise *ge, unsigned nd, bool idx64, unsigned tmask,
                            unsigned umask, std::vector<int> &ktypes, unsigned ntmask = 0,
                            unsigned tile = 64, unsigned zmask = 0, unsigned quads = 4, unsigned vq = 4,
                            bool pairs_ok = true, unsigned skew = 0, bool loose = false) {
  std::string s;
  // elements a lane moves at a time: 4, or (plain variant only) 2 when the
  // widest type has 8 bytes, so that the widest access stays at 16 bytes
  const unsigned VQ = tmask ? 4 : vq;
  const char *I = idx64 ? "ga_ssize" : "ga_int";
  const char *N = idx64 ? "ga_size" : "ga_uint";
  emit_header(ge, s);
  if (loose) s += "typedef ga_uint __attribute__((ext_vector_type(4), aligned(4))) ga_chunk16u;\n";
  appendf(s, "KERNEL void __launch_bounds__(%u) elem(", tmask ? tile * tile / 16 : 256u);
  for (unsigned d = 0; d < nd; d++) {
    appendf(s, "%sconst ga_size dim%u", d ? ", " : "", d);
    ktypes.push_back(GA_SIZE);
  }
  for (const ge_arg &a : ge->args) {
    if (a.is_array()) {
      appendf(s, ", GLOBAL_MEM %s *%s_data, const ga_size %s_offset", ctype(a.typecode),
              a.name.c_str(), a.name.c_str());
      ktypes.push_back(GA_BUFFER);
      ktypes.push_back(GA_SIZE);
      for (unsigned d = 0; d < nd; d++) {
        appendf(s, ", const ga_ssize %s_str_%u", a.name.c_str(), d);
        ktypes.push_back(GA_SSIZE);
      }
    } else {
      appendf(s, ", %s %s", ctype(a.typecode), a.name.c_str());
      ktypes.push_back(a.typecode);
    }
  }
  s += ", const ga_uint ga_gx, const ga_uint ga_ltx) {\n";
  ktypes.push_back(GA_UINT);
  ktypes.push_back(GA_UINT);

  std::vector<int> aidx(ge->args.size(), -1);
  {
    int k = 0;
    for (size_t j = 0; j < ge->args.size(); j++)
      if (ge->args[j].is_array()) aidx[j] = k++;
  }
  auto is_t = [&](size_t j) { return aidx[j] >= 0 && ((tmask >> aidx[j]) & 1u); };
  auto is_u = [&](size_t j) { return aidx[j] >= 0 && ((umask >> aidx[j]) & 1u); };
  // read-only arrays whose stride along x is zero: one load serves a lane's four elements
  auto is_z = [&](size_t j) {
    return aidx[j] >= 0 && ((zmask >> aidx[j]) & 1u) && !ge->args[j].writes();
  };
  // the same along y (bits 16.. of zmask; transposed variant only): one load
  // serves the four rows a lane works on
  auto is_y = [&](size_t j) {
    return skew == 0 && aidx[j] >= 0 && ((zmask >> (16 + aidx[j])) & 1u) && !ge->args[j].writes();
  };
  auto quad_t = [&](const ge_arg &a) {
    return loose ? "ga_chunk16u" : chunk_type(gpuarray_get_elsize(a.typecode) * VQ);
  };
  // 16-byte accesses of arrays whose every element is touched once carry the
  // streaming hint (ntmask); broadcast operands stay cacheable
  auto is_nt = [&](size_t j) { return aidx[j] >= 0 && ((ntmask >> aidx[j]) & 1u); };
  auto quad_load = [&](size_t j, const std::string &dst, const std::string &ptr_expr) {
    // ptr_expr is "*(T *)(addr)": strip the leading '*' to get the pointer
    std::string o;
    if (is_nt(j)) appendf(o, "%s = __builtin_nontemporal_load(%s);\n", dst.c_str(), ptr_expr.c_str() + 1);
    else appendf(o, "%s = %s;\n", dst.c_str(), ptr_expr.c_str());
    return o;
  };
  auto quad_store = [&](size_t j, const std::string &ptr_expr, const std::string &val) {
    std::string o;
    if (is_nt(j)) appendf(o, "__builtin_nontemporal_store(%s, %s);\n", val.c_str(), ptr_expr.c_str() + 1);
    else appendf(o, "%s = %s;\n", ptr_expr.c_str(), val.c_str());
    return o;
  };

  for (const ge_arg &a : ge->args)
    if (a.is_array())
      appendf(s, "GLOBAL_MEM char *%s_b = (GLOBAL_MEM char *)%s_data + %s_offset;\n",
              a.name.c_str(), a.name.c_str(), a.name.c_str());
  const unsigned xd = nd - 1;

  // element (q, i) of array a, given the row offset expression `rowoff`
  auto elem_at = [&](const ge_arg &a, const std::string &rowoff, const std::string &x) {
    std::string at;
    appendf(at, "*(GLOBAL_MEM %s *)(%s_b + (%s + (%s)(%s) * (%s)%s_str_%u))", ctype(a.typecode),
            a.name.c_str(), rowoff.c_str(), I, x.c_str(), I, a.name.c_str(), xd);
    return at;
  };
  auto quad_at = [&](const ge_arg &a, const std::string &rowoff, const std::string &x) {
    std::string at;
    appendf(at, "*(GLOBAL_MEM %s *)(%s_b + (%s + (%s)(%s) * (%s)%s_str_%u))", quad_t(a),
            a.name.c_str(), rowoff.c_str(), I, x.c_str(), I, a.name.c_str(), xd);
    return at;
  };

  if (tmask == 0) {
    appendf(s, "const %s ga_tx = LID_0 & ((1u << ga_ltx) - 1u);\n", N);
    appendf(s, "const %s ga_ty = LID_0 >> ga_ltx;\n", N);
    appendf(s, "const %s ga_bx = GID_0 %% ga_gx;\nconst %s ga_by = GID_0 / ga_gx;\n", N, N);
    appendf(s, "%s ga_rows = 1;\n", N);
    for (unsigned d = 0; d + 1 < nd; d++) appendf(s, "ga_rows *= (%s)dim%u;\n", N, d);
    appendf(s, "const %s ga_row = ga_by * (256u >> ga_ltx) + ga_ty;\n", N);
    s += "if (ga_row >= ga_rows) return;\n";
    for (const ge_arg &a : ge->args)
      if (a.is_array()) appendf(s, "%s %s_o = 0;\n", I, a.name.c_str());
    if (nd >= 2) {
      appendf(s, "{ %s ga_r = ga_row; %s ga_c;\n", N, N);
      for (unsigned d = nd - 1; d-- > 0;) {
        if (d > 0) appendf(s, "ga_c = ga_r %% (%s)dim%u; ga_r = ga_r / (%s)dim%u;\n", N, d, N, d);
        else s += "ga_c = ga_r;\n";
        for (const ge_arg &a : ge->args)
          if (a.is_array())
            appendf(s, "%s_o += (%s)ga_c * (%s)%s_str_%u;\n", a.name.c_str(), I, I,
                    a.name.c_str(), d);
      }
      s += "}\n";
    }
    // quad index q = (bx*quads + e) * TX + tx, x = VQ*q
    appendf(s, "const %s ga_q0 = (ga_bx * %uu << ga_ltx) + ga_tx;\n", N, quads);
    appendf(s, "const %s ga_nq = (%s)dim%u / %uu;\n", N, N, xd, VQ);
    // loose (four-byte elements on any layout, `skew` names the result): the
    // quads of a row start ga_sy elements before it, so that the result's lie
    // on 16-byte boundaries; a quad that an end of the row cuts is moved
    // element by element (positions before the row wrap to huge values)
    const char *skew_name = nullptr;
    for (size_t j = 0; j < ge->args.size(); j++)
      if (loose && skew && aidx[j] == (int)skew - 1) skew_name = ge->args[j].name.c_str();
    if (loose)
      appendf(s, "const %s ga_sy = (%s)((((ga_size)%s_b + (ga_size)(ga_ssize)%s_o) & 15u) >> 2);\n", N, N,
              skew_name, skew_name);
    const std::string XQ = loose ? " - ga_sy" : "";
    const std::string WHOLE = loose ? " && ga_x + 3u < (" + std::string(N) + ")dim" + std::to_string(xd) : "";
    auto emit_cut = [&](bool store) {
      if (!loose) return;
      s += "else {\n";
      for (size_t j = 0; j < ge->args.size(); j++) {
        const ge_arg &a = ge->args[j];
        if (!a.is_array() || !(store ? a.writes() : a.reads())) continue;
        for (int i = 0; i < 4; i++) {
          char xi[32];
          snprintf(xi, sizeof(xi), "ga_x + %du", i);
          const std::string at = elem_at(a, a.name + "_o", (!store && is_z(j)) ? "0" : xi);
          if (store) appendf(s, "if (%s < (%s)dim%u) %s = %s_u[ga_e].e[%d];\n", xi, N, xd, at.c_str(), a.name.c_str(), i);
          else appendf(s, "if (%s < (%s)dim%u) %s_u[ga_e].e[%d] = %s;\n", xi, N, xd, a.name.c_str(), i, at.c_str());
        }
      }
      s += "}\n";
    };
    for (const ge_arg &a : ge->args)
      if (a.is_array())
        appendf(s, "union { %s c; %s e[%u]; } %s_u[4];\n", quad_t(a), ctype(a.typecode), VQ,
                a.name.c_str());
    appendf(s, "#pragma unroll\nfor (int ga_e = 0; ga_e < %u; ga_e++) {\n", quads);
    appendf(s, "const %s ga_x = %uu * (ga_q0 + ((%s)ga_e << ga_ltx))%s;\n", N, VQ, N, XQ.c_str());
    appendf(s, "if (ga_x < (%s)dim%u%s) {\n", N, xd, WHOLE.c_str());
    for (size_t j = 0; j < ge->args.size(); j++) {
      const ge_arg &a = ge->args[j];
      if (!a.is_array() || !a.reads()) continue;
      if (is_u(j)) {
        s += quad_load(j, a.name + "_u[ga_e].c", quad_at(a, a.name + "_o", "ga_x"));
      } else if (is_z(j)) {
        appendf(s, "%s_u[ga_e].e[0] = %s;\n", a.name.c_str(), elem_at(a, a.name + "_o", "0").c_str());
        for (int i = 1; i < (int)VQ; i++)
          appendf(s, "%s_u[ga_e].e[%d] = %s_u[ga_e].e[0];\n", a.name.c_str(), i, a.name.c_str());
      } else {
        for (int i = 0; i < (int)VQ; i++) {
          char xi[32];
          snprintf(xi, sizeof(xi), "ga_x + %du", i);
          appendf(s, "%s_u[ga_e].e[%d] = %s;\n", a.name.c_str(), i,
                  elem_at(a, a.name + "_o", xi).c_str());
        }
      }
    }
    s += "}\n";
    emit_cut(false);
    s += "}\n";
    appendf(s, "#pragma unroll\nfor (int ga_e = 0; ga_e < %u; ga_e++) {\n", quads);
    appendf(s, "const %s ga_x = %uu * (ga_q0 + ((%s)ga_e << ga_ltx))%s;\n", N, VQ, N, XQ.c_str());
    if (loose) {
      // some element of the quad in the row (a quad that starts before the row has wrapped)
      appendf(s, "if (ga_x < (%s)dim%u || ga_x + 3u < 3u) {\n", N, xd);
      appendf(s, "#pragma unroll\nfor (int ga_v = 0; ga_v < %u; ga_v++) if (ga_x + ga_v < (%s)dim%u) {\n", VQ, N, xd);
    } else {
      appendf(s, "if (ga_x < (%s)dim%u) {\n", N, xd);
      appendf(s, "#pragma unroll\nfor (int ga_v = 0; ga_v < %u; ga_v++) {\n", VQ);
    }
    for (const ge_arg &a : ge->args)
      if (a.is_array()) emit_load(ge, s, a, a.name + "_u[ga_e].e[ga_v]");
    s += ge->expr;
    s += ";\n";
    for (const ge_arg &a : ge->args)
      if (a.is_array()) emit_store(ge, s, a, a.name + "_u[ga_e].e[ga_v]");
    s += "}\n";
    if (loose) appendf(s, "if (ga_x < (%s)dim%u%s) {\n", N, xd, WHOLE.c_str());
    for (size_t j = 0; j < ge->args.size(); j++) {
      const ge_arg &a = ge->args[j];
      if (!a.is_array() || !a.writes()) continue;
      if (is_u(j)) {
        s += quad_store(j, quad_at(a, a.name + "_o", "ga_x"), a.name + "_u[ga_e].c");
      } else {
        for (int i = 0; i < (int)VQ; i++) {
          char xi[32];
          snprintf(xi, sizeof(xi), "ga_x + %du", i);
          appendf(s, "%s = %s_u[ga_e].e[%d];\n", elem_at(a, a.name + "_o", xi).c_str(),
                  a.name.c_str(), i);
        }
      }
    }
    if (loose) {
      s += "}\n";
      emit_cut(true);
    }
    s += "}\n}\n}\n";
    return s;
  }

  // ---- transposed, nd >= 2 ----
  const unsigned yd = nd - 2;
  const unsigned T = tile, Q = tile / 4;
  // Rows of the array `skew` names (its number among the arrays, plus one; a
  // direct result of four-byte elements) that do not start on 64-byte
  // boundaries: a tile's window on row y is moved left by the ga_sy elements
  // (0, 4, 8 or 12) that put its first element on such a boundary, so that a
  // group stores whole 64-byte blocks only; the blocks a rectangular tile
  // would share with its neighbours reach memory as two partial writes
  // (out = in.T of 8192 x 8192 floats, rows 32 bytes into a line: 136 us
  // against 89 on whole lines).  The staged tiles then hold SK more columns,
  // fetched by one more pass of the group, and the grid has tiles for SK more
  // columns than the rows have.
  // `loose` (every array of four-byte elements): nothing is asked of bases,
  // pitches and extents.  A lane's four elements are then one access that is
  // only known to lie on a four-byte boundary (the windows still put the
  // result's on 16), rows can start at any of the 16 elements of a block, and
  // the quads that an extent cuts are moved element by element.
  const unsigned SK = skew ? (loose ? 15u : 12u) : 0u, W = T + SK, LP = W | 1u;   // (an odd pitch of the staged tile, for its banks)
  const unsigned NP = (W + Q - 1) / Q;      // passes of Q columns over a staged tile
  const std::string TP = std::to_string(LP) + "u";
  const char *skew_name = nullptr;
  for (size_t j = 0; j < ge->args.size(); j++)
    if (skew && aidx[j] == (int)skew - 1) skew_name = ge->args[j].name.c_str();
  const char *XB = skew ? "ga_xs" : "ga_x0";   // where a row's window starts
  // (inside a loop over the lane's rows: the window of row ga_y0 + ga_ly)
  auto emit_row_window = [&]() {
    if (!skew) return;
    appendf(s, "const %s ga_sy = (%s)((((ga_size)%s_b + (ga_size)(ga_ssize)(%s_o + (%s)(ga_y0 + ga_ly) * (%s)%s_str_%u)) & 63u) >> 2);\n",
            N, N, skew_name, skew_name, I, I, skew_name, yd);
    appendf(s, "const %s ga_xs = ga_x0 - ga_sy;\n", N);
  };
  // column of the staged tile that holds element GA_QP(v) of the row's window
  const std::string TCOL = skew ? std::to_string(SK) + "u - ga_sy + " : "";
  // x of column ga_lx of the staged tile (below 0 wraps to a huge value and fails the extent test)
  const std::string TX = skew ? "ga_x0 + ga_lx - " + std::to_string(SK) + "u" : "ga_x0 + ga_lx";
  const std::string LXOK = NP * Q > W ? "ga_lx < " + std::to_string(W) + "u && " : "";
  // A lane's four elements along an axis (its "quad").  With elements of up
  // to four bytes they are adjacent, one access of up to 16 bytes.  With
  // eight-byte elements in the kernel they are two pairs, half a tile apart:
  // four adjacent doubles per lane are two 16-byte accesses that lie 32 bytes
  // from the neighbouring lane's, so every access instruction of a wavefront
  // touches twice the lines it uses; as pairs, the 16 lanes of a line cover
  // two runs of 256 contiguous bytes.  Measured on MI355X, kernel time, quads /
  // pairs: out = in.T of 4096 x 4096 doubles 47.3 / 44.6 us (71 -> 75 % of
  // peak), a.T + b on the same 70.1 / 66.3; kernels of narrower elements
  // keep their adjacent quads (out = in.T of 8192 x 8192 floats 81.6 us either way).
  size_t widest = 1;
  for (const ge_arg &a : ge->args)
    if (a.is_array()) widest = std::max(widest, gpuarray_get_elsize(a.typecode));
  const bool halves = widest == 8 && pairs_ok;
  const unsigned NH = halves ? 2 : 1, VE = 4 / NH;   // accesses per quad, elements per access
  auto vec_t = [&](const ge_arg &a) {
    return loose ? "ga_chunk16u" : chunk_type(gpuarray_get_elsize(a.typecode) * VE);
  };
  for (size_t j = 0; j < ge->args.size(); j++)
    if (is_t(j))
      appendf(s, "LOCAL_MEM %s %s_t[%u * %u];\n", ctype(ge->args[j].typecode),
              ge->args[j].name.c_str(), T, LP);
  // T x T tile, T*T/16 lanes: ga_lo picks a quad along one axis, ga_hi a line
  // along the other; four passes of T/4 lines cover the tile
  // Lane -> (quad ga_lo, line ga_hi): the quad from the low bits, so that 16
  // adjacent lanes touch 256 contiguous bytes of one line.  With a row pitch
  // of T + 1 words this puts two (T = 64) or four (T = 128) of every 32 lanes
  // on the same local-memory bank in both phases (the bank-conflict counter
  // reads half of the LDS cycles for T = 64); a lane order that avoids it (8
  // quads x 4 lines per 32 lanes) halves the contiguous run to 128 bytes and
  // measured no faster at 4096 x 4096 and 4 to 10 % slower at 8192 x 8192 and
  // 16384 x 16384: the kernel waits on memory, not on LDS.
  appendf(s, "const %s ga_lo = LID_0 & %uu;\nconst %s ga_hi = LID_0 / %uu;\n", N, Q - 1, N, Q);
  // position of element i of the lane's quad along the quad's axis
  if (halves) appendf(s, "#define GA_QP(i) (2u * ga_lo + ((i) & 1u) + ((i) >> 1) * %uu)\n", T / 2);
  else s += "#define GA_QP(i) (4u * ga_lo + (i))\n";
  appendf(s, "const %s ga_gy = ((%s)dim%u + %uu) / %uu;\n", N, N, yd, T - 1, T);
  // Tiles of one plane are handed out in bands of ga_ltx tile rows, walking
  // down a band's rows first: groups that run together then read runs that
  // are adjacent in the transposed operand's memory and write runs that are
  // adjacent in the output's (ga_ltx = 1: plain row-major order).
  appendf(s, "const %s ga_pl = ga_gx * ga_gy;\n", N);
  appendf(s, "%s ga_r = GID_0 / ga_pl;\n", N);
  appendf(s, "const %s ga_g = GID_0 - ga_r * ga_pl;\n", N);
  // Low half of ga_ltx = 0: diagonal order instead.  The plane is cut into
  // panels of ga_pw tile columns (high half of ga_ltx; 0: one panel), and tile
  // row r of a panel is walked along a diagonal, (bx, (r + bx) mod gy):
  // consecutive groups then differ in both coordinates, so neither the rows
  // they read nor the rows they write start a whole number of row pitches
  // apart (with a power-of-two pitch such rows fall on the same memory
  // channels), while a panel keeps the groups that run together within a
  // bounded span of the output's rows.
  appendf(s, "%s ga_bx, ga_by;\nconst %s ga_ord = ga_ltx & 0xffffu;\n", N, N);
  s += "if (ga_ord == 0u) {\n";
  appendf(s, "%s ga_pw = ga_ltx >> 16;\nif (ga_pw == 0u || ga_pw > ga_gx) ga_pw = ga_gx;\n", N);
  appendf(s, "const %s ga_pn = ga_g / (ga_pw * ga_gy);\n", N);
  appendf(s, "const %s ga_pl2 = ga_g - ga_pn * ga_pw * ga_gy;\n", N);
  appendf(s, "const %s ga_rest = ga_gx - ga_pn * ga_pw;\n", N);
  appendf(s, "const %s ga_w = ga_rest < ga_pw ? ga_rest : ga_pw;\n", N);
  appendf(s, "const %s ga_tr = ga_pl2 / ga_w;\n", N);
  appendf(s, "const %s ga_tc = ga_pl2 - ga_tr * ga_w;\n", N);
  s += "ga_bx = ga_pn * ga_pw + ga_tc;\nga_by = (ga_tr + ga_tc) % ga_gy;\n} else {\n";
  appendf(s, "const %s ga_band = ga_g / (ga_ord * ga_gx);\n", N);
  appendf(s, "const %s ga_in = ga_g - ga_band * ga_ord * ga_gx;\n", N);
  appendf(s, "const %s ga_left = ga_gy - ga_band * ga_ord;\n", N);
  appendf(s, "const %s ga_bh = ga_left < ga_ord ? ga_left : ga_ord;\n", N);
  s += "ga_bx = ga_in / ga_bh;\nga_by = ga_band * ga_ord + (ga_in - ga_bx * ga_bh);\n}\n";
  for (const ge_arg &a : ge->args)
    if (a.is_array()) appendf(s, "%s %s_o = 0;\n", I, a.name.c_str());
  if (nd >= 3) {
    appendf(s, "{ %s ga_c;\n", N);
    for (unsigned d = nd - 2; d-- > 0;) {
      if (d > 0) appendf(s, "ga_c = ga_r %% (%s)dim%u; ga_r = ga_r / (%s)dim%u;\n", N, d, N, d);
      else s += "ga_c = ga_r;\n";
      for (const ge_arg &a : ge->args)
        if (a.is_array())
          appendf(s, "%s_o += (%s)ga_c * (%s)%s_str_%u;\n", a.name.c_str(), I, I, a.name.c_str(), d);
    }
    s += "}\n";
  }
  appendf(s, "const %s ga_x0 = ga_bx * %uu;\nconst %s ga_y0 = ga_by * %uu;\n", N, T, N, T);
  // byte offset of (y, x) for array a
  auto off_yx = [&](const ge_arg &a, const char *y, const char *x) {
    std::string o;
    appendf(o, "(%s_o + (%s)(%s) * (%s)%s_str_%u + (%s)(%s) * (%s)%s_str_%u)", a.name.c_str(), I,
            y, I, a.name.c_str(), yd, I, x, I, a.name.c_str(), xd);
    return o;
  };
  bool any_tr = false, any_tw = false;
  for (size_t j = 0; j < ge->args.size(); j++) {
    if (!is_t(j)) continue;
    if (ge->args[j].reads()) any_tr = true;
    if (ge->args[j].writes()) any_tw = true;
  }
  // access h of the quad of array j (h < NH): along y at column `x` (phase 1
  // and 3), or along x at row `y` (the direct operands and results of phase 2)
  auto vec_ptr = [&](const ge_arg &a, bool along_y, unsigned h, const char *other) {
    char q[64];
    snprintf(q, sizeof(q), "%s + GA_QP(%uu)", along_y ? "ga_y0" : XB, h * VE);
    std::string pe;
    appendf(pe, "*(GLOBAL_MEM %s *)(%s_b + %s)", vec_t(a), a.name.c_str(),
            (along_y ? off_yx(a, q, other) : off_yx(a, other, q)).c_str());
    return pe;
  };
  // is access h of the quad, whose other coordinate is in range, in range itself?
  auto in_range = [&](bool along_y, unsigned h) {
    std::string c;
    appendf(c, "%s + GA_QP(%uu) < (%s)dim%u", along_y ? "ga_y0" : XB, h * VE, N, along_y ? yd : xd);
    if (loose)   // the whole quad (a window can start below 0: its first positions wrap to huge values)
      appendf(c, " && %s + GA_QP(%uu) + 3u < (%s)dim%u", along_y ? "ga_y0" : XB, h * VE, N, along_y ? yd : xd);
    return c;
  };
  // loose: the elements of a quad that the extent cuts, one by one
  // (`reg` names the lane's copy of the quad; element i of it is reg.e[i])
  auto emit_cut_quad = [&](const ge_arg &a, bool along_y, const char *other, const std::string &reg, bool store) {
    if (!loose) return;
    s += "else {\n";
    for (int i = 0; i < 4; i++) {
      char q[64];
      snprintf(q, sizeof(q), "%s + GA_QP(%du)", along_y ? "ga_y0" : XB, i);
      std::string pe;
      appendf(pe, "*(GLOBAL_MEM %s *)(%s_b + %s)", ctype(a.typecode), a.name.c_str(),
              (along_y ? off_yx(a, q, other) : off_yx(a, other, q)).c_str());
      appendf(s, "if (%s < (%s)dim%u) ", q, N, along_y ? yd : xd);
      if (store) appendf(s, "%s = %s.e[%d];\n", pe.c_str(), reg.c_str(), i);
      else appendf(s, "%s.e[%d] = %s;\n", reg.c_str(), i, pe.c_str());
    }
    s += "}\n";
  };
  // loads of the operands that phase 2 reads straight from memory
  auto emit_direct_loads = [&]() {
    for (size_t j = 0; j < ge->args.size(); j++) {
      const ge_arg &a = ge->args[j];
      if (a.is_array() && !is_t(j))
        appendf(s, "union { %s p[%u]; %s e[4]; } %s_u[4];\n", vec_t(a), NH, ctype(a.typecode), a.name.c_str());
    }
    s += "#pragma unroll\nfor (int ga_k = 0; ga_k < 4; ga_k++) {\n";
    appendf(s, "const %s ga_ly = ga_hi + %uu * (%s)ga_k;\n", N, Q, N);
    appendf(s, "if (ga_y0 + ga_ly < (%s)dim%u) {\n", N, yd);
    emit_row_window();
    for (size_t j = 0; j < ge->args.size(); j++) {
      const ge_arg &a = ge->args[j];
      if (!a.is_array() || is_t(j) || !a.reads()) continue;
      if (is_y(j)) s += "if (ga_k == 0) {\n";
      if (is_u(j)) {
        for (unsigned h = 0; h < NH; h++) {
          appendf(s, "if (%s) ", in_range(false, h).c_str());
          char dst[64];
          snprintf(dst, sizeof(dst), "%s_u[ga_k].p[%u]", a.name.c_str(), h);
          s += quad_load(j, dst, vec_ptr(a, false, h, "ga_y0 + ga_ly"));
          emit_cut_quad(a, false, "ga_y0 + ga_ly", a.name + "_u[ga_k]", false);
        }
      } else if (is_z(j)) {
        // (loose: some element of a cut quad may be in range, and the row's element 0 always exists)
        appendf(s, "if (%s) {\n%s_u[ga_k].e[0] = *(GLOBAL_MEM %s *)(%s_b + %s);\n", loose ? "true" : in_range(false, 0).c_str(),
                a.name.c_str(), ctype(a.typecode), a.name.c_str(), off_yx(a, "ga_y0 + ga_ly", "0").c_str());
        for (int i = 1; i < 4; i++)
          appendf(s, "%s_u[ga_k].e[%d] = %s_u[ga_k].e[0];\n", a.name.c_str(), i, a.name.c_str());
        s += "}\n";
      } else {
        for (int i = 0; i < 4; i++) {
          char xi[48];
          snprintf(xi, sizeof(xi), "%s + GA_QP(%du)", XB, i);
          appendf(s, "if (%s < (%s)dim%u) %s_u[ga_k].e[%d] = *(GLOBAL_MEM %s *)(%s_b + %s);\n", xi, N, xd,
                  a.name.c_str(), i, ctype(a.typecode), a.name.c_str(), off_yx(a, "ga_y0 + ga_ly", xi).c_str());
        }
      }
      // a lane's row 0 is in range whenever one of its later rows is
      if (is_y(j)) {
        s += "} else {\n";
        for (unsigned h = 0; h < NH; h++)
          appendf(s, "%s_u[ga_k].p[%u] = %s_u[0].p[%u];\n", a.name.c_str(), h, a.name.c_str(), h);
        s += "}\n";
      }
    }
    s += "}\n}\n";
  };
  // phase 1: transposed reads.  lane: y quad of ga_lo, x column ga_hi + Q k
  if (any_tr) {
    for (size_t j = 0; j < ge->args.size(); j++) {
      const ge_arg &a = ge->args[j];
      if (is_t(j) && a.reads())
        appendf(s, "union { %s p[%u]; %s e[4]; } %s_in[%u];\n", vec_t(a), NH, ctype(a.typecode),
                a.name.c_str(), NP);
    }
    appendf(s, "#pragma unroll\nfor (int ga_k = 0; ga_k < %u; ga_k++) {\n", NP);
    appendf(s, "const %s ga_lx = ga_hi + %uu * (%s)ga_k;\n", N, Q, N);
    appendf(s, "if (%s%s < (%s)dim%u) {\n", LXOK.c_str(), TX.c_str(), N, xd);
    for (size_t j = 0; j < ge->args.size(); j++) {
      const ge_arg &a = ge->args[j];
      if (!is_t(j) || !a.reads()) continue;
      for (unsigned h = 0; h < NH; h++) {
        appendf(s, "if (%s) ", in_range(true, h).c_str());
        char dst[64];
        snprintf(dst, sizeof(dst), "%s_in[ga_k].p[%u]", a.name.c_str(), h);
        s += quad_load(j, dst, vec_ptr(a, true, h, TX.c_str()));
        emit_cut_quad(a, true, TX.c_str(), a.name + "_in[ga_k]", false);
      }
    }
    s += "}\n}\n";
    // the direct operands of phase 2 are asked for here, behind the tile's
    // loads and before the barrier, so that their latency is not paid after it
    emit_direct_loads();
    appendf(s, "#pragma unroll\nfor (int ga_k = 0; ga_k < %u; ga_k++) {\n", NP);
    appendf(s, "const %s ga_lx = ga_hi + %uu * (%s)ga_k;\n", N, Q, N);
    appendf(s, "if (%s%s < (%s)dim%u) {\n", LXOK.c_str(), TX.c_str(), N, xd);
    for (size_t j = 0; j < ge->args.size(); j++) {
      const ge_arg &a = ge->args[j];
      if (!is_t(j) || !a.reads()) continue;
      appendf(s, "#pragma unroll\nfor (int ga_i = 0; ga_i < 4; ga_i++) "
                 "if (ga_y0 + GA_QP(ga_i) < (%s)dim%u) %s_t[GA_QP(ga_i) * %uu + ga_lx] = %s_in[ga_k].e[ga_i];\n",
              N, yd, a.name.c_str(), LP, a.name.c_str());
    }
    s += "}\n}\nlocal_barrier();\n";
  }
  // phase 2: the expression.  lane: x quad of ga_lo, y row ga_hi + Q k
  if (!any_tr) emit_direct_loads();
  s += "#pragma unroll\nfor (int ga_k = 0; ga_k < 4; ga_k++) {\n";
  appendf(s, "const %s ga_ly = ga_hi + %uu * (%s)ga_k;\n", N, Q, N);
  appendf(s, "if (ga_y0 + ga_ly < (%s)dim%u) {\n", N, yd);
  emit_row_window();
  appendf(s, "#pragma unroll\nfor (int ga_v = 0; ga_v < 4; ga_v++) if (%s + GA_QP(ga_v) < (%s)dim%u) {\n", XB, N, xd);
  for (size_t j = 0; j < ge->args.size(); j++) {
    const ge_arg &a = ge->args[j];
    if (!a.is_array()) continue;
    if (is_t(j)) emit_load(ge, s, a, a.name + "_t[ga_ly * " + TP + " + " + TCOL + "GA_QP(ga_v)]");
    else emit_load(ge, s, a, a.name + "_u[ga_k].e[ga_v]");
  }
  s += ge->expr;
  s += ";\n";
  for (size_t j = 0; j < ge->args.size(); j++) {
    const ge_arg &a = ge->args[j];
    if (!a.is_array()) continue;
    if (is_t(j)) emit_store(ge, s, a, a.name + "_t[ga_ly * " + TP + " + " + TCOL + "GA_QP(ga_v)]");
    else emit_store(ge, s, a, a.name + "_u[ga_k].e[ga_v]");
  }
  s += "}\n";
  for (size_t j = 0; j < ge->args.size(); j++) {
    const ge_arg &a = ge->args[j];
    if (!a.is_array() || is_t(j) || !a.writes()) continue;
    if (is_u(j)) {
      for (unsigned h = 0; h < NH; h++) {
        appendf(s, "if (%s) ", in_range(false, h).c_str());
        char val[64];
        snprintf(val, sizeof(val), "%s_u[ga_k].p[%u]", a.name.c_str(), h);
        s += quad_store(j, vec_ptr(a, false, h, "ga_y0 + ga_ly"), val);
        emit_cut_quad(a, false, "ga_y0 + ga_ly", a.name + "_u[ga_k]", true);
      }
    } else {
      for (int i = 0; i < 4; i++) {
        char xi[48];
        snprintf(xi, sizeof(xi), "%s + GA_QP(%du)", XB, i);
        appendf(s, "if (%s < (%s)dim%u) *(GLOBAL_MEM %s *)(%s_b + %s) = %s_u[ga_k].e[%d];\n", xi, N, xd,
                ctype(a.typecode), a.name.c_str(), off_yx(a, "ga_y0 + ga_ly", xi).c_str(), a.name.c_str(), i);
      }
    }
  }
  s += "}\n}\n";
  // phase 3: transposed writes, mirror of phase 1
  if (any_tw) {
    s += "local_barrier();\n#pragma unroll\nfor (int ga_k = 0; ga_k < 4; ga_k++) {\n";
    appendf(s, "const %s ga_lx = ga_hi + %uu * (%s)ga_k;\n", N, Q, N);
    appendf(s, "if (ga_x0 + ga_lx < (%s)dim%u) {\n", N, xd);
    for (size_t j = 0; j < ge->args.size(); j++) {
      const ge_arg &a = ge->args[j];
      if (!is_t(j) || !a.writes()) continue;
      appendf(s, "{ union { %s p[%u]; %s e[4]; } ga_o;\n#pragma unroll\nfor (int ga_i = 0; ga_i < 4; ga_i++) "
                 "ga_o.e[ga_i] = %s_t[GA_QP(ga_i) * %uu + ga_lx];\n",
              vec_t(a), NH, ctype(a.typecode), a.name.c_str(), LP);
      for (unsigned h = 0; h < NH; h++) {
        appendf(s, "if (%s) ", in_range(true, h).c_str());
        char val[32];
        snprintf(val, sizeof(val), "ga_o.p[%u]", h);
        s += quad_store(j, vec_ptr(a, true, h, "ga_x0 + ga_lx"), val);
      }
      s += "}\n";
    }
    s += "}\n}\n";
  }
  s += "#undef GA_QP\n}\n";
  return s;
}

int build_kernel(GpuElemwise *ge, GpuKernel *k, const std::string &src,
                 const std::vector<int> &ktypes) {
  const char *strs[1] = {src.c_str()};
  size_t lens[1] = {src.size()};
  return GpuKernel_init(k, ge->ctx, 1, strs, lens, "elem", (unsigned)ktypes.size(), ktypes.data(),
                        ge->kflags, nullptr);
}

// ---- flat path ------------------------------------------------------------------

// reference check_contig (:547-576): returns -1 when shapes differ.
int check_flat(GpuElemwise *ge, void **args, size_t *n_out, bool *flat) {
  const GpuArray *first = nullptr;
  size_t n = 1;
  bool c_all = true, f_all = true;
  for (size_t i = 0; i < ge->args.size(); i++) {
    if (!ge->args[i].is_array()) continue;
    const GpuArray *v = (const GpuArray *)args[i];
    if (first == nullptr) {
      first = v;
      for (unsigned j = 0; j < v->nd; j++) n *= v->dimensions[j];
    } else {
      if (v->nd != first->nd) return -1;
      for (unsigned j = 0; j < v->nd; j++)
        if (v->dimensions[j] != first->dimensions[j]) return -1;
    }
    c_all = c_all && GpuArray_IS_C_CONTIGUOUS(v);
    f_all = f_all && GpuArray_IS_F_CONTIGUOUS(v);
  }
  *flat = c_all || f_all;
  *n_out = n;
  return GA_NO_ERROR;
}

// Operands of a flat call that are addressed through the coordinates of the
// flat index (see gen_flat): which arrays, the iteration space, the
// multipliers that stand in for the divisions, byte strides per array.
struct flat_periodic {
  unsigned pmask = 0, pnd = 2;
  unsigned pvmask = 0;   // of pmask: operands a chunk of which is one aligned load (when there is no head)
  unsigned pumask = 0;   // of pmask: a chunk inside one row is one load on four-byte boundaries
  unsigned d1 = 1, d2 = 1, k1 = 0, k2 = 0;
  uint64_t m1 = 0, m2 = 0;
  std::vector<std::array<ssize_t, 3>> ps;   // indexed by array
};

// Launch the flat kernel over n elements; offs[k] is the byte offset of
// array k's first element in its buffer.
int call_flat(GpuElemwise *ge, void **args, size_t n, const size_t *offs,
              const flat_periodic *pi = nullptr) {
  const ga_tuning *tn = ga_hip_tuning(ge->ctx);
  unsigned l = 0;
  int err;
  unsigned int vec_ok = (ge->vec > 1 || ge->unroll > 1) ? 1u : 0u, head = ~0u;
  std::vector<unsigned> heads;
  const unsigned pmask = pi ? pi->pmask : 0u;
  for (size_t i = 0; i < ge->args.size(); i++) {
    if (!ge->args[i].is_array()) continue;
    GpuArray *a = (GpuArray *)args[i];
    if ((pmask >> heads.size()) & 1u) {   // not walked in chunks: no say in the alignment
      heads.push_back(~0u);
      l++;
      continue;
    }
    // Elements from this array's start to its next chunk boundary.  The
    // first written array (else the first array) sets the head of the
    // vector path; an array with another count is moved element by element.
    const size_t elsz = gpuarray_get_elsize(a->typecode), chunk = elsz * ge->vec;
    const size_t mis = ((uintptr_t)a->data->devptr + offs[l++]) % chunk;
    if (mis % elsz != 0) vec_ok = 0;
    heads.push_back((unsigned)((chunk - mis) % chunk / elsz));
    if (head == ~0u && ge->args[i].writes()) head = heads.back();
  }
  if (head == ~0u) head = heads.empty() ? 0 : heads[0];
  if (n < (size_t)head + ge->vec || heads.size() > 24) vec_ok = 0;
  unsigned int vec_arg = vec_ok ? 1u + head : 0u;
  for (size_t q = 0; vec_ok && q < heads.size(); q++)
    if (heads[q] != head && heads[q] != ~0u) vec_arg |= 1u << (8 + q);
  if (!TUNE(tn, ELEMWISE_MIXED_ALIGN, 1) && (vec_arg >> 8)) vec_arg = 0;
  if (vec_arg == 0) vec_ok = 0;

  // Grid: one lane per chunk (or per element) up to a fixed number of groups
  // per compute unit; beyond that the lanes stride over the range.
  // Measured on MI355X at 2^28 fp32 elements (3 GiB of traffic): one chunk per
  // lane over the whole range sustains 6.5 TB/s, a grid capped at 8..64 groups
  // per compute unit that strides over the range 4.2..5.2 TB/s.  So the cap
  // only matters far beyond that size.  Fewer groups resident on a compute
  // unit (the eight that fit cut down by asking for local memory nobody uses)
  // are slower as well: 8 groups 495 us, 6 507, 5 589, 4 592, 3 572, 2 635.
  const size_t ncu = ga_hip_numprocs(ge->ctx);
  const size_t per_cu = TUNE(tn, ELEMWISE_GROUPS_PER_CU, 2048);
  size_t cap = ncu * (per_cu ? per_cu : 2048);
  size_t units = vec_ok ? (n - head) / ge->vec + 1 : n;
  // A compute unit holds eight groups of this kernel at a time.  A grid of
  // one to two such fills runs its second, partial fill at a fraction of the
  // chip: two adjacent chunks per lane (four up to four fills) make it a
  // single fill.  Measured on MI355X, c = a*b + 0.5f on floats, kernel time
  // with 1 / 2 / 4 chunks per lane: 3 * 2^20 elements 8.3 / 7.3 / 8.5 us, 2^22
  // 10.0 / 8.9 / 9.9, 3 * 2^21 13.7 / 13.7 / 12.5, 2^23 17.3 / 18.0 / 16.5;
  // below (2^21: 5.8 / 6.4 / 7.8) and above (3 * 2^22: 25.0 / 26.3 / 26.9,
  // 2^24 32.6 / 34.1 / 35.3, 2^28 496 / 509 / 531) one chunk per lane is best.
  //
  // Arrays of narrower elements than the widest move in chunks of fewer than
  // 16 bytes.  Where one whole side of the kernel is narrow, two chunks per
  // lane, 256 chunks apart, are faster at every size beyond one fill (kernel
  // time for 2^27 elements, one chunk per lane / two / four: bytes to floats
  // 119.9 / 100.4 / 117.9 us, two byte arrays to floats 163.9 / 127.6 / 138.4,
  // floats to bytes 112.6 / 102.1 / 106.8, floats to halves 127.5 / 120.4 /
  // 130.2, doubles to floats 252.0 / 241.4 / 258.4, a > b to a byte 187.5 /
  // 181.6 / 198.0); where a wide array is read and a wide one written they
  // are slower (float + half to float 200.5 / 212.9, halves to floats 122.0 /
  // 124.9, two floats to a half 203.0 / 206.5).
  unsigned tiled_u = 0;
  if (vec_ok && !ge->flat_forced && !ge->tile && pi == nullptr) {
    // whole chunks only: the extra unit that covers head and tail does not add a group's worth of work
    const size_t g1 = (units - 1 + GE_LANES - 1) / GE_LANES, fill = ncu * 8;
    if (g1 > fill && g1 <= 2 * fill) tiled_u = 2;
    else if (g1 > 2 * fill && g1 <= 4 * fill) tiled_u = ge->narrow_side ? 2 : 4;
    else if (g1 > 4 * fill && ge->narrow_side) tiled_u = 2;
  }
  GpuKernel *k = &ge->k_flat;
  if (tiled_u) {
    auto it = ge->k_flat_tiled.find(tiled_u);
    if (it == ge->k_flat_tiled.end()) {
      std::vector<int> ktypes;
      std::string src = gen_flat(ge, ktypes, tiled_u, 1);
      GpuKernel nk = {nullptr, nullptr};
      if ((err = build_kernel(ge, &nk, src, ktypes)) != GA_NO_ERROR) return err;
      it = ge->k_flat_tiled.emplace(tiled_u, nk).first;
    }
    k = &it->second;
  }
  if (pi != nullptr) {
    const unsigned pv = (vec_ok && head == 0) ? pi->pvmask : 0u;
    const unsigned pu = vec_ok ? pi->pumask & ~pv : 0u;
    const std::array<uint32_t, 4> key = {{pi->pmask, pi->pnd, pv, pu}};
    auto it = ge->k_flat_periodic.find(key);
    if (it == ge->k_flat_periodic.end()) {
      std::vector<int> ktypes;
      std::string src = gen_flat(ge, ktypes, 0, -1, pi->pmask, pi->pnd, pv, pu);
      GpuKernel nk = {nullptr, nullptr};
      if ((err = build_kernel(ge, &nk, src, ktypes)) != GA_NO_ERROR) return err;
      it = ge->k_flat_periodic.emplace(key, nk).first;
    }
    k = &it->second;
  }
  const bool tile = tiled_u ? true : ge->tile;
  const unsigned unroll = tiled_u ? tiled_u : ge->unroll;

  if (ge->args.size() > 255)
    return ga_err_set(ge->ctx->err, GA_UNSUPPORTED_ERROR, "More than 255 arguments");
  ew_launch &L = ge->pending;
  L.slots.clear();
  l = 0;
  L.value(n);
  for (size_t i = 0; i < ge->args.size(); i++) {
    if (ge->args[i].is_array()) {
      L.array(i);
      L.value(offs[l++]);
    } else {
      L.scalar(i);
    }
  }
  L.value(vec_arg);
  if (pi != nullptr) {
    L.value(pi->d1);
    L.value(pi->d2);
    L.value(pi->m1);
    L.value(pi->k1);
    L.value(pi->m2);
    L.value(pi->k2);
    for (size_t q = 0; q < pi->ps.size(); q++)
      if ((pi->pmask >> q) & 1u)
        for (int j = 0; j < 3; j++) L.value(pi->ps[q][j]);
  }
  size_t per_group = GE_LANES * (size_t)((vec_ok && tile) ? unroll : 1);
  size_t want = (units + per_group - 1) / per_group;
  L.k = k;
  L.gs = want < 1 ? 1 : (want > cap ? cap : want);
  L.ls = GE_LANES;
  L.valid = true;
  return GA_NO_ERROR;
}

// ---- general path ---------------------------------------------------------------

// Reference check_basic (:272-383) up to, not including, the collapse:
// fills ge->dims / ge->strs with the padded, broadcast-adjusted view of
// every array and returns nd and n.
int check_general(GpuElemwise *ge, void **args, int flags, size_t *n_out, unsigned *nd_out) {
  gpucontext *ctx = ge->ctx;
  const GpuArray *out = nullptr;
  unsigned nd = 0, seen = 0;
  for (size_t i = 0; i < ge->args.size(); i++) {
    if (!ge->args[i].is_array()) continue;
    const GpuArray *v = (const GpuArray *)args[i];
    if (seen == 0) {
      nd = v->nd;
    } else if (v->nd != nd) {
      if (!(flags & GE_PADSHAPE))
        return ga_err_fmt(ctx->err, GA_VALUE_ERROR, "Arg %zu has differing nd = %u", i, v->nd);
      nd = std::max(nd, v->nd);
    }
    seen++;
    if (out == nullptr && ge->args[i].writes()) out = v;
  }
  if (out == nullptr) return ga_err_set(ctx->err, GA_VALUE_ERROR, "No output arrays");
  if (out->nd != nd)
    // the output fixes the iteration space, so it cannot be the padded one
    return ga_err_fmt(ctx->err, GA_VALUE_ERROR,
                      "Output has nd = %u but an input has nd = %u: outputs do not broadcast",
                      out->nd, nd);

  ge->dims.assign(out->dimensions, out->dimensions + nd);
  ge->strs.assign(ge->narray, std::vector<ssize_t>(nd ? nd : 1, 0));
  unsigned p = 0;
  for (size_t i = 0; i < ge->args.size(); i++) {
    if (!ge->args[i].is_array()) continue;
    const GpuArray *v = (const GpuArray *)args[i];
    const unsigned pad = nd - v->nd;
    for (unsigned j = 0; j < nd; j++) {
      const size_t vd = j < pad ? 1 : v->dimensions[j - pad];
      if (vd != ge->dims[j]) {
        if (!(flags & GE_BROADCAST) || ge->args[i].writes() || vd != 1)
          return ga_err_fmt(ctx->err, GA_VALUE_ERROR,
                            "Mismatched dimension %u for input %zu (expected %zu got %zu)", j, i,
                            ge->dims[j], vd);
      }
      // a dim of extent 1 never moves: stride 0 whether or not it broadcasts
      ge->strs[p][j] = (j < pad || vd == 1) ? 0 : v->strides[j - pad];
    }
    p++;
  }
  size_t n = 1;
  for (unsigned j = 0; j < nd; j++) n *= ge->dims[j];
  *n_out = n;
  *nd_out = nd;
  return GA_NO_ERROR;
}

inline size_t sabs(ssize_t v) { return v < 0 ? (size_t)(-v) : (size_t)v; }

// One call of the strided kernels: the arrays' layout brought into the order
// the kernels walk it, the choice between the scalar, four-per-lane and
// transposed-tile forms, the launch.
class strided_call {
 public:
  strided_call(GpuElemwise *ge_, void **args_, size_t n_, unsigned nd_)
      : ge(ge_), ctx(ge_->ctx), tn(ga_hip_tuning(ge_->ctx)), args(args_), n(n_), nd(nd_),
        na(ge_->narray), dims(ge_->dims), strs(ge_->strs) {}

  int run() {
    describe_arrays();
    normalise_layout();
    if (is_one_dense_run()) return call_flat(ge, args, n, offs.data());
    {
      int err = GA_NO_ERROR;
      if (narrow_plane_in_registers(err)) return err;
    }
    {
      int err = GA_NO_ERROR;
      if (tiles_of_short_records(err)) return err;
    }
    find_transposed_operands();
    choose_offset_width();
    choose_vector_access();
    {
      flat_periodic pi;
      if (dense_with_broadcast_operands(pi)) return call_flat(ge, args, n, offs.data(), &pi);
    }
    int err;
    if ((err = choose_grid()) != GA_NO_ERROR) return err;
    if ((err = get_kernel()) != GA_NO_ERROR) return err;
    return launch();
  }

 private:
  GpuElemwise *ge;
  gpucontext *ctx;
  const ga_tuning *tn;
  void **args;
  const size_t n;
  unsigned nd;
  const unsigned na;
  std::vector<size_t> &dims;
  std::vector<std::vector<ssize_t>> &strs;
  std::vector<size_t> elsz, offs;   // per array: element size, byte offset of element 0
  int outk = -1;                    // the (first) output among the arrays
  unsigned tmask = 0;               // arrays read or written through transposed tiles
  bool idx64 = false;               // 64-bit offsets in the kernel
  bool vec4 = false;                // four elements per lane
  unsigned umask = 0;               // vec4: arrays with 16-byte access along x
  unsigned ntmask = 0;              // vec4: arrays touched once, streamed past the caches
  unsigned zmask = 0;               // vec4: arrays whose stride along x (bits 16..: along y) is zero
  size_t gx = 0, groups = 0;
  unsigned ltx = 0, tile = 64, quads = 4;
  unsigned vq = 4;                  // vec4: elements a lane moves at a time (2 for 8-byte types, plain variant)
  unsigned skew = 0;                // transposed tiles: 1 + the array whose rows the tiles' windows follow
  bool loose = false;               // transposed tiles of four-byte elements on any bases, pitches and extents
  GpuKernel *kernel = nullptr;

  void describe_arrays() {
    // which array is the (first) output, and per-array element sizes / offsets
    elsz.assign(na, 0);
    offs.assign(na, 0);
    {
      unsigned k = 0;
      for (size_t i = 0; i < ge->args.size(); i++) {
        if (!ge->args[i].is_array()) continue;
        const GpuArray *v = (const GpuArray *)args[i];
        elsz[k] = gpuarray_get_elsize(v->typecode);
        offs[k] = v->offset;
        if (outk < 0 && ge->args[i].writes()) outk = (int)k;
        k++;
      }
    }
  }

  void normalise_layout() {
    if (nd == 0) {  // 0-d arrays: one element
      nd = 1;
      dims.assign(1, 1);
      for (auto &s : strs) s.assign(1, 0);
    }

    // Sort dims so the output's stride shrinks towards the last dim (stable),
    // then drop size-1 dims and fuse runs.
    {
      std::vector<unsigned> order(nd);
      for (unsigned j = 0; j < nd; j++) order[j] = j;
      std::stable_sort(order.begin(), order.end(), [&](unsigned a, unsigned b) {
        return sabs(strs[outk][a]) > sabs(strs[outk][b]);
      });
      std::vector<size_t> d2(nd);
      for (unsigned j = 0; j < nd; j++) d2[j] = dims[order[j]];
      dims = d2;
      for (unsigned k = 0; k < na; k++) {
        std::vector<ssize_t> s2(nd);
        for (unsigned j = 0; j < nd; j++) s2[j] = strs[k][order[j]];
        strs[k] = s2;
      }
    }
    ge->strp.resize(na);
    for (unsigned k = 0; k < na; k++) ge->strp[k] = strs[k].data();
    gpuarray_elemwise_collapse(na, &nd, dims.data(), ge->strp.data());
  }

  // A plane with one short extent F (2 to 15) of elements of one to eight bytes
  // (the figures are for four-byte ones) where some
  // array has the short dim innermost and another the long one - (N, F) taken as
  // its transpose, or written as one: too narrow for tiles through the LDS, which
  // F of 64 or 128 columns fill.  A lane takes four positions along the long dim
  // and all F of the short one in registers (gen_narrow_block).  out = in.T of
  // 256 MiB of floats, (N, F) -> (F, N), before / now in % of 8 TB/s: F = 2
  // 54 / 73, 3 47 / 67, 4 37 / 70, 5 30 / 66, 7 25 / 67, 8 22 / 70, 11 17 / 63,
  // 12 19 / 63, 13 30 / 63, 15 33 / 61; (F, N) -> (N, F): 2 29 / 81, 3 29 / 78,
  // 5 37 / 74, 7 34 / 76, 9 32 / 74, 11 39 / 69, 13 32 / 69, 15 34 / 58.  16 and
  // more fill a quarter of a small tile's rows and stay with the tiles (73 and
  // 77 % against 62 and 77).  From 4096 positions on: below, either kernel takes
  // the 4 us of a launch.  With three dims the first counts planes, each cut into
  // groups of its own - images between channels last and channels first, (B, H,
  // W, C) <-> (B, C, H, W) with H and W fused: (16, 1024, 1024, 3) 75 -> 66 us
  // and back 175 -> 63, (256, 56, 56, 8) 28.6 -> 8.2 - from planes of 256
  // positions on (shorter ones leave most of a group idle: (65536, 4, 4, 3) 4.8
  // us with the strided kernel, 17 this way).
  bool narrow_plane_in_registers(int &err) {
    const unsigned long fmax = TUNE(tn, ELEMWISE_NARROW, 15);
    if (fmax == 0 || (nd != 2 && nd != 3) || na > 31) return false;
    const unsigned sd = dims[nd - 2] <= dims[nd - 1] ? nd - 2 : nd - 1, ld = sd == nd - 1 ? nd - 2 : nd - 1;
    const size_t F = dims[sd], L = dims[ld];
    // Wider ones whole through the LDS (gen_narrow_staged), where the tiles are
    // filled badly.  out = in.T of 256 MiB of floats, tiles / this kernel in % of
    // 8 TB/s: (N, F) -> (F, N) F = 17 37 / 58, 19 39 / 59, 22 45 / 60, 25 51 / 59,
    // 27 51 / 58, 31 56 / 59, then level (34 57 / 58) and behind (40 64 / 56, 56
    // 71 / 47: the result's rows leave a group in pieces of 1 KiB); (F, N) -> (N,
    // F), F no multiple of four: 17 41 / 71, 23 47 / 73, 29 43 / 67, 35 50 / 65, 41
    // 53 / 57, 50 37 / 59, 57 36 / 43, 63 41 / 46.
    const unsigned long smax = sd == nd - 1 ? TUNE(tn, ELEMWISE_NARROW_STAGED, 64) : TUNE(tn, ELEMWISE_NARROW_STAGED_WIDE, 31);
    const bool wide = F > 16;
    if (F < 2 || F > (wide ? smax : fmax) || F > 64 || n / F < TUNE(tn, ELEMWISE_NARROW_MIN, 4096)) return false;
    if (L < TUNE(tn, ELEMWISE_NARROW_MIN_PLANE, 256)) return false;
    // a short extent of whole quads innermost in the result: four elements per
    // lane of the strided kernel are a chunk of the result and coalesced single
    // elements of the operands (out = in.T of (4, N) 78 against 75 % of peak, of
    // (8, N) 79 against 74)
    // positions per lane: the elements of a chunk of the smallest type
    size_t es = 16;
    bool same = true;
    for (unsigned k = 0; k < na; k++) {
      if (elsz[k] != 1 && elsz[k] != 2 && elsz[k] != 4 && elsz[k] != 8) return false;
      es = std::min(es, elsz[k]);
      same = same && elsz[k] == elsz[0];
    }
    const size_t E = 16 / es;
    if (wide && !(same && es == 4)) return false;
    // (two-byte elements: (8, N) -> (N, 8) of halves 54 % there, 73 % here)
    if (sd == nd - 1 && F % E == 0 && same && es >= 4 && TUNE(tn, ELEMWISE_NARROW_QUADS, 0) == 0) return false;
    size_t held = 0;   // 16-byte chunks in a lane's registers
    unsigned bmask = 0, cmask = 0, umask = 0, smask = 0, nt = 0, zmask_l = 0;
    bool crossed = false;   // some array runs along the long dim and moves along the short one
    const unsigned long stage = TUNE(tn, ELEMWISE_NARROW_LDS, 2);   // 1: staged when read, 2: when written
    size_t lds = 0;
    {
      unsigned k = 0;
      for (size_t i = 0; i < ge->args.size(); i++) {
        if (!ge->args[i].is_array()) continue;
        const size_t ek = elsz[k], cprk = E * ek / 16;
        if (offs[k] % ek != 0) return false;
        const bool base16 = offs[k] % 16 == 0 && (nd == 2 || strs[k][0] % 16 == 0);
        if (nd == 3 && strs[k][0] % (ssize_t)ek != 0) return false;
        if (base16 && strs[k][sd] == (ssize_t)ek && strs[k][ld] == (ssize_t)(ek * F)) {
          bmask |= 1u << k;
          held += F * cprk;
          const bool want = (ge->args[i].reads() ? (stage & 1) : 0) || (ge->args[i].writes() ? (stage & 2) : 0);
          if (wide) {
            lds += 260 * 4 * (F | 1);
            if (lds > 72 * 1024) return false;
          } else if (want && lds + 4096 * F * cprk <= 64 * 1024) {
            smask |= 1u << k;
            lds += 4096 * F * cprk;
          }
        } else if (strs[k][ld] == (ssize_t)ek && strs[k][sd] % (ssize_t)ek == 0) {
          const bool whole = base16 && strs[k][sd] % 16 == 0;
          // a lane's positions of a row of wider elements are several chunks: written, they would
          // reach memory as pieces of lines (bytes with the short dim innermost to floats in planes
          // 157 us that way, 34 with single bytes fetched and whole chunks stored by the strided kernel)
          if (cprk > 1 && ge->args[i].writes()) return false;
          cmask |= 1u << k;
          held += F * cprk;
          if (strs[k][sd] != 0) crossed = true;
          if (!whole) umask |= 1u << k;
        } else if (strs[k][ld] == 0 && !ge->args[i].writes()) {
          zmask_l |= 1u << k;
        }
        k++;
      }
    }
    if (bmask == 0 || !crossed || (!wide && held > TUNE(tn, ELEMWISE_NARROW_CHUNKS, 32))) return false;
    // arrays that take part once, whole, are streamed (the rest, broadcast or
    // overlapping, stays cacheable)
    {
      const unsigned long m = TUNE(tn, ELEMWISE_NARROW_NT, 3);
      if (m & 1) nt |= cmask;
      if (m & 2) nt |= wide ? bmask : smask;
      if (m & 4) nt |= bmask;
      for (unsigned k = 0; k < na; k++)
        if (strs[k][sd] == 0) nt &= ~(1u << k);
    }
    choose_offset_width();
    gx = wide ? (L + 255) / 256 : (L + 256 * E - 1) / (256 * E);
    groups = gx * (nd == 3 ? dims[0] : 1);
    ltx = 0;
    if (groups > 0x7fffffffull || gx > 0x7fffffffull) return false;
    char key[64];
    snprintf(key, sizeof(key), "%s%u:%zu:%u:%d:%x:%x:%x:%x:%x:%zu:%x", wide ? "w" : "n", nd, F, sd, idx64 ? 1 : 0, bmask, cmask, nt, umask,
             smask, es, wide ? 0u : zmask_l);
    auto it = ge->k_strided.find(key);
    if (it != ge->k_strided.end()) {
      kernel = &it->second;
    } else {
      std::vector<int> ktypes;
      std::string src = wide ? gen_narrow_staged(ge, idx64, (unsigned)F, sd, bmask, cmask, nt, ktypes, umask, nd)
                             : gen_narrow_block(ge, idx64, (unsigned)F, sd, bmask, cmask, nt, ktypes, umask, smask, nd, (unsigned)es, zmask_l);
      GpuKernel nk = {nullptr, nullptr};
      err = build_kernel(ge, &nk, src, ktypes);
      if (err != GA_NO_ERROR) return true;
      kernel = &ge->k_strided.emplace(key, nk).first->second;
    }
    err = launch();
    return true;
  }

  // Matrices of short records taken as their transposes (gen_record_tiles): three
  // dims (four with planes), the inner one of 2 to 64 elements (up to 256 bytes;
  // all arrays of one element size) with unit stride; the result's records follow one another along X, a read-only
  // operand's along Y.  Neither counts as a transposed operand for the tiles (both
  // have their smallest stride on the inner dim), and a lane of the strided
  // kernels walks the short inner dim.
  // (side of a tile in records; records of 8 floats 69 / 76 % of peak with 32 / 16, of 32 69 / 75 % with 16 / 8,
  // of 2 67 / 74 / 59 % with 64 / 32 / 16)
  // (by the record's bytes; records of up to 6 bytes get runs of 128 bytes and more from a side of 64)
  static unsigned record_tile_side(size_t fb) { return fb <= 6 ? 64 : fb <= 28 ? 32 : fb <= 124 ? 16 : 8; }
  bool tiles_of_short_records(int &err) {
    const unsigned long fmax = TUNE(tn, ELEMWISE_RECORDS, 64);
    if (fmax == 0 || (nd != 3 && nd != 4) || na > 31) return false;
    const size_t F = dims[nd - 1], X = dims[nd - 2], Y = dims[nd - 3];
    if (F < 2 || F > fmax || F > 64 || X < 32 || Y < 32 || X > 0x7fffffffull || Y > 0x7fffffffull ||
        n < TUNE(tn, ELEMWISE_RECORDS_MIN, 65536))
      return false;
    unsigned tm = 0, pm = 0;
    const size_t es = elsz[0];
    if ((es != 1 && es != 2 && es != 4 && es != 8) || F * es > 256) return false;
    {
      unsigned k = 0;
      for (size_t i = 0; i < ge->args.size(); i++) {
        if (!ge->args[i].is_array()) continue;
        if (elsz[k] != es || offs[k] % es != 0) return false;
        for (unsigned j = 0; j < nd; j++)
          if (strs[k][j] % (ssize_t)es != 0) return false;
        const bool unit = strs[k][nd - 1] == (ssize_t)es;
        if (unit && strs[k][nd - 2] == (ssize_t)(es * F)) pm |= 1u << k;
        else if (unit && strs[k][nd - 3] == (ssize_t)(es * F) && !ge->args[i].writes()) tm |= 1u << k;
        else if (ge->args[i].writes()) return false;
        k++;
      }
    }
    if (tm == 0 || !((pm >> outk) & 1u)) return false;
    unsigned T = record_tile_side(F * es);
    {
      const unsigned long ft = TUNE(tn, ELEMWISE_RECORDS_TILE, 0);
      if (ft == 8 || ft == 16 || ft == 32 || ft == 64) T = (unsigned)ft;
    }
    const size_t V = 16 / es, B = 64 / es;
    while (((size_t)T * F) % V != 0 && T < 64) T *= 2;   // a run of whole chunks
    if (((size_t)T * F) % V != 0) return false;
    // Windows moved onto the result's 64-byte blocks where its rows, or the tiles' pieces of them,
    // do not start on such blocks by themselves: (4729, 4729, 3) floats transposed (1, 0, 2) 41 ->
    // 54 % of peak, (3663, 3663, 5) 47 -> 59 %, (2590, 2590, 10) 54 -> 61 % ((4736, 4736, 3), whole
    // lines, runs at 73 %); moved windows on rows of whole blocks cost 6 to 10 points.
    if (X * F + 64 + (size_t)64 * F >= 0x7fffffffull) return false;
    bool skewed = offs[outk] % 64 != 0 || ((size_t)T * F * es) % 64 != 0;
    for (unsigned j = 0; j + 2 < nd; j++) skewed = skewed || strs[outk][j] % 64 != 0;
    {
      const unsigned long sk = TUNE(tn, ELEMWISE_RECORDS_SKEW, 1);
      // (records of 33 and 50 floats on such rows: 59 and 60 % rectangular, 59 and 58 % moved)
      skewed = sk == 2 || (sk == 1 && skewed && F * es <= 124);
    }
    // (the windows of neighbouring tiles meet only if a tile's piece of a row is whole blocks)
    while (skewed && ((size_t)T * F) % B != 0 && T < 64) T *= 2;
    if (skewed && ((size_t)T * F) % B != 0) skewed = false;
    const unsigned extra = skewed ? (unsigned)((B - 1 + F - 1) / F + 1) : 0;
    size_t lds = 0;
    for (unsigned k = 0; k < na; k++)
      if ((tm >> k) & 1u) lds += (size_t)(T + extra) * (T * F + V) * es;
    if (lds > 80 * 1024) return false;
    choose_offset_width();
    // Transposed arrays whose runs are no whole 128-byte lines: the lines in which a tile's runs
    // begin and end belong to the next tile along Y too, and streamed they were fetched again
    // ((4729, 4729, 3) floats read 1.58 times the array).  They stay cacheable: records of 3 floats
    // on such rows 54 -> 66 % of peak, of 5 59 -> 66, of 10 61 -> 69, of 25 63 -> 65; bytes in
    // records of 2 30 -> 40 %.  Numbering the tiles along Y first, consecutive numbers on one die,
    // measured 3 to 6 points behind that on floats and 1 to 4 ahead on bytes: a knob, off.
    bool lines = ((size_t)T * F * es) % 128 == 0;
    for (unsigned k = 0; k < na && lines; k++)
      if ((tm >> k) & 1u) lines = offs[k] % 128 == 0 && strs[k][nd - 2] % 128 == 0 && (nd == 3 || strs[k][0] % 128 == 0);
    const unsigned long ntm = TUNE(tn, ELEMWISE_RECORDS_NT, 3);
    const unsigned nt = ((ntm & 1) ? pm : 0u) | (((ntm & 2) && (lines || (ntm & 4))) ? tm : 0u);
    const unsigned long ym = TUNE(tn, ELEMWISE_RECORDS_YMAJOR, 0);
    const bool ymajor = ym == 2 || (ym == 1 && !lines);
    gx = (X * F + (skewed ? B - 1 : 0) + (size_t)T * F - 1) / ((size_t)T * F);
    const size_t gy = (Y + T - 1) / T;
    ltx = (unsigned)gy;
    groups = gx * gy * (nd == 4 ? dims[0] : 1);
    if (groups > 0x7fffffffull) return false;
    char key[64];
    snprintf(key, sizeof(key), "r%u:%zu:%u:%d:%x:%x:%x:%d:%zu:%d", nd, F, T, idx64 ? 1 : 0, tm, pm, nt, skewed ? outk : -1, es,
             ymajor ? 1 : 0);
    auto it = ge->k_strided.find(key);
    if (it != ge->k_strided.end()) {
      kernel = &it->second;
    } else {
      std::vector<int> ktypes;
      std::string src = gen_record_tiles(ge, nd, idx64, (unsigned)F, T, tm, pm, nt, ktypes, skewed ? outk : -1, (unsigned)es, ymajor);
      GpuKernel nk = {nullptr, nullptr};
      err = build_kernel(ge, &nk, src, ktypes);
      if (err != GA_NO_ERROR) return true;
      kernel = &ge->k_strided.emplace(key, nk).first->second;
    }
    err = launch();
    return true;
  }

  bool is_one_dense_run() const {
    // One evenly strided run with every array stepping by its own element
    // size is the flat case again (all-Fortran inputs, sliced-then-dense...).
    if (nd != 1) return false;
    bool unit = true;
    for (unsigned k = 0; k < na && unit; k++)
      unit = dims[0] == 1 || strs[k][0] == (ssize_t)elsz[k];
    return unit;
  }

  // Dense arrays (one run in C order over the collapsed dims) combined with
  // read-only operands that are broadcast along at least one dim: the flat
  // kernel walks the dense arrays in 16-byte chunks whatever the extents are
  // and reads the broadcast operands through the coordinates of the flat
  // index.  Taken when the four-per-lane strided kernel cannot be (an inner
  // extent that is not a multiple of 4, rows off a 16-byte boundary), where
  // the other choice is one element per lane and one row per lane group.
  // Measured on MI355X, kernel time, floats: (2^24, 3) + (1, 3) 161 -> 60 us,
  // (65536, 1001) + (1, 1001) 125 -> 88, (2^22, 17) + (1, 17) 307 -> 90,
  // (2^22, 10) * (2^22, 1) 159 -> 51, (2^20, 3, 5) + (1, 3, 1) 55 -> 21.
  // Where the four-per-lane kernel can be taken it stays, except when every
  // broadcast operand is constant along the inner dim and a dense array is
  // read: (8192, 8192) * (8192, 1) 86 -> 80 us, (4096, 10, 4096) * (1, 10, 1)
  // 220 -> 201, (64, 3, 512, 512) - (1, 3, 1, 1) 65 -> 61; an operand with
  // unit stride along an inner extent of whole chunks is fetched a chunk per
  // load ((8192, 8192) + (1, 8192) 89 -> 81 us).  With an operand that varies
  // along the inner dim and cannot be fetched that way the strided kernel is
  // the faster one (87 against 92 us, channels last 79 against 94), and so it
  // is when nothing dense is read (outer product 49 against 79).
  bool dense_with_broadcast_operands(flat_periodic &pi) const {
    const unsigned long mode = TUNE(tn, ELEMWISE_PERIODIC, 1);
    if (mode == 0 || tmask != 0) return false;
    bool inner_constant = true, dense_read = false;
    const size_t V = ge->vec;
    if ((nd != 2 && nd != 3) || n >= ((size_t)1 << 31) || na > 24) return false;
    pi.ps.assign(na, std::array<ssize_t, 3>{{0, 0, 0}});
    unsigned l = 0;
    for (size_t i = 0; i < ge->args.size(); i++) {
      if (!ge->args[i].is_array()) continue;
      const unsigned k = l++;
      bool dense = true;
      size_t run = elsz[k];
      for (unsigned j = nd; j-- > 0;) {
        if (strs[k][j] != (ssize_t)run) dense = false;
        run *= dims[j];
      }
      if (dense) {
        dense_read = dense_read || ge->args[i].reads();
        continue;
      }
      bool has_zero = false;
      for (unsigned j = 0; j < nd; j++) has_zero = has_zero || strs[k][j] == 0;
      const ssize_t sx = strs[k][nd - 1];
      if (ge->args[i].writes() || !has_zero || (sx != 0 && sx != (ssize_t)elsz[k])) return false;
      // one aligned load per chunk: unit stride along an inner extent of whole
      // chunks, every other stride and the first element on chunk boundaries
      bool whole_chunks = sx == (ssize_t)elsz[k] && V > 1 && dims[nd - 1] % V == 0;
      {
        const size_t cb = elsz[k] * V;
        const GpuArray *v = (const GpuArray *)args[i];
        if (((uintptr_t)v->data->devptr + offs[k]) % cb != 0) whole_chunks = false;
        for (unsigned j = 0; j + 1 < nd; j++)
          if (strs[k][j] % (ssize_t)cb != 0) whole_chunks = false;
      }
      if (whole_chunks) pi.pvmask |= 1u << k;
      // one load on four-byte boundaries for the chunks inside a row: the
      // operand's own base and outer strides only need the element's alignment.
      // A wavefront with a chunk that straddles two rows runs both ways, so
      // this is for long rows.  Measured on MI355X, o = a + b with b one row,
      // element by element / this way: rows of 50257 floats 91.2 -> 86.4 us
      // (73.6 -> 77.7 % of peak), of 2050 91.1 -> 84.6, (512, 64, 2050) +
      // (512, 1, 2050) 93.9 -> 88.4, rows of 1001 87.7 -> 85.8 (but 16 MB of
      // them 8.0 -> 8.3); rows of 17 90.3 -> 116.9, of 10 54.1 -> 70.0.
      if (sx == 4 && elsz[k] == 4 && V == 4 &&
          dims[nd - 1] >= (size_t)TUNE(tn, ELEMWISE_PERIODIC_ROWLOAD, 1024) && TUNE(tn, ELEMWISE_PERIODIC_ROWLOAD, 1024) != 0) {
        const GpuArray *v = (const GpuArray *)args[i];
        bool ok = ((uintptr_t)v->data->devptr + offs[k]) % 4 == 0;
        for (unsigned j = 0; j + 1 < nd; j++) ok = ok && strs[k][j] % 4 == 0;
        if (ok) pi.pumask |= 1u << k;
      }
      inner_constant = inner_constant && (sx == 0 || (whole_chunks && TUNE(tn, ELEMWISE_PERIODIC_VEC, 1)));
      pi.pmask |= 1u << k;
      for (unsigned j = 0; j < nd; j++) pi.ps[k][3 - nd + j] = strs[k][j];
    }
    if (pi.pmask == 0) return false;
    // (four per lane on any layout, `loose`, does not count here: rows of a few
    // elements are all cut quads - (2^24, 3) + (1, 3) 154 us that way, 60 us flat)
    if (vec4 && !loose && mode != 2 && !(inner_constant && dense_read)) return false;
    pi.pnd = nd;
    auto magic = [](unsigned d, uint64_t &m, unsigned &k) {
      unsigned c = 0;
      while (((uint64_t)1 << c) < d) c++;
      k = 31 + c;                                   // exact for dividends below 2^31
      m = (((uint64_t)1 << k) + d - 1) / d;
    };
    pi.d2 = (unsigned)dims[nd - 1];
    pi.d1 = (unsigned)dims[nd - 2];
    magic(pi.d2, pi.m2, pi.k2);
    magic(pi.d1, pi.m1, pi.k1);
    return true;
  }

  void find_transposed_operands() {
    // Transposed operands: small stride on some outer dim, large on x.
    // (from 12 elements along that dim on: out = in.T of (N, 13) floats 470 us with
    // single elements per lane, 222 through tiles, of (N, 15) 539 / 200; of (N, 11)
    // 395 / 436, of (N, 8) 299 / 341)
    if (nd >= 2 && dims[nd - 1] >= 16) {
      // candidate y axis: the outer dim on which most arrays have their
      // smallest non-zero stride
      std::vector<unsigned> votes(nd, 0);
      std::vector<int> best(na, -1);
      for (unsigned k = 0; k < na; k++) {
        size_t sx = sabs(strs[k][nd - 1]);
        if (sx == 0) continue;
        int b = -1;
        size_t bs = sx;
        for (unsigned j = 0; j + 1 < nd; j++) {
          size_t sj = sabs(strs[k][j]);
          if (sj != 0 && sj < bs && sj <= 4 * elsz[k] && dims[j] >= (size_t)TUNE(tn, ELEMWISE_TMIN, 12)) { bs = sj; b = (int)j; }
        }
        best[k] = b;
        if (b >= 0) votes[b]++;
      }
      int y = -1;
      for (unsigned j = 0; j + 1 < nd; j++)
        if (votes[j] > 0 && (y < 0 || votes[j] > votes[y])) y = (int)j;
      if (y >= 0) {
        size_t lds = 0;
        for (unsigned k = 0; k < na; k++)
          if (best[k] == y) { tmask |= 1u << k; lds += 64 * 65 * elsz[k]; }
        if (lds > 64 * 1024 || na > 31) tmask = 0;
        if (tmask && (unsigned)y != nd - 2) {
          // rotate y into position nd-2
          size_t dy = dims[y];
          dims.erase(dims.begin() + y);
          dims.insert(dims.begin() + (nd - 2), dy);
          for (unsigned k = 0; k < na; k++) {
            ssize_t sy = strs[k][y];
            strs[k].erase(strs[k].begin() + y);
            strs[k].insert(strs[k].begin() + (nd - 2), sy);
          }
        }
      }
    }
  }

  bool array_writes(unsigned k) const {
    unsigned l = 0;
    for (size_t i = 0; i < ge->args.size(); i++)
      if (ge->args[i].is_array() && l++ == k) return ge->args[i].writes();
    return false;
  }

  void choose_offset_width() {
    // 32-bit offsets when every reachable byte offset fits
    idx64 = n >= (size_t)GA_SADDR32_MAX;
    for (unsigned k = 0; k < na && !idx64; k++) {
      size_t reach = elsz[k];
      for (unsigned j = 0; j < nd; j++) reach += (dims[j] - 1) * sabs(strs[k][j]);
      if (reach >= (size_t)GA_SADDR32_MAX) idx64 = true;
    }
  }

  void choose_vector_access() {
    // Four elements per lane when the layout allows it (see gen_strided_vec).
    // Without transposed operands and with 8-byte elements a lane moves two
    // elements at a time, not four: its widest access is then 16 bytes, and a
    // wavefront's accesses lie side by side (four doubles per lane are two
    // 16-byte accesses 32 bytes apart from the neighbour's; kernel times,
    // four / two per lane: a[:, :4096] + b[:, 4096:] of 8192 x 8192 doubles
    // 144.1 / 121.6 us, the same of 64-bit integers 143.6 / 122.9, (4096, 8192)
    // + (1, 8192) doubles as a strided call 117.5 / 81.7).
    vq = 4;
    if (tmask == 0 && TUNE(tn, ELEMWISE_PAIRS, 1) != 0)
      for (unsigned k = 0; k < na; k++)
        if (elsz[k] == 8) vq = 2;
    vec4 = TUNE(tn, ELEMWISE_VEC4, 1) != 0 && dims[nd - 1] % vq == 0 &&
                strs[outk][nd - 1] == (ssize_t)elsz[outk] && na <= 31;
    if (vec4 && tmask && dims[nd - 2] % 4 != 0) vec4 = false;
    for (unsigned k = 0; k < na && vec4; k++) {
      if (elsz[k] > 8) { vec4 = false; break; }
      const size_t q = vq * elsz[k];
      unsigned l2 = 0;
      const GpuArray *v = nullptr;
      for (size_t i = 0; i < ge->args.size(); i++)
        if (ge->args[i].is_array() && l2++ == k) { v = (const GpuArray *)args[i]; break; }
      const bool base_ok = ((uintptr_t)v->data->devptr + v->offset) % q == 0;
      const bool tr = (tmask >> k) & 1u;
      const unsigned unit_dim = tr ? nd - 2 : nd - 1;
      bool aligned = base_ok && strs[k][unit_dim] == (ssize_t)elsz[k];
      for (unsigned j = 0; j < nd && aligned; j++)
        if (j != unit_dim && strs[k][j] % (ssize_t)q != 0) aligned = false;
      if (tr) {
        if (!aligned) vec4 = false;          // a transposed operand must be vector-accessible
      } else if (aligned) {
        umask |= 1u << k;
      } else if (strs[k][nd - 1] == 0 && TUNE(tn, ELEMWISE_ZMASK, 1) != 0) {
        zmask |= 1u << k;
      }
      if (!tr && tmask && k < 16 && strs[k][nd - 2] == 0 && TUNE(tn, ELEMWISE_ZMASK, 1) != 0)
        zmask |= 1u << (16 + k);
    }
    if (vec4 && !((umask >> outk) & 1u)) vec4 = false;
    // Transposed operands whose layout fails the above - an extent that is no
    // multiple of four, rows that start off the 16-byte boundaries - still
    // move four elements per lane when every array has four-byte elements:
    // accesses that only assume a four-byte boundary, and the quads that an
    // extent cuts element by element (see the generator).  Measured on
    // MI355X, out = in.T of floats, one element per lane against this:
    // 8190 x 8190 154.9 / 110.6 us, 8191 x 8193 150.1 / 106.2; 8192 x 8192
    // inside wider buffers, the result's pitch 8318 floats 154.1 / 96.3, the
    // operand's 8319 floats 117.2 / 101.4, extents 8190 on pitches of 8320
    // floats 102.9 / 93.1; out = in.T + b of 8190 x 8190 207.4 / 158.4.
    // The same without transposed operands (a row's quads then start on the
    // result's 16-byte boundaries): o = a + b on 8192 rows of 8191 floats
    // inside pitches of 8320 137.9 / 122.5 us (73 -> 82 % of peak), rows of
    // 8192 that start one element in 144.0 / 121.9, pitches of 8319 floats
    // 141.8 / 125.6, 65536 rows of 1001 in pitches of 1003 141.9 / 122.2.
    // Only for arrays that cannot all sit in the 256 MB of the last-level cache:
    // on data that does, the kernel with one element per lane (fewer
    // instructions, no cut quads) is the faster one.  Side of a square
    // float array, transposed copy and o = a + b on row views, one element per
    // lane against this, the same buffers every call / rotating through more
    // buffers than the cache holds: 2047 +53 % / +9 % and +5 % / -2 %, 4095
    // +39 % / -15 % and +22 % / -16 %, 8190 -29 % / -29 % and -12 % / -11 %.
    loose = false;
    size_t footprint = 0;
    for (unsigned k = 0; k < na; k++) {
      bool once = true;
      for (unsigned j = 0; j < nd && once; j++)
        if (dims[j] > 1 && strs[k][j] == 0) once = false;
      if (once) footprint += n * elsz[k];
    }
    if (!vec4 && !((tmask >> outk) & 1u) && TUNE(tn, ELEMWISE_VEC4, 1) != 0 &&
        footprint >= (size_t)TUNE(tn, ELEMWISE_LOOSE_MIN_BYTES, 256u << 20) &&
        TUNE(tn, ELEMWISE_LOOSE, 1) != 0 && na <= 31 && strs[outk][nd - 1] == 4) {
      bool ok = true;
      unsigned um = 0, zm = 0;
      for (unsigned k = 0; k < na && ok; k++) {
        const bool tr = (tmask >> k) & 1u;
        if (elsz[k] != 4) ok = false;
        else if (tr) ok = strs[k][nd - 2] == 4 && !array_writes(k);
        else if (strs[k][nd - 1] == 4) um |= 1u << k;
        else if (strs[k][nd - 1] == 0 && TUNE(tn, ELEMWISE_ZMASK, 1) != 0) zm |= 1u << k;
        if (!tr && tmask && k < 16 && strs[k][nd - 2] == 0 && TUNE(tn, ELEMWISE_ZMASK, 1) != 0) zm |= 1u << (16 + k);
      }
      if (ok) {
        loose = vec4 = true;
        vq = 4;
        umask = um;
        zmask = zm;
      }
    }
    // arrays read or written exactly once per element stream past the caches
    if (vec4 && ge->nontemporal) {
      for (unsigned k = 0; k < na; k++) {
        bool once = true;
        for (unsigned j = 0; j < nd && once; j++)
          if (dims[j] > 1 && strs[k][j] == 0) once = false;
        // A transposed operand whose rows do not start on 128-byte lines: a
        // tile's 512-byte pieces of them share their first and last line with
        // the neighbouring tiles', and a streamed line is fetched again by the
        // neighbour (out = in.T of 8190 x 8190 floats read 1.38 times the array).
        // Such an operand stays cacheable: (5000, 3000) -> (3000, 5000) 27.1 ->
        // 21.2 us (55 -> 71 % of peak), 8190 x 8190 110.8 -> 97.7, (50000, 1000) ->
        // (1000, 50000) 80.8 -> 76.4; on whole lines streaming is ahead (a.T + b
        // of 8192 x 8192 121.6 us streamed, 128.0 cacheable).
        if (once && ((tmask >> k) & 1u) && TUNE(tn, ELEMWISE_NT_LINES, 1) != 0) {
          unsigned l2 = 0;
          const GpuArray *v = nullptr;
          for (size_t i = 0; i < ge->args.size(); i++)
            if (ge->args[i].is_array() && l2++ == k) { v = (const GpuArray *)args[i]; break; }
          bool lines = ((uintptr_t)v->data->devptr + v->offset) % 128 == 0;
          for (unsigned j = 0; j < nd && lines; j++)
            if (j != nd - 2 && dims[j] > 1 && strs[k][j] % 128 != 0) lines = false;
          if (!lines) once = false;
        }
        if (once) ntmask |= 1u << k;
      }
      ntmask &= (unsigned)TUNE(tn, ELEMWISE_NT_MASK, 0xffffffffu);
    }
  }

  int choose_grid() {
    // launch geometry
    if (tmask == 0) {
      size_t inner = vec4 ? dims[nd - 1] / vq : dims[nd - 1];   // lanes needed along x
      // (loose: a row's quads start up to three elements before it)
      skew = 0;
      if (vec4 && loose) { inner = (dims[nd - 1] + 6) / 4; skew = (unsigned)outk + 1; }
      // as many lanes along x as the inner extent needs (a power of two), the
      // rest of the 256 along the rows: 2^24 floats in rows of 3 took 191 us
      // with a floor of 16 lanes along x, 61 us without
      ltx = 0;
      while (ltx < 8 && ((size_t)1 << ltx) < inner) ltx++;
      size_t tx = (size_t)1 << ltx, ty = 256 >> ltx;
      size_t rows = n / dims[nd - 1];
      // Quads (of four elements) per lane, each a group's width apart along
      // x.  One per lane when a quad of the widest type has 16 bytes, as in
      // the flat kernel; narrower types get more, and so do grids of one to
      // four fills of the chip.  Kernel times with 4 / 2 / 1 quads per lane,
      // floats: outer product into 8192 x 8192 49.8 / 45.2 / 39.7 us,
      // (8192, 8192) + (1, 8192) 87.5 / 85.6 / 80.1, (4096, 10, 4096) *
      // (1, 10, 1) 220 / 216 / 199, a[:, ::2] + b 168.7 / 168.8 / 162.6,
      // (4096, 4096) + (1, 4096) 23.3 / 22.4 / 20.9; halves (8192, 8192) +
      // (1, 8192) 46.3 / 46.2 / 53.9; (64, 100000) * (64, 1), three fills at
      // one quad per lane, 7.9 / 9.0 / 9.2.
      if (vec4) {
        size_t widest = 1;
        for (unsigned k = 0; k < na; k++) widest = std::max(widest, elsz[k]);
        quads = vq * widest >= 16 ? 1 : (unsigned)(16 / (vq * widest));
        const size_t fill = (size_t)ga_hip_numprocs(ctx) * 8;
        const size_t g1 = ((inner + quads * tx - 1) / (quads * tx)) * ((rows + ty - 1) / ty);
        if (g1 > fill && g1 <= 2 * fill) quads = std::min(4u, quads * 2);
        else if (g1 > 2 * fill && g1 <= 4 * fill) quads = 4;
        const unsigned long forced = TUNE(tn, ELEMWISE_QUADS, 0);
        if (forced == 1 || forced == 2 || forced == 4) quads = (unsigned)forced;
      }
      gx = (inner + quads * tx - 1) / (quads * tx);
      groups = gx * ((rows + ty - 1) / ty);
    } else {
      // Transposed tiles.  A group takes a 64 x 64 tile (256 lanes) or a
      // 128 x 128 tile (1024 lanes).  The tiles of a plane are handed out
      // either in bands of `ltx` tile rows, down a band's rows first, or
      // (ltx = 0) along diagonals, so that groups running together differ in
      // both tile coordinates.  Measured on MI355X, kernel time of
      // out = in.T of floats, small / large tiles, each in row-major order
      // (bands of 1), bands of 8 and diagonal order:
      //    4096 x  4096   24.5  25.3  24.4 |  24.8  23.9  23.6 us
      //    8192 x  8192  108.9 103.1  93.4 |  88.1  88.1  82.1
      //   16384 x 16384  433   471   406   | 364   422   398
      //    2048 x 16384   51.1  52.5  48.7 |  47.0  49.5  44.9
      //   16384 x  2048   50.8  53.4  61.1 |  48.2  47.0  53.8
      //    6144 x  6144   54.5  56.7  57.4 |  53.6  53.7  57.3
      //    3000 x  5000   31.1  29.5  36.6 |  27.3  27.5  28.7
      // and the same in.T with two broadcast operands on 4096 x 4096 25.7 /
      // 25.7 / 24.9 | 26.1 / 25.8 / 25.1 (a plain copy of as many bytes: 22.3).
      // So: the large tile from half a group per compute unit on, when its
      // staging copies leave room for two groups per unit; diagonal
      // order when every row pitch involved is a power of two of 4 to 32 KiB
      // (rows that many bytes apart fall on the same memory channels, and
      // row-major order then has all groups of a tile row read such rows);
      // row-major order otherwise.
      // Two tiles per group, with the second tile's loads issued before the
      // first one's results are stored, measured no better (the same
      // in.T + b*c 24.0 -> 24.5 us, 8192 x 8192 82.0 -> 83.5): two resident
      // groups per compute unit already overlap one's loads with the other's
      // stores.
      skew = 0;
      if (vec4) {
        // Rows of the result off the 64-byte blocks of memory: the tiles' windows
        // follow the rows (see the generator).  Measured on MI355X, out = in.T
        // of 8192 x 8192 floats, rectangular against skewed tiles: result rows
        // 32 bytes into a block 135.8 / 92.6 us, a pitch of 8328 floats (the
        // rows walk through the four phases) 114.1 / 95.5, both pitches 8200
        // floats 114.5 / 102.4; (5000, 3000) -> (3000, 5000) 27.2 / 25.9.
        // (large arrays only, like `loose`: 2047 x 2047 floats ran 12 to 19 % slower this way)
        size_t moved = 0;
        for (unsigned k = 0; k < na; k++)
          if (strs[k][nd - 1] != 0 && strs[k][nd - 2] != 0) moved += n * elsz[k];
        if (outk >= 0 && !((tmask >> outk) & 1u) && elsz[outk] == 4 && TUNE(tn, ELEMWISE_SKEW, 1) != 0 &&
            moved >= (size_t)TUNE(tn, ELEMWISE_LOOSE_MIN_BYTES, 256u << 20)) {
          bool wide = false;
          for (unsigned k = 0; k < na; k++) wide = wide || elsz[k] > 4;
          const GpuArray *ov = nullptr;
          unsigned l2 = 0;
          for (size_t i = 0; i < ge->args.size(); i++)
            if (ge->args[i].is_array() && l2++ == (unsigned)outk) { ov = (const GpuArray *)args[i]; break; }
          bool whole = ((uintptr_t)ov->data->devptr + ov->offset) % 64 == 0;
          for (unsigned j = 0; j + 1 < nd && whole; j++)
            if (dims[j] > 1 && strs[outk][j] % 64 != 0) whole = false;
          if (!wide && !whole) skew = (unsigned)outk + 1;
        }
        const size_t cols = skew ? (loose ? 15 : 12) : 0;
        size_t lds128 = 0;
        for (unsigned k = 0; k < na; k++)
          if ((tmask >> k) & 1u) lds128 += (size_t)128 * ((128 + cols) | 1) * elsz[k];
        const size_t tiles128 = ((dims[nd - 1] + cols + 127) / 128) * ((dims[nd - 2] + 127) / 128) *
                                (n / dims[nd - 1] / dims[nd - 2]);
        // large against small tiles on smaller planes: 1536 x 1536 4.6 / 4.9 us,
        // 2048 x 2048 6.2 / 6.9, 16 planes of 512 x 512 6.0 / 6.6, 3072 x 3072
        // 15.3 / 14.8, 1024 x 1024 4.2 / 4.2
        const size_t min128 = TUNE(tn, ELEMWISE_TTILE_MIN, ga_hip_numprocs(ctx) / 2);
        tile = (tiles128 >= min128 && lds128 <= 80 * 1024) ? 128 : 64;
        // A narrow plane - (N, 48) taken as its transpose - leaves most of a large
        // tile empty: the small one where it is filled better by a tenth and more.
        // out = in.T of 256 MiB of floats, large / small tiles: rows of 20
        // 232 / 147 us (29 / 46 % of peak), of 33 171 / 116, of 48 125 / 103, of 49
        // 138 / 105, of 130 117 / 104; of 100 101 / 118 and of 196 107 / 114 fill
        // both alike and keep the large one.
        if (tile == 128 && TUNE(tn, ELEMWISE_TTILE_FILL, 1) != 0) {
          auto fill = [&](size_t t) {
            const double fx = (double)dims[nd - 1] / (double)((dims[nd - 1] + t - 1) / t * t);
            const double fy = (double)dims[nd - 2] / (double)((dims[nd - 2] + t - 1) / t * t);
            return fx * fy;
          };
          if (fill(64) > fill(128) + 0.1) tile = 64;
        }
        const unsigned long ft = TUNE(tn, ELEMWISE_TTILE, 0);
        if (ft == 64 || (ft == 128 && lds128 <= 160 * 1024)) tile = (unsigned)ft;
        const size_t tiles = ((dims[nd - 1] + cols + tile - 1) / tile) * ((dims[nd - 2] + tile - 1) / tile);
        bool aliasing = true;   // every pitch a power of two of 4 to 32 KiB
        for (unsigned k = 0; k < na && aliasing; k++) {
          // operands that are broadcast along x or y are a row or a column, not a plane
          if (strs[k][nd - 1] == 0 || strs[k][nd - 2] == 0) continue;
          const size_t pitch = sabs(strs[k][((tmask >> k) & 1u) ? nd - 1 : nd - 2]);
          aliasing = (pitch & (pitch - 1)) == 0 && pitch >= 4096 && pitch <= 32768;
        }
        const unsigned long dflt = aliasing ? 0 : (tile == 128 ? 1 : (tiles >= 8192 ? 8 : 1));
        ltx = (unsigned)TUNE(tn, ELEMWISE_BAND, dflt) & 0xffffu;
        if (ltx == 0) ltx |= ((unsigned)TUNE(tn, ELEMWISE_PANEL, 0) & 0xffffu) << 16;
      }
      gx = (dims[nd - 1] + (skew ? (loose ? 15 : 12) : 0) + tile - 1) / tile;
      size_t gy = (dims[nd - 2] + tile - 1) / tile;
      size_t outer = n / dims[nd - 1] / dims[nd - 2];
      groups = gx * gy * outer;
    }
    if (!idx64 && (groups >= (size_t)GA_SADDR32_MAX || gx >= (size_t)GA_SADDR32_MAX)) idx64 = true;
    if (groups > 0x7fffffffull || gx > 0xffffffffull)
      return ga_err_set(ctx->err, GA_XLARGE_ERROR, "Iteration space needs more groups than one launch has");
    return GA_NO_ERROR;
  }

  int get_kernel() {
    // (0: a lane's four 8-byte elements along a transposed tile's axes stay adjacent)
    const bool tpairs = TUNE(tn, ELEMWISE_TPAIRS, 1) != 0;
    char key[64];
    snprintf(key, sizeof(key), "%s%u:%d:%x:%x:%x:%x:%u:%u:%u:%d:%u", vec4 ? (loose ? "l" : "v") : "s", nd, idx64 ? 1 : 0, tmask,
             vec4 ? umask : 0u, ntmask, vec4 ? zmask : 0u, tile, quads, vq, tpairs ? 1 : 0, vec4 ? skew : 0u);
    auto it = ge->k_strided.find(key);
    if (it != ge->k_strided.end()) {
      kernel = &it->second;
    } else {
      std::vector<int> ktypes;
      std::string src = vec4 ? gen_strided_vec(ge, nd, idx64, tmask, umask, ktypes, ntmask, tile, zmask, quads, vq, tpairs, skew, loose)
                             : gen_strided(ge, nd, idx64, tmask, ktypes);
      GpuKernel nk = {nullptr, nullptr};
      int err = build_kernel(ge, &nk, src, ktypes);
      if (err != GA_NO_ERROR) return err;
      kernel = &ge->k_strided.emplace(key, nk).first->second;
    }
    return GA_NO_ERROR;
  }

  // (leaves the launch to GpuElemwise_call, see ew_launch)
  int launch() {
    if (ge->args.size() > 255)
      return ga_err_set(ctx->err, GA_UNSUPPORTED_ERROR, "More than 255 arguments");
    ew_launch &L = ge->pending;
    L.slots.clear();
    unsigned l = 0;
    for (unsigned j = 0; j < nd; j++) L.value(dims[j]);
    for (size_t i = 0; i < ge->args.size(); i++) {
      if (ge->args[i].is_array()) {
        const GpuArray *v = (const GpuArray *)args[i];
        L.array(i);
        L.value(v->offset);
        for (unsigned j = 0; j < nd; j++) L.value(strs[l][j]);
        l++;
      } else {
        L.scalar(i);
      }
    }
    const unsigned int gx32 = (unsigned int)gx;
    L.value(gx32);
    L.value(ltx);
    L.k = kernel;
    L.gs = groups;
    L.ls = (vec4 && tmask) ? (size_t)tile * tile / 16 : 256;
    L.valid = true;
    return GA_NO_ERROR;
  }
};

int call_general(GpuElemwise *ge, void **args, size_t n, unsigned nd) {
  return strided_call(ge, args, n, nd).run();
}

}  // namespace

// Fill the descriptor part of an operator (no context, no kernels).
static int ge_describe(GpuElemwise *ge, const char *preamble, const char *expr, unsigned int n,
                       gpuelemwise_arg *args, int flags, ga_errrec *err) {
  ge->expr = expr;
  ge->preamble = preamble ? preamble : "";
  ge->flags = flags;
  size_t maxel = 1;
  for (unsigned int i = 0; i < n; i++) {
    ge_arg a;
    a.name = args[i].name ? args[i].name : "";
    a.typecode = args[i].typecode;
    a.flags = args[i].flags;
    if (a.name.empty() || gpuarray_get_type(a.typecode)->cluda_name == nullptr)
      return ga_err_fmt(err, GA_VALUE_ERROR, "Argument %u has no name or an unknown type (%d)", i,
                        a.typecode);
    if (a.is_array()) {
      ge->narray++;
      maxel = std::max(maxel, gpuarray_get_elsize(a.typecode));
    }
    ge->args.push_back(a);
  }
  ge->kflags = gpuarray_type_flagsa(n, args);
  // chunk = 16 bytes of the widest element type (32 bytes measured slower for
  // every mix of types: floats 121 -> 142 us for 2^26 elements, bytes to floats
  // 126 -> 182 for 2^27); fewer chunks in flight when many arrays are live at once
  ge->vec = maxel >= 16 ? 1 : (unsigned)(16 / maxel);
  ge->unroll = ge->narray <= 8 ? 2 : 1;
  {
    // narrow inputs: every array read has elements of a quarter of the widest
    // or less; narrow outputs: every array written is narrower than the widest
    // and either at most one wide array is read or they are a quarter or less
    bool in_quarter = true, out_narrow = true, out_quarter = true, any_in = false;
    unsigned wide_in = 0;
    for (const ge_arg &a : ge->args) {
      if (!a.is_array()) continue;
      const size_t es = gpuarray_get_elsize(a.typecode);
      if (a.reads()) {
        any_in = true;
        if (es * 4 > maxel) in_quarter = false;
        if (es == maxel) wide_in++;
      }
      if (a.writes()) {
        if (es >= maxel) out_narrow = false;
        if (es * 4 > maxel) out_quarter = false;
      }
    }
    ge->narrow_side = ge->narray <= 8 && ((any_in && in_quarter) || (out_narrow && (wide_in <= 1 || out_quarter)));
  }
  const ga_tuning *tn = ga_hip_tuning(ge->ctx);
  ge->flat_forced = tn->is_set(KNOB_ELEMWISE_UNROLL) || tn->is_set(KNOB_ELEMWISE_TILE);
  ge->unroll = (unsigned)TUNE(tn, ELEMWISE_UNROLL, ge->unroll);
  if (ge->unroll < 1) ge->unroll = 1;
  ge->tile = TUNE(tn, ELEMWISE_TILE, 0) != 0;
  ge->nontemporal = TUNE(tn, ELEMWISE_NT, 1) != 0;
  ge->flat_nt_mask = (unsigned)TUNE(tn, ELEMWISE_FLAT_NT_MASK, 0xffffffffu);
  return GA_NO_ERROR;
}

extern "C" {

// Kernel text for one variant, for checks that have no device: strided == 0
// gives the flat kernel, otherwise the strided kernel for (nd, idx64, tmask).
// The caller frees the result.
GPUARRAY_PUBLIC char *ga_elemwise_gen_source(const char *preamble, const char *expr,
                                             unsigned int n, gpuelemwise_arg *args, int flags,
                                             int strided, unsigned int nd, int idx64,
                                             unsigned int tmask) {
  GpuElemwise ge;
  if (expr == nullptr || ge_describe(&ge, preamble, expr, n, args, flags, ga_global_err) != GA_NO_ERROR)
    return nullptr;
  std::vector<int> ktypes;
  // strided: 0 flat, 1 strided one element per lane, 2 strided four elements per
  // lane (then bits 16.. of tmask carry the mask of arrays with unit x stride),
  // 3 the same with streaming 16-byte accesses on every array, 4 as 3 with
  // 128 x 128 transposed tiles; 5 and 6: the flat kernel with 2 and 4 adjacent
  // chunks per lane; 7 as 4, every array in neither mask taken as constant along x;
  // 8 as 4, every array that is not staged through LDS taken as constant along y
  if (strided == 5 || strided == 6) return strdup(gen_flat(&ge, ktypes, strided == 5 ? 2 : 4, 1).c_str());
  // 10: as 3 with one group of two elements per lane (8-byte types, no transposed operand)
  // 11: as 4, the tiles' windows on a row starting on the 64-byte blocks of the last array's rows
  // 12: as 11 for four-byte elements on any bases, pitches and extents
  // 13: as 3 for the same
  // 9: the flat kernel with the arrays in tmask read through the coordinates of the flat index (nd = 2 or 3)
  // (idx64 then carries the mask of those fetched a whole chunk at a time)
  // (and its bits 16.. the mask of those that fetch a chunk inside one row with one load on four-byte boundaries)
  if (strided == 9)
    return strdup(gen_flat(&ge, ktypes, 0, -1, tmask, nd, (unsigned)idx64 & 0xffffu, (unsigned)idx64 >> 16).c_str());
  // 14: a narrow plane in registers: nd carries the short extent (plus 256: planes, three dims), idx64 bit 0 the offsets' width, bit 1 the
  // short dim, bit 2 streaming accesses, bit 3 the first kind of arrays through the LDS, bit 4 the second kind
  // on four-byte boundaries, bit 5 the arrays of neither kind constant along the long dim; tmask the arrays with the short dim innermost, its bits 16.. those with the long one
  if (strided == 14) {
    unsigned es = 8;   // the smallest element size among the arrays
    for (const ge_arg &a : ge.args)
      if (a.is_array()) es = std::min(es, (unsigned)gpuarray_get_elsize(a.typecode));
    return strdup(gen_narrow_block(&ge, (idx64 & 1) != 0, nd & 0xffu, (((unsigned)idx64 >> 1) & 1u) + (nd >> 8), tmask & 0xffffu,
                                   tmask >> 16, (idx64 & 4) ? tmask >> 16 : 0u, ktypes, (idx64 & 16) ? tmask >> 16 : 0u,
                                   (idx64 & 8) ? tmask & 0xffffu : 0u, 2 + (nd >> 8), es,
                                   (idx64 & 32) ? ~(tmask | (tmask >> 16)) & ((1u << ge.narray) - 1u) : 0u).c_str());
  }
  // 16: tiles of short records: nd carries the record's elements (plus 256: planes, four dims), idx64 bit 0 the
  // offsets' width, bit 2 streaming accesses, bit 3 windows moved onto the last array's 64-byte blocks, bit 4 tiles
  // numbered along Y first; tmask the
  // arrays whose records follow one another along Y, its bits 16.. those laid out like the result
  if (strided == 16) {
    unsigned es = 4;   // the element size of every array: the first one's
    for (const ge_arg &a : ge.args)
      if (a.is_array()) {
        es = (unsigned)gpuarray_get_elsize(a.typecode);
        break;
      }
    const unsigned F = nd & 0xffu, fb = F * es;
    unsigned T = fb <= 6 ? 64 : fb <= 28 ? 32 : fb <= 124 ? 16 : 8;
    while ((T * F) % (((idx64 & 8) ? 64 : 16) / es) != 0 && T < 64) T *= 2;
    return strdup(gen_record_tiles(&ge, 3 + (nd >> 8), (idx64 & 1) != 0, F, T, tmask & 0xffffu, tmask >> 16,
                                   (idx64 & 4) ? tmask >> 16 : 0u, ktypes, (idx64 & 8) ? (int)ge.narray - 1 : -1, es,
                                   (idx64 & 16) != 0).c_str());
  }
  // 15: the same arguments for a wider short extent, whole through the LDS
  if (strided == 15)
    return strdup(gen_narrow_staged(&ge, (idx64 & 1) != 0, nd & 0xffu, (((unsigned)idx64 >> 1) & 1u) + (nd >> 8), tmask & 0xffffu,
                                    tmask >> 16, (idx64 & 4) ? 0xffffu : 0u, ktypes, (idx64 & 16) ? tmask >> 16 : 0u,
                                    2 + (nd >> 8)).c_str());
  std::string src = strided >= 2 ? gen_strided_vec(&ge, nd, idx64 != 0, tmask & 0xffffu, tmask >> 16, ktypes,
                                                   strided >= 3 ? 0xffffffffu : 0u, strided >= 4 && strided != 13 ? 128 : 64,
                                                   strided == 7 ? ~(tmask | (tmask >> 16)) & 0xffffu
                                                   : strided == 8 ? (~tmask & 0xffffu) << 16 : 0u,
                                                   strided == 10 ? 1 : 4, strided == 10 ? 2 : 4, true,
                                                   strided >= 11 && strided <= 13 ? ge.narray : 0,
                                                   strided == 12 || strided == 13)
                    : strided  ? gen_strided(&ge, nd, idx64 != 0, tmask, ktypes)
                               : gen_flat(&ge, ktypes);
  return strdup(src.c_str());
}

GpuElemwise *GpuElemwise_new(gpucontext *ctx, const char *preamble, const char *expr,
                             unsigned int n, gpuelemwise_arg *args, unsigned int nd, int flags) {
  (void)nd;  // strided kernels are specialised on the call's layout and built on first use
  if (expr == nullptr || (n > 0 && args == nullptr)) {
    ga_err_set(ctx->err, GA_VALUE_ERROR, "GpuElemwise_new: NULL expression or arguments");
    return nullptr;
  }
  GpuElemwise *ge = new (std::nothrow) GpuElemwise();
  if (ge == nullptr) {
    ga_err_set(ctx->err, GA_MEMORY_ERROR, "Out of memory");
    return nullptr;
  }
  ge->ctx = ctx;
  if (ge_describe(ge, preamble, expr, n, args, flags, ctx->err) != GA_NO_ERROR) {
    delete ge;
    return nullptr;
  }

  std::vector<int> ktypes;
  std::string src = gen_flat(ge, ktypes);
  if (build_kernel(ge, &ge->k_flat, src, ktypes) != GA_NO_ERROR) {
    GpuElemwise_free(ge);
    return nullptr;
  }
  return ge;
}

void GpuElemwise_free(GpuElemwise *ge) {
  if (ge == nullptr) return;
  if (ge->k_flat.k != nullptr || ge->k_flat.args != nullptr) GpuKernel_clear(&ge->k_flat);
  for (auto &kv : ge->k_flat_tiled) GpuKernel_clear(&kv.second);
  for (auto &kv : ge->k_flat_periodic) GpuKernel_clear(&kv.second);
  for (auto &kv : ge->k_strided) GpuKernel_clear(&kv.second);
  delete ge;
}

namespace {

int ew_issue(const ew_launch &L, void **args) {
  void *fixed[96];
  std::vector<void *> many;
  void **argv = fixed;
  if (L.slots.size() > 96) {
    many.resize(L.slots.size());
    argv = many.data();
  }
  for (size_t i = 0; i < L.slots.size(); i++) {
    const ew_slot &s = L.slots[i];
    argv[i] = s.kind == ew_slot::VALUE ? (void *)&s.value
              : s.kind == ew_slot::ARRAY ? (void *)((GpuArray *)args[s.arg])->data : args[s.arg];
  }
  return GpuKernel_call(L.k, 1, &L.gs, &L.ls, 0, argv);
}

// The key of a call (see ew_memo); 0 when the call is not one to remember.
unsigned ew_key(const GpuElemwise *ge, void **args, int flags, int64_t *key) {
  if (ge->narray > 8 || ge->args.size() > 255) return 0;
  unsigned n = 0;
  key[n++] = flags;
  key[n++] = (int64_t)ga_hip_tuning(ge->ctx)->generation;
  for (size_t i = 0; i < ge->args.size(); i++) {
    if (!ge->args[i].is_array()) continue;
    const GpuArray *v = (const GpuArray *)args[i];
    if (v == nullptr || v->data == nullptr || v->nd > 8) return 0;
    key[n++] = (int64_t)v->nd | ((int64_t)(unsigned)v->flags << 8) | ((int64_t)v->typecode << 40);
    for (unsigned j = 0; j < v->nd; j++) {
      key[n++] = (int64_t)v->dimensions[j];
      key[n++] = (int64_t)v->strides[j];
    }
    key[n++] = (int64_t)v->offset;
    key[n++] = (int64_t)((uintptr_t)v->data->devptr & 255u);
  }
  return n;   // at most 2 + 8 * (3 + 16) = 154
}

int ew_plan(GpuElemwise *ge, void **args, int flags) {
  size_t n = 0;
  bool flat = false;
  if (check_flat(ge, args, &n, &flat) == GA_NO_ERROR && flat) {
    if (n == 0) return GA_NO_ERROR;
    std::vector<size_t> offs;
    for (size_t i = 0; i < ge->args.size(); i++)
      if (ge->args[i].is_array()) offs.push_back(((GpuArray *)args[i])->offset);
    if (offs.empty()) return ga_err_set(ge->ctx->err, GA_VALUE_ERROR, "No output arrays");
    return call_flat(ge, args, n, offs.data());
  }
  unsigned nd = 0;
  int err = check_general(ge, args, flags, &n, &nd);
  if (err != GA_NO_ERROR) return err;
  if (n == 0) return GA_NO_ERROR;
  return call_general(ge, args, n, nd);
}

}  // namespace

int GpuElemwise_call(GpuElemwise *ge, void **args, int flags) {
  // ELEMWISE_MEMO: 0 plans every call anew; 2 plans every call anew and
  // compares with the kept plan where there is one (a difference is a planner
  // input missing from the key: the process stops)
  const unsigned long mode = TUNE(ga_hip_tuning(ge->ctx), ELEMWISE_MEMO, 1);
  int64_t key[EW_KEYMAX];
  const unsigned nkey = mode ? ew_key(ge, args, flags, key) : 0;
  ew_memo *hit = nullptr;
  if (nkey != 0) {
    for (size_t i = 0; i < ge->memo.size(); i++) {
      ew_memo &m = ge->memo[i];
      if (m.nkey == nkey && memcmp(m.key, key, nkey * sizeof(int64_t)) == 0) {
        hit = &m;
        break;
      }
    }
  }
  if (hit != nullptr && mode != 2) return ew_issue(hit->launch, args);
  ge->pending.valid = false;
  const int err = ew_plan(ge, args, flags);
  if (err != GA_NO_ERROR || !ge->pending.valid) {   // (an empty iteration space launches nothing)
    if (hit != nullptr) {
      fprintf(stderr, "libgpuarray: a remembered elementwise plan exists for a call that planning refuses (%d)\n", err);
      abort();
    }
    return err;
  }
  const ew_launch &L = ge->pending;
  if (hit != nullptr) {
    const ew_launch &H = hit->launch;
    bool same = H.k == L.k && H.gs == L.gs && H.ls == L.ls && H.slots.size() == L.slots.size();
    for (size_t i = 0; same && i < L.slots.size(); i++)
      same = H.slots[i].kind == L.slots[i].kind && H.slots[i].arg == L.slots[i].arg &&
             H.slots[i].value == L.slots[i].value;
    if (!same) {
      fprintf(stderr, "libgpuarray: a remembered elementwise plan differs from the plan made anew\n");
      abort();
    }
  } else if (nkey != 0) {
    // a few entries, replaced in turn once all are taken
    const bool room = ge->memo.size() < EW_ENTRIES;
    if (room) ge->memo.emplace_back();
    ew_memo &m = room ? ge->memo.back() : ge->memo[ge->memo_next++ % EW_ENTRIES];
    m.nkey = nkey;
    memcpy(m.key, key, nkey * sizeof(int64_t));
    m.launch = L;
  }
  return ew_issue(L, args);
}

}  // extern "C"
