/* CPU restatement of the reference's elementwise and reduction path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing the library ships may include, link or
 * call this file; it exists so that tests, the smoke check and the CPU leg of
 * the benchmark have an independent statement of what the reference computes.
 *
 * Each function follows the reference code it cites, loop order included, in
 * plain scalar C on host memory.  The reference's own C sources cannot be
 * built here as a checker: every translation unit on this path includes
 * headers its build system generates (private_config.h from
 * src/private_config.h.in, gpuarray/abi_version.h from src/CMakeLists.txt:
 * 118-127), so there is no oracle/_ref; this restatement is pinned instead by
 * the reference's literal test vectors (tests/check_util.c:41-148,
 * tests/check_elemwise.c:39-880, pygpu/tests/test_tools.py:6-118), by the CPU
 * loops of tests/check_reduction.c:125-142,215-232,303-331,402-419 on its own
 * PCG32 data, and by NumPy / closed forms.
 *
 * Parity unpinned (no reference path exists): float16 sums.  The reference
 * refuses them (pygpu/reduction.py:156-160); orc_reduk follows the same
 * template with a float accumulator and is checked against NumPy only.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <sys/types.h>

/* ---- PCG XSH RR 64/32, the generator of tests/check_reduction.c:32-63 ---- */
static uint64_t pcg_state = 1;
void orc_pcg_seed(uint64_t seed) { pcg_state = seed; }
static uint32_t pcg_ror(uint32_t x, uint32_t n) {
  n &= 0x1f;
  return n ? (x >> n) | (x << (32 - n)) : x;
}
uint32_t orc_pcg_rand(void) {
  pcg_state = pcg_state * 6364136223846793005ULL + 1442695040888963407ULL;
  return pcg_ror((uint32_t)((pcg_state ^ (pcg_state >> 18)) >> 27), (uint32_t)(pcg_state >> 59));
}
double orc_pcg_rand01(void) {
  uint64_t u = orc_pcg_rand(), l = orc_pcg_rand();
  return (double)(u << 32 | l) / 18446744073709551616.0;
}
/* fill n floats exactly as the reference tests do: pSrc[i] = pcgRand01() */
void orc_pcg_fill_f32(float *dst, size_t n, uint64_t seed) {
  orc_pcg_seed(seed);
  for (size_t i = 0; i < n; i++) dst[i] = (float)orc_pcg_rand01();
}

/* ---- float -> half, src/gpuarray/util.h:107-183 --------------------------- */
uint16_t orc_float2half(float f) {
  union { float f; uint32_t u; } b;
  b.f = f;
  uint16_t sgn = (uint16_t)((b.u & 0x80000000u) >> 16);
  uint32_t e = b.u & 0x7f800000u, sig;
  if (e >= 0x47800000u) {
    if (e == 0x7f800000u) {
      sig = b.u & 0x007fffffu;
      if (sig != 0) {
        uint16_t r = (uint16_t)(0x7c00u + (sig >> 13));
        if (r == 0x7c00u) r++;
        return (uint16_t)(r + sgn);
      }
      return (uint16_t)(sgn + 0x7c00u);
    }
    return (uint16_t)(sgn + 0x7c00u);
  }
  if (e <= 0x38000000u) {
    if (e < 0x33000000u) return sgn;
    e >>= 23;
    sig = 0x00800000u + (b.u & 0x007fffffu);
    sig >>= (113 - e);
    sig += 0x00001000u;
    return (uint16_t)(sgn + (uint16_t)(sig >> 13));
  }
  uint16_t he = (uint16_t)((e - 0x38000000u) >> 13);
  sig = (b.u & 0x007fffffu) + 0x00001000u;
  return (uint16_t)(sgn + he + (uint16_t)(sig >> 13));
}

/* ---- dimension collapsing, src/gpuarray_util.c:153-188 -------------------- */
static void shift_sz(size_t *r, unsigned i, unsigned nd) {
  memmove(&r[i], &r[i + 1], (nd - i - 1) * sizeof(size_t));
}
static void shift_ss(ssize_t *r, unsigned i, unsigned nd) {
  if (r) memmove(&r[i], &r[i + 1], (nd - i - 1) * sizeof(ssize_t));
}
void orc_collapse(unsigned n, unsigned *pnd, size_t *dims, ssize_t **strs) {
  unsigned nd = *pnd, i, k;
  for (i = nd; i > 0; i--) {
    if (nd > 1 && dims[i - 1] == 1) {
      shift_sz(dims, i - 1, nd);
      for (k = 0; k < n; k++) shift_ss(strs[k], i - 1, nd);
      nd--;
    }
  }
  for (i = nd - 1; i > 0; i--) {
    int collapse = 1;
    for (k = 0; k < n; k++)
      collapse &= (strs[k] == NULL || strs[k][i - 1] == (ssize_t)dims[i] * strs[k][i]);
    if (collapse) {
      dims[i - 1] *= dims[i];
      shift_sz(dims, i, nd);
      for (k = 0; k < n; k++)
        if (strs[k] != NULL) {
          strs[k][i - 1] = strs[k][i];
          shift_ss(strs[k], i, nd);
        }
      nd--;
    }
  }
  *pnd = nd;
}

/* ---- argument checking, src/gpuarray_elemwise.c:272-383 ---------------------
 * narr arrays; and[k], ad[k][], as[k][] their rank, dims and byte strides;
 * is_out[k] marks GE_WRITE arrays.  flags: 0x100 broadcast, 0x200 nocollapse,
 * 0x400 padshape.  On success (0) nd/dims/strs (row-major narr x maxnd) hold
 * the planned iteration space and *call32 the 32-bit decision; 2 is
 * GA_VALUE_ERROR. */
int orc_check_basic(unsigned narr, const unsigned *and_, const size_t *const *ad,
                    const ssize_t *const *as, const size_t *aoff, const int *is_out, int flags,
                    unsigned maxnd, unsigned *nd_out, size_t *dims, ssize_t *strs, size_t *n_out,
                    int *call32_out) {
  unsigned nd = 0, i, j;
  int out = -1, call32 = 1;
  size_t n = 1;
  for (i = 0; i < narr; i++) {
    if (i == 0) nd = and_[i];
    else if (and_[i] != nd) {
      if (flags & 0x400) nd = and_[i] > nd ? and_[i] : nd;
      else return 2;
    }
    if (out < 0 && is_out[i]) out = (int)i;
  }
  if (out < 0 || nd > maxnd) return 2;
  if (and_[out] != nd) return 2; /* the reference reads past the output's dims here */
  memcpy(dims, ad[out], nd * sizeof(size_t));
  for (i = 0; i < narr; i++) {
    memset(&strs[i * maxnd], 0, nd * sizeof(ssize_t));
    memcpy(&strs[i * maxnd + (nd - and_[i])], as[i], and_[i] * sizeof(ssize_t));
  }
  for (j = 0; j < nd; j++) {
    for (i = 0; i < narr; i++) {
      size_t vd = j < nd - and_[i] ? 1 : ad[i][j - (nd - and_[i])];
      if (dims[j] != vd) {
        if (!(flags & 0x100) || is_out[i] || vd != 1) return 2;
      }
      if (vd == 1) strs[i * maxnd + j] = 0;
      call32 &= aoff[i] < 4294967295UL;
      call32 &= (-2147483648L < strs[i * maxnd + j] && strs[i * maxnd + j] < 2147483647L);
    }
    n *= dims[j];
  }
  call32 &= n < 4294967295UL;
  if (!(flags & 0x200) && nd > 1) {
    ssize_t *rows[64];
    if (narr > 64) return 2;
    for (i = 0; i < narr; i++) rows[i] = &strs[i * maxnd];
    orc_collapse(narr, &nd, dims, rows);
  }
  *nd_out = nd;
  *n_out = n;
  *call32_out = call32;
  return 0;
}

/* ---- the strided kernel body, src/gpuarray_elemwise.c:198-238 ----------------
 * For flat index i: unravel from the last dim with % and /, add pos*stride to
 * every array's byte offset, load, evaluate, store.  The expression is chosen
 * by `expr`; operands are raw byte pointers (base + offset applied by the
 * caller), so any strides, negative ones included, work.  Scalars come in
 * `sc` as doubles/ints reinterpreted per expression. */
enum {
  ORC_MULADD_HALF_F32 = 0, /* c = a*b + 0.5f          (3 arrays: a b c, float)      */
  ORC_A_PLUS_BC_F32 = 1,   /* out = a + b*c           (4 arrays: a b c out, float)  */
  ORC_ADD_U32 = 2,         /* c = a + b               (3 arrays, uint32)            */
  ORC_ADD_F16 = 3,         /* c = a + b with GE_CONVERT_F16 (3 arrays, half)        */
  ORC_AXPB_U32 = 4,        /* c = a + x*b             (a b c uint32, scalar x u32)  */
  ORC_SAXPY_I32_F32 = 5,   /* y = a*x + y             (x int32, y float, scalar a)  */
  ORC_COPY_F32 = 6,        /* dst = src               (2 arrays, float)             */
  ORC_COPY_F16_F32 = 7,    /* dst = src, half -> float through GE_CONVERT_F16       */
  ORC_COPY_I32_I64 = 8     /* dst = src, int32 -> int64                             */
};

static float half2float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1f, m = h & 0x3ffu, bits;
  if (e == 0x1f) bits = sign | 0x7f800000u | (m << 13);
  else if (e == 0) {
    if (m == 0) bits = sign;
    else {
      int sh = 0;
      while (!(m & 0x400u)) { m <<= 1; sh++; }
      bits = sign | ((uint32_t)(113 - sh) << 23) | ((m & 0x3ffu) << 13);
    }
  } else bits = sign | ((e + 112) << 23) | (m << 13);
  float f;
  memcpy(&f, &bits, 4);
  return f;
}
float orc_half2float(uint16_t h) { return half2float(h); }

/* device-side float->half is round-to-nearest-even (src/cluda_cuda.h:70-77
 * cvt.rn, src/cluda_opencl.h:46-55 vstore_half_rte) */
static uint16_t float2half_rte(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  int32_t e = (int32_t)((x >> 23) & 0xff) - 127 + 15;
  uint32_t m = x & 0x7fffffu;
  if (((x >> 23) & 0xff) == 0xff) return (uint16_t)(sign | 0x7c00u | (m ? (0x200u | (m >> 13)) : 0));
  if (e >= 0x1f) return (uint16_t)(sign | 0x7c00u);
  if (e <= 0) {
    if (e < -10) return (uint16_t)sign;
    m |= 0x800000u;
    uint32_t shift = (uint32_t)(14 - e);
    uint32_t hm = m >> shift, rem = m & ((1u << shift) - 1), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (hm & 1))) hm++;
    return (uint16_t)(sign | hm);
  }
  uint32_t hm = m >> 13, rem = m & 0x1fffu;
  uint32_t r = ((uint32_t)e << 10) | hm;
  if (rem > 0x1000u || (rem == 0x1000u && (r & 1))) r++;
  return (uint16_t)(sign | r);
}
uint16_t orc_float2half_rte(float f) { return float2half_rte(f); }

int orc_elemwise(int expr, size_t n, unsigned nd, const size_t *dims, unsigned narr,
                 char *const *base, const ssize_t *strs /* narr x nd */, const void *sc) {
  for (size_t i = 0; i < n; i++) {
    size_t ii = i, pos;
    char *p[8];
    if (narr > 8) return 2;
    for (unsigned k = 0; k < narr; k++) p[k] = base[k];
    for (unsigned d = nd; d > 0; d--) {
      if (d - 1 > 0) { pos = ii % dims[d - 1]; ii = ii / dims[d - 1]; } else pos = ii;
      for (unsigned k = 0; k < narr; k++) p[k] += (ssize_t)pos * strs[k * nd + (d - 1)];
    }
    switch (expr) {
    case ORC_MULADD_HALF_F32: {
      volatile float prod = *(float *)p[0] * *(float *)p[1]; /* two roundings, no contraction */
      *(float *)p[2] = prod + 0.5f;
      break;
    }
    case ORC_A_PLUS_BC_F32: {
      volatile float prod = *(float *)p[1] * *(float *)p[2];
      *(float *)p[3] = *(float *)p[0] + prod;
      break;
    }
    case ORC_ADD_U32: *(uint32_t *)p[2] = *(uint32_t *)p[0] + *(uint32_t *)p[1]; break;
    case ORC_ADD_F16: {
      float a = half2float(*(uint16_t *)p[0]), b = half2float(*(uint16_t *)p[1]);
      *(uint16_t *)p[2] = float2half_rte(a + b);
      break;
    }
    case ORC_AXPB_U32:
      *(uint32_t *)p[2] = *(uint32_t *)p[0] + *(const uint32_t *)sc * *(uint32_t *)p[1];
      break;
    case ORC_SAXPY_I32_F32: {
      volatile float prod = *(const float *)sc * (float)*(int32_t *)p[0];
      *(float *)p[1] = prod + *(float *)p[1];
      break;
    }
    case ORC_COPY_F32: *(float *)p[1] = *(float *)p[0]; break;
    case ORC_COPY_F16_F32: *(float *)p[1] = half2float(*(uint16_t *)p[0]); break;
    case ORC_COPY_I32_I64: *(int64_t *)p[1] = *(int32_t *)p[0]; break;
    default: return 5;
    }
  }
  return 0;
}

/* The flat kernel, src/gpuarray_elemwise.c:472-532, for c = a*b + 0.5f: the
 * CPU leg of the benchmark. */
void orc_elemwise_contig_muladd(size_t n, const float *a, const float *b, float *c) {
  for (size_t i = 0; i < n; i++) {
    volatile float prod = a[i] * b[i];
    c[i] = prod + 0.5f;
  }
}

/* ---- GpuKernel_sched, src/gpuarray_kernel.c:38-89 --------------------------- */
void orc_sched(size_t n, size_t max_l, size_t min_l, unsigned numprocs, size_t max_g, size_t *gs,
               size_t *ls) {
  size_t target_g = (size_t)numprocs * 32, target_l = 512;
  int want_ls = 0;
  if (target_g > max_g) target_g = max_g;
  if (target_l > max_l) target_l = max_l;
  if (*ls == 0) { want_ls = 1; *ls = min_l; }
  if (*gs == 0) {
    *gs = ((n - 1) / *ls) + 1;
    if (*gs > target_g) *gs = target_g;
  }
  if (want_ls && n > (*ls * *gs)) {
    *ls = ((n / min_l) / *gs) * min_l;
    if (*ls > target_l) *ls = target_l;
  }
}

/* ---- maxandargmax, src/gpuarray_reduction.c:545-607 -------------------------
 * For every coordinate of the free axes (ascending axis order) scan the
 * reduced axes in reduxList order, last listed axis fastest, with a strict
 * '>' against the running maximum that starts at the first element; the
 * index is sum_k i_k * prod_{j>k} dim[r_j] (src/gpuarray/array.h:626-635).
 * Element type: 0 float, 1 double, 2 int32, 3 half (compared as float).
 * dmax / darg are addressed through their own byte strides. */
static double load_as_double(const char *p, int et) {
  switch (et) {
  case 0: return *(const float *)p;
  case 1: return *(const double *)p;
  case 2: return *(const int32_t *)p;
  default: return half2float(*(const uint16_t *)p);
  }
}
static size_t et_size(int et) { return et == 1 ? 8 : (et == 3 ? 2 : 4); }

int orc_maxandargmax(const char *src, int et, unsigned nd, const size_t *dims,
                     const ssize_t *strides, unsigned nr, const unsigned *redux, char *dmax,
                     const ssize_t *dmax_str, char *darg, const ssize_t *darg_str) {
  unsigned freeax[32], nf = 0;
  size_t fcount = 1, rcount = 1;
  if (nd > 32 || nr == 0 || nr > nd) return 4;
  for (unsigned a = 0; a < nd; a++) {
    int isr = 0;
    for (unsigned k = 0; k < nr; k++) isr |= redux[k] == a;
    if (!isr) { freeax[nf++] = a; fcount *= dims[a]; }
  }
  for (unsigned k = 0; k < nr; k++) {
    if (redux[k] >= nd) return 4;
    for (unsigned j = 0; j < k; j++) if (redux[j] == redux[k]) return 4;
    rcount *= dims[redux[k]];
  }
  for (size_t f = 0; f < fcount; f++) {
    /* free coordinate, last free axis fastest */
    size_t t = f;
    ssize_t so = 0, mo = 0, ao = 0;
    for (unsigned k = nf; k > 0; k--) {
      size_t c = t % dims[freeax[k - 1]];
      t /= dims[freeax[k - 1]];
      so += (ssize_t)c * strides[freeax[k - 1]];
      mo += (ssize_t)c * dmax_str[k - 1];
      ao += (ssize_t)c * darg_str[k - 1];
    }
    const char *best = src + so; /* all reduced coordinates 0 */
    double bestv = load_as_double(best, et);
    int64_t besti = 0;
    for (size_t r = 0; r < rcount; r++) {
      size_t u = r;
      ssize_t ro = 0;
      for (unsigned k = nr; k > 0; k--) {
        size_t c = u % dims[redux[k - 1]];
        u /= dims[redux[k - 1]];
        ro += (ssize_t)c * strides[redux[k - 1]];
      }
      double v = load_as_double(src + so + ro, et);
      if (v > bestv) { bestv = v; besti = (int64_t)r; best = src + so + ro; }
    }
    memcpy(dmax + mo, best, et_size(et));
    *(int64_t *)(darg + ao) = besti;
  }
  return 0;
}

/* ---- the Python reduction kernel, pygpu/reduction.py:33-134 -----------------
 * One work-group of `ls` lanes per output: lane `lid` folds elements lid,
 * lid+ls, ... of the flattened reduced index into an accumulator of the
 * OUTPUT type starting from the neutral element; the lanes are then combined
 * by the halving tree ldata[lid] = REDUCE(ldata[lid], ldata[lid+s]),
 * s = ls/2 .. 1.  Free coordinates come from the group id in C order; the
 * output is written densely (out[gid]).
 *   op: 0 sum, 1 prod, 2 all (&&), 3 any (||)
 *   in/out element types: 0 float, 1 double, 2 int32, 3 half, 4 int64, 5 uint8
 */
static void acc_load(double *accd, int64_t *acci, const char *p, int in_t, int out_t, int op) {
  (void)out_t; (void)op;
  switch (in_t) {
  case 0: *accd = *(const float *)p; *acci = (int64_t)*(const float *)p; break;
  case 1: *accd = *(const double *)p; *acci = (int64_t)*(const double *)p; break;
  case 2: *accd = *(const int32_t *)p; *acci = *(const int32_t *)p; break;
  case 3: *accd = half2float(*(const uint16_t *)p); *acci = (int64_t)*accd; break;
  case 4: *accd = (double)*(const int64_t *)p; *acci = *(const int64_t *)p; break;
  default: *accd = *(const uint8_t *)p; *acci = *(const uint8_t *)p; break;
  }
}

int orc_reduk(int op, const char *src, int in_t, unsigned nd, const size_t *dims,
              const ssize_t *strides, const int *redux /* nd flags */, char *out, int out_t,
              size_t ls) {
  size_t gs = 1, n = 1;
  for (unsigned d = 0; d < nd; d++) {
    if (redux[d]) n *= dims[d]; else gs *= dims[d];
  }
  const int isint = out_t == 2 || out_t == 4 || out_t == 5;
  const int isf32 = out_t == 0 || out_t == 3;
  double *ld = (double *)malloc(ls * sizeof(double));
  int64_t *li = (int64_t *)malloc(ls * sizeof(int64_t));
  if (!ld || !li) { free(ld); free(li); return 1; }
  for (size_t g = 0; g < gs; g++) {
    /* free position from the group id, C order */
    size_t t = g;
    ssize_t fo = 0;
    for (unsigned d = nd; d > 0; d--) {
      if (redux[d - 1]) continue;
      size_t c = t % dims[d - 1];
      t /= dims[d - 1];
      fo += (ssize_t)c * strides[d - 1];
    }
    for (size_t lid = 0; lid < ls; lid++) {
      double ad = (op == 1 || op == 2) ? 1.0 : 0.0;
      int64_t ai = (op == 1 || op == 2) ? 1 : 0;
      float af = (float)ad;
      for (size_t i = lid; i < n; i += ls) {
        size_t u = i;
        ssize_t ro = 0;
        for (unsigned d = nd; d > 0; d--) {
          if (!redux[d - 1]) continue;
          size_t c = u % dims[d - 1];
          u /= dims[d - 1];
          ro += (ssize_t)c * strides[d - 1];
        }
        double xd;
        int64_t xi;
        acc_load(&xd, &xi, src + fo + ro, in_t, out_t, op);
        switch (op) {
        case 0:
          if (isint) ai = (int64_t)((uint64_t)ai + (uint64_t)xi);
          else if (isf32) { volatile float s = af + (float)xd; af = s; }
          else ad = ad + xd;
          break;
        case 1:
          if (isint) ai = (int64_t)((uint64_t)ai * (uint64_t)xi);
          else if (isf32) { volatile float s = af * (float)xd; af = s; }
          else ad = ad * xd;
          break;
        case 2: ai = (ai && (xd != 0.0)) ? 1 : 0; break;
        default: ai = (ai || (xd != 0.0)) ? 1 : 0; break;
        }
      }
      ld[lid] = isf32 ? (double)af : ad;
      li[lid] = ai;
    }
    for (size_t s = ls / 2; s >= 1; s /= 2) {
      for (size_t lid = 0; lid < s; lid++) {
        switch (op) {
        case 0:
          if (isint || op >= 2) li[lid] = (int64_t)((uint64_t)li[lid] + (uint64_t)li[lid + s]);
          else if (isf32) { volatile float r = (float)ld[lid] + (float)ld[lid + s]; ld[lid] = r; }
          else ld[lid] = ld[lid] + ld[lid + s];
          break;
        case 1:
          if (isint) li[lid] = (int64_t)((uint64_t)li[lid] * (uint64_t)li[lid + s]);
          else if (isf32) { volatile float r = (float)ld[lid] * (float)ld[lid + s]; ld[lid] = r; }
          else ld[lid] = ld[lid] * ld[lid + s];
          break;
        case 2: li[lid] = (li[lid] && li[lid + s]) ? 1 : 0; break;
        default: li[lid] = (li[lid] || li[lid + s]) ? 1 : 0; break;
        }
      }
      if (s == 1) break;
    }
    const int boolish = op >= 2;
    switch (out_t) {
    case 0: ((float *)out)[g] = boolish ? (float)li[0] : (float)ld[0]; break;
    case 1: ((double *)out)[g] = boolish ? (double)li[0] : ld[0]; break;
    case 2: ((int32_t *)out)[g] = (int32_t)li[0]; break;
    case 3: ((uint16_t *)out)[g] = float2half_rte((float)ld[0]); break;
    case 4: ((int64_t *)out)[g] = li[0]; break;
    default: ((uint8_t *)out)[g] = (uint8_t)li[0]; break;
    }
  }
  free(ld);
  free(li);
  return 0;
}

/* ---- take1, src/gpuarray_array.c:325-383 (kernel text) and :385-548 -------
 * r is C-contiguous [n0, n1]; for every (i0, i1): the index ind[i0] is
 * wrapped once when negative, an index still outside [0, d0) sets *err = -1
 * and leaves the element alone; i1 is unravelled over v's trailing dims,
 * last dim fastest (:352-361), into a byte position through v's strides.
 * Elements are moved as `elsz` bytes (same type on both sides).
 * ind_kind: size in bytes of an index, negative when the type is signed. */
int orc_take1(char *r, const char *v, size_t elsz, unsigned nd, const size_t *vdims,
              const ssize_t *vstr, const void *ind, int ind_kind, size_t n0, int *err) {
  size_t n1 = 1;
  for (unsigned j = 1; j < nd; j++) n1 *= vdims[j];
  for (size_t i0 = 0; i0 < n0; i0++) {
    for (size_t i1 = 0; i1 < n1; i1++) {
      long long ii0;
      switch (ind_kind) {
      case -1: ii0 = ((const int8_t *)ind)[i0]; break;
      case 1: ii0 = ((const uint8_t *)ind)[i0]; break;
      case -2: ii0 = ((const int16_t *)ind)[i0]; break;
      case 2: ii0 = ((const uint16_t *)ind)[i0]; break;
      case -4: ii0 = ((const int32_t *)ind)[i0]; break;
      case 4: ii0 = ((const uint32_t *)ind)[i0]; break;
      case -8: ii0 = ((const int64_t *)ind)[i0]; break;
      case 8: ii0 = (long long)((const uint64_t *)ind)[i0]; break;
      default: return 4;
      }
      ssize_t pos = 0;
      size_t idx = i1;
      if (ii0 < 0) ii0 += (long long)vdims[0];
      if (ii0 < 0 || ii0 >= (long long)vdims[0]) { *err = -1; continue; }
      pos += ii0 * vstr[0];
      for (unsigned j = nd - 1; j >= 1; j--) {
        size_t ij = idx % vdims[j];
        idx /= vdims[j];
        pos += (ssize_t)ij * vstr[j];
      }
      memcpy(r + (i0 * n1 + i1) * elsz, v + pos, elsz);
    }
  }
  return 0;
}

/* ---- the same kernel with a map expression over two arrays and a scalar ------
 * pygpu/reduction.py:33-134 with `arguments` = (a, b, s) and `map_expr` set
 * (the use of pygpu/tests/test_reduction.py:57-84): each array has its own
 * strides over the common dims (0 on a broadcast dim, pygpu/tools.py
 * check_args); element i of the flattened reduced index contributes
 * REDUCE(acc, map(a[i], b[i], s)); accumulator and output have type `t`
 * (0 float, 1 double).
 *   map: 0 a*b   1 fabs(a-b)   2 s*a+b   3 a*a
 *   red: 0 a+b from 0          1 max(a,b) from -inf */
static double map2(int map, double a, double b, double s, int t) {
  if (t == 0) {
    volatile float r;
    float fa = (float)a, fb = (float)b, fs = (float)s;
    switch (map) {
    case 0: r = fa * fb; break;
    case 1: r = fabsf(fa - fb); break;
    case 2: { volatile float m = fs * fa; r = m + fb; break; }
    default: r = fa * fa; break;
    }
    return r;
  }
  switch (map) {
  case 0: return a * b;
  case 1: return fabs(a - b);
  case 2: { volatile double m = s * a; return m + b; }
  default: return a * a;
  }
}
static double red2(int red, double x, double y, int t) {
  if (red == 1) return (y > x) ? y : x;
  if (t == 0) { volatile float r = (float)x + (float)y; return r; }
  return x + y;
}
int orc_reduk_map2(int map, int red, int t, unsigned nd, const size_t *dims, const char *a,
                   const ssize_t *astr, const char *b, const ssize_t *bstr, double s,
                   const int *redux, char *out, size_t ls) {
  size_t gs = 1, n = 1;
  for (unsigned d = 0; d < nd; d++) {
    if (redux[d]) n *= dims[d]; else gs *= dims[d];
  }
  double *ld = (double *)malloc(ls * sizeof(double));
  if (!ld) return 1;
  for (size_t g = 0; g < gs; g++) {
    size_t tt = g;
    ssize_t fa = 0, fb = 0;
    for (unsigned d = nd; d > 0; d--) {
      if (redux[d - 1]) continue;
      size_t c = tt % dims[d - 1];
      tt /= dims[d - 1];
      fa += (ssize_t)c * astr[d - 1];
      fb += (ssize_t)c * bstr[d - 1];
    }
    for (size_t lid = 0; lid < ls; lid++) {
      double acc = red == 1 ? -INFINITY : 0.0;
      for (size_t i = lid; i < n; i += ls) {
        size_t u = i;
        ssize_t ra = 0, rb = 0;
        for (unsigned d = nd; d > 0; d--) {
          if (!redux[d - 1]) continue;
          size_t c = u % dims[d - 1];
          u /= dims[d - 1];
          ra += (ssize_t)c * astr[d - 1];
          rb += (ssize_t)c * bstr[d - 1];
        }
        double xa = t == 0 ? *(const float *)(a + fa + ra) : *(const double *)(a + fa + ra);
        double xb = t == 0 ? *(const float *)(b + fb + rb) : *(const double *)(b + fb + rb);
        acc = red2(red, acc, map2(map, xa, xb, s, t), t);
      }
      ld[lid] = acc;
    }
    for (size_t cur = ls / 2; cur >= 1; cur /= 2)
      for (size_t lid = 0; lid < cur; lid++) ld[lid] = red2(red, ld[lid], ld[lid + cur], t);
    if (t == 0) ((float *)out)[g] = (float)ld[0];
    else ((double *)out)[g] = ld[0];
  }
  free(ld);
  return 0;
}
