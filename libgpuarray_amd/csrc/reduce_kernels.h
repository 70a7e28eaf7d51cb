/* Reduction kernels for gfx950, written for 64-lane wavefronts.
 *
 * This text is compiled at run time behind a short list of #defines that the
 * host planner emits (element types, operation, lane geometry):
 *
 *   RD_NSRC     number of source arrays (1 for a plain reduction; more when
 *               an elementwise expression over several arrays feeds the
 *               reduction)
 *   RD_ACC_T    accumulator type           RD_KIND      operation, RD_K_* below
 *   RD_DST_T    value result type          RD_DST_HALF  value result is ga_half
 *   RD_IDX_T    index result type          RD_ARG       carry (value, index)
 *   RD_HAS_D0 / RD_HAS_D1                  which results are written
 *   RD_NEUTRAL  neutral element of the operation, of type RD_ACC_T
 *   RD_FLT      the reduced values are floating (NaN rules apply)
 *   RD_CUSTOM_OP(a, b) / RD_NEUTRAL  the caller's combination and its neutral
 *               element when RD_KIND is RD_K_CUSTOM
 *   RD_G        lanes that share one output in redux_row: 64 or 256
 *   RD_VEC      elements per load in redux_row (inner reduced stride is the
 *               element size and everything is aligned when > 1)
 *   RD_ES       element step of the inner reduced dim inside a load: the dim
 *               advances by RD_ES elements per index (a [::2] or [::4] view), a
 *               load fetches RD_VEC*RD_ES contiguous elements and every
 *               RD_ES-th one is used
 *   RD_FAST8    one-byte elements combined four per 32-bit operation (sum, any,
 *               all; 1: unsigned bytes, 2: signed), 0: off
 *   RD_COL_FAST8  redux_col: any / all over one-byte elements work on whole words
 *   RD_XCD      redux_col: groups that follow one another in the kernel's order run on one die
 *   RD_CLOOSE   redux_col: a lane's RD_CV adjacent elements are fetched with a
 *               load that only assumes the elements' own alignment, and the
 *               inner free dim need not be a multiple of RD_CV (the lane that
 *               holds its end fetches its elements one by one)
 *   RD_SROWS    also emit redux_srows (short contiguous rows staged in LDS)
 *   RD_PCOLS    emit redux_pcols (leading dims of a dense array reduced over
 *               short kept rows, the array walked as one run of chunks)
 *   RD_WANT     which kernels the text holds: bit 0 redux_row, bit 1 redux_col,
 *               bit 2 redux_wrows, bit 3 the second pass (redux_final, and
 *               redux_final_cols beside redux_col)
 *   RD_TAIL     rows that are misaligned for the vector load or whose extent
 *               is not a multiple of RD_VEC (one source, contiguous rows): a
 *               row is read from the vector boundary at or below its start,
 *               `sh` elements early, and every element is tested against
 *               [sh, sh + extent); RD_ELSZ0 is the element size in bytes
 *   RD_U        loads in flight per lane
 *   RD_LO       redux_row: outer reduced coordinates handled side by side by
 *               the RD_G lanes when the inner reduced dim is short (1: none)
 *   RD_IDX32    every count and flat index of the call is below 2^31: 32-bit divisions
 *   RD_RISING   redux_col: the flattened index grows along the scan and fits 31 bits
 *   RD_CV       redux_col: adjacent outputs per lane, fetched with one load
 *   RD_CY       redux_col: lane rows of a group that share the reduced range
 *               (a power of two up to 16); 256 / RD_CY lanes lie along the free dim
 *   RD_L        redux_wrows: lanes that share a row (power of two, <= 64);
 *               64 / RD_L rows sit side by side in a wavefront
 *   RD_RB       redux_wrows: sets of rows whose loads a wavefront issues together
 *   RD_NT       streaming (non-temporal) loads in redux_row
 *   RD_INTERLEAVE  redux_row with one reduced dim: splits take every
 *               nsplit-th unit instead of a contiguous range
 *
 * and, also emitted by the planner, the part that depends on the number and
 * types of the sources (inserted at the @RD_GENERATED@ mark below): the kernels' source
 * parameters, the registers of one lane's loads (rd_unit, rd_one), how they
 * are filled, and the value computed from them (the source element itself, or
 * the caller's expression over the elements of all sources).
 *
 * Semantics (reference src/gpuarray_reduction.c:545-607 for max/argmax,
 * pygpu/reduction.py:33-134 for sum/prod/any/all):
 *   - the accumulator has the result's type; each element is converted to it
 *     before the operation;
 *   - arg-reductions return the flattened index over the reduced axes in the
 *     caller's axis order; ties keep the lowest index.  The reference scans
 *     sequentially with a strict compare, which is the same thing; here the
 *     (value, index) pair is combined with "better value, or equal value and
 *     lower index", so the result does not depend on the shape of the tree;
 *   - NaN never wins a strict compare, so the reference ignores a NaN unless
 *     it is the first element scanned, in which case it stays.  Elements
 *     other than the first are therefore mapped to -inf (max) / +inf (min),
 *     and the result is overwritten when element 0 is NaN;
 *   - sums use a fixed order (per lane sequential over its units, pairwise
 *     inside a unit, then the cross-lane network below), so results are
 *     reproducible run to run.
 *
 * The kernels:
 *   redux_row    lanes run along the fastest REDUCED dim; RD_G lanes
 *                cooperate on one output; a row can be cut in `nsplit` pieces
 *                that each leave a partial.
 *   redux_wrows  the same for short rows (one pass of a wavefront covers a
 *                row): a wavefront takes several rows at a time and issues all
 *                their loads before it combines the first.
 *   redux_srows  many short contiguous rows: a group copies its rows to LDS
 *                with full-width loads and each lane then walks one row.
 *   redux_col    lanes run along the fastest FREE dim (coalesced), a lane owns
 *                RD_CV adjacent outputs and walks the reduced range; RD_CY
 *                lane rows share the range and meet in LDS.
 *   redux_final, redux_final_cols  second pass: combine the partials of an
 *                output (a wavefront per output; or lanes along the outputs
 *                when the partials lie split-major).
 */
#include "cluda.h"

#define RD_K_SUM 0
#define RD_K_PROD 1
#define RD_K_PRODNZ 2
#define RD_K_MIN 3
#define RD_K_MAX 4
#define RD_K_AND 5
#define RD_K_OR 6
#define RD_K_XOR 7
#define RD_K_ALL 8
#define RD_K_ANY 9
#define RD_K_CUSTOM 10

#define RD_MAXD 8

/* Iteration space, by value.  Dims are sorted slowest first and collapsed.
 * Strides are in bytes.  `rmul` is what one step along a reduced dim adds to
 * the flattened index. */
struct rd_plan {
  ga_long fdim[RD_MAXD], fd0str[RD_MAXD], fd1str[RD_MAXD];
  ga_long rdim[RD_MAXD], rmul[RD_MAXD];
  ga_long nrows;   /* number of outputs */
  ga_long rtotal;  /* elements reduced per output */
  ga_long nseg;    /* redux_row: segments per pass over the inner reduced dim */
  ga_long units;   /* redux_row: (outer reduced count) * nseg; redux_col: the
                    * launch's groups, rounded down to a multiple of 8 */
  ga_long upb;     /* work per split: units (row) or elements (col) */
  ga_long gx;      /* redux_col: groups along the inner free dim */
  ga_long router;  /* redux_row with RD_LO > 1: count of outer reduced coordinates;
                    * redux_pcols: the number of slabs when more than one */
  ga_int nf, nr, nsplit, split_major;   /* split_major: layout of redux_col's partials */
  ga_int rising, fused;   /* rising: the flattened index grows with the position in the
                           * reduced range, and the range has fewer than 2^31 positions;
                           * fused: the group that finishes an output's last piece also
                           * combines its partials (no second pass) */
  ga_long fsstr[RD_NSRC][RD_MAXD], rsstr[RD_NSRC][RD_MAXD];   /* per source */
};

struct rd_acc {
  RD_ACC_T v;
#if RD_ARG
  ga_long i;
#endif
};

#define RD_IDX_NONE 0x7fffffffffffffffLL

static __device__ inline rd_acc rd_neutral() {
  rd_acc a;
  a.v = RD_NEUTRAL;
#if RD_ARG
  a.i = RD_IDX_NONE;
#endif
  return a;
}

static __device__ inline rd_acc rd_combine(rd_acc a, rd_acc b) {
#if RD_KIND == RD_K_SUM
  a.v = a.v + b.v;
#elif RD_KIND == RD_K_PROD || RD_KIND == RD_K_PRODNZ
  a.v = a.v * b.v;
#elif RD_KIND == RD_K_AND
  a.v = a.v & b.v;
#elif RD_KIND == RD_K_OR
  a.v = a.v | b.v;
#elif RD_KIND == RD_K_XOR
  a.v = a.v ^ b.v;
#elif RD_KIND == RD_K_ALL
  a.v = (a.v && b.v) ? 1 : 0;
#elif RD_KIND == RD_K_ANY
  a.v = (a.v || b.v) ? 1 : 0;
#elif RD_KIND == RD_K_CUSTOM
  a.v = (RD_ACC_T)RD_CUSTOM_OP(a.v, b.v);
#elif RD_KIND == RD_K_MAX
#if RD_ARG
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) a = b;
#else
  if (b.v > a.v) a = b;
#endif
#elif RD_KIND == RD_K_MIN
#if RD_ARG
  if (b.v < a.v || (b.v == a.v && b.i < a.i)) a = b;
#else
  if (b.v < a.v) a = b;
#endif
#endif
  return a;
}

/* One reduced value (a source element, or the caller's expression over the
 * sources' elements), converted for the operation. */
template <typename T>
static __device__ inline rd_acc rd_elem(const T x, ga_long idx) {
  rd_acc a;
#if RD_KIND == RD_K_ALL || RD_KIND == RD_K_ANY
  a.v = (x != 0) ? 1 : 0;
#elif RD_KIND == RD_K_PRODNZ
  a.v = (x == 0) ? (RD_ACC_T)1 : (RD_ACC_T)x;
#elif RD_KIND == RD_K_MAX && RD_FLT
  a.v = (x != x) ? (RD_ACC_T)(-INFINITY) : (RD_ACC_T)x;
#elif RD_KIND == RD_K_MIN && RD_FLT
  a.v = (x != x) ? (RD_ACC_T)(INFINITY) : (RD_ACC_T)x;
#else
  a.v = (RD_ACC_T)x;
#endif
#if RD_ARG
  a.i = idx;
#else
  (void)idx;
#endif
  return a;
}

/* An element's value for a strict compare against a running best that is not
 * a NaN (the first element of the scan went through rd_elem, or the scan
 * started from the neutral value): a NaN loses every such compare by itself,
 * so it needs no mapping. */
template <typename T>
static __device__ inline RD_ACC_T rd_later(const T x) {
#if (RD_KIND == RD_K_MAX || RD_KIND == RD_K_MIN) && RD_FLT
  return (RD_ACC_T)x;
#else
  return rd_elem(x, 0).v;
#endif
}

/* ---- cross-lane network --------------------------------------------------
 * Data-parallel-primitive moves on 32-bit words; an accumulator is moved
 * word by word.  Steps: swap with the neighbour (quad_perm 1,0,3,2), with the
 * other pair (quad_perm 2,3,0,1), mirror within 8, mirror within 16 - after
 * which all 16 lanes of a row agree - then row 0 -> row 1 and row 2 -> row 3
 * (row_bcast:15), rows 0-1 -> rows 2-3 (row_bcast:31).  Lane 63 ends up with
 * the combination of all 64 lanes and is broadcast by a lane read. */
#define RD_DPP_XOR1 0xB1
#define RD_DPP_XOR2 0x4E
#define RD_DPP_HALF_MIRROR 0x141
#define RD_DPP_MIRROR 0x140
#define RD_DPP_BCAST15 0x142
#define RD_DPP_BCAST31 0x143

#define RD_ACC_WORDS ((sizeof(rd_acc) + 3) / 4)

template <int CTRL, int ROWMASK>
static __device__ inline rd_acc rd_dpp(rd_acc x, rd_acc fallback) {
  union { rd_acc a; ga_int w[RD_ACC_WORDS]; } in, old, out;
  in.a = x;
  old.a = fallback;
#pragma unroll
  for (unsigned k = 0; k < RD_ACC_WORDS; k++)
    out.w[k] = __builtin_amdgcn_update_dpp(old.w[k], in.w[k], CTRL, ROWMASK, 0xf, false);
  return out.a;
}

static __device__ inline rd_acc rd_readlane63(rd_acc x) {
  union { rd_acc a; ga_int w[RD_ACC_WORDS]; } in, out;
  in.a = x;
#pragma unroll
  for (unsigned k = 0; k < RD_ACC_WORDS; k++) out.w[k] = __builtin_amdgcn_readlane(in.w[k], 63);
  return out.a;
}

/* Every lane returns the combination of the 64 lanes. */
static __device__ inline rd_acc rd_wave_reduce(rd_acc a) {
  const rd_acc nt = rd_neutral();
  a = rd_combine(a, rd_dpp<RD_DPP_XOR1, 0xf>(a, nt));
  a = rd_combine(a, rd_dpp<RD_DPP_XOR2, 0xf>(a, nt));
  a = rd_combine(a, rd_dpp<RD_DPP_HALF_MIRROR, 0xf>(a, nt));
  a = rd_combine(a, rd_dpp<RD_DPP_MIRROR, 0xf>(a, nt));
  a = rd_combine(a, rd_dpp<RD_DPP_BCAST15, 0xa>(a, nt));
  a = rd_combine(a, rd_dpp<RD_DPP_BCAST31, 0xc>(a, nt));
  return rd_readlane63(a);
}

/* The same over aligned segments of L lanes (a power of two): the first
 * log2(L) steps of the network.  Up to 16 lanes every lane of a segment ends
 * with the result; for 32 the upper 16 lanes do; for 64 all do.  Lane L-1 of
 * a segment holds it in every case. */
template <int L>
static __device__ inline rd_acc rd_seg_reduce(rd_acc a) {
  const rd_acc nt = rd_neutral();
  if (L >= 2) a = rd_combine(a, rd_dpp<RD_DPP_XOR1, 0xf>(a, nt));
  if (L >= 4) a = rd_combine(a, rd_dpp<RD_DPP_XOR2, 0xf>(a, nt));
  if (L >= 8) a = rd_combine(a, rd_dpp<RD_DPP_HALF_MIRROR, 0xf>(a, nt));
  if (L >= 16) a = rd_combine(a, rd_dpp<RD_DPP_MIRROR, 0xf>(a, nt));
  if (L >= 32) a = rd_combine(a, rd_dpp<RD_DPP_BCAST15, 0xa>(a, nt));
  if (L >= 64) {
    a = rd_combine(a, rd_dpp<RD_DPP_BCAST31, 0xc>(a, nt));
    a = rd_readlane63(a);
  }
  return a;
}

/* Combination over the 4 wavefronts of a 256-lane group, through LDS. */
static __device__ inline rd_acc rd_block_reduce(rd_acc a, rd_acc *lds) {
  a = rd_wave_reduce(a);
  const unsigned wave = LID_0 >> 6, lane = LID_0 & 63u;
  if (lane == 0) lds[wave] = a;
  local_barrier();
  rd_acc r = lds[0];
  r = rd_combine(r, lds[1]);
  r = rd_combine(r, lds[2]);
  r = rd_combine(r, lds[3]);
  return r;
}

/* ---- addressing ------------------------------------------------------------ */

/* Offsets of output `row` (flat index over the free dims, slowest first):
 * one per source, and the two destinations'. */
/* q = a / b and the remainder, for non-negative a and positive b.  RD_IDX32:
 * the plan says that every count and flat index of this call is below 2^31,
 * and the division is a 32-bit one (the 64-bit one is a long sequence of
 * instructions, slow to run and slower to compile). */
static __device__ inline ga_long rd_divmod(ga_long a, ga_long b, ga_long *rem) {
#if RD_IDX32
  const ga_uint q = (ga_uint)a / (ga_uint)b;
  *rem = (ga_long)((ga_uint)a - q * (ga_uint)b);
  return (ga_long)q;
#else
  const ga_long q = a / b;
  *rem = a - q * b;
  return q;
#endif
}

static __device__ inline void rd_row_offsets(const rd_plan &p, ga_long row, ga_long *so,
                                             ga_long *d0o, ga_long *d1o) {
  ga_long a = 0, b = 0;
#pragma unroll
  for (int k = 0; k < RD_NSRC; k++) so[k] = 0;
  for (int d = p.nf - 1; d >= 0; d--) {
    ga_long c;
    if (d > 0) { row = rd_divmod(row, p.fdim[d], &c); } else { c = row; }
#pragma unroll
    for (int k = 0; k < RD_NSRC; k++) so[k] += c * p.fsstr[k][d];
    a += c * p.fd0str[d];
    b += c * p.fd1str[d];
  }
  *d0o = a; *d1o = b;
}

/* Byte offsets (per source) and index base of outer reduced coordinate `ro`
 * (flat over the reduced dims 0..ri-1). */
static __device__ inline void rd_outer_offsets(const rd_plan &p, int ri, ga_long ro, ga_long *rb,
                                               ga_long *ib) {
  ga_long x = 0;
#pragma unroll
  for (int k = 0; k < RD_NSRC; k++) rb[k] = 0;
  for (int d = ri - 1; d >= 0; d--) {
    ga_long c;
    if (d > 0) { ro = rd_divmod(ro, p.rdim[d], &c); } else { c = ro; }
#pragma unroll
    for (int k = 0; k < RD_NSRC; k++) rb[k] += c * p.rsstr[k][d];
    x += c * p.rmul[d];
  }
  *ib = x;
}

/* ---- the part that depends on the sources ------------------------------------
 * Emitted by the planner:
 *   RD_SRC_PARAMS            kernel parameters: (pointer, byte offset) per source
 *   RD_SRC_BASES(b)          b[k] = pointer + offset, for every source
 *   RD_SCALAR_PARAMS / RD_SCALAR_FPARAMS / RD_SCALAR_ARGS
 *                            scalar arguments of the caller's expression as
 *                            trailing kernel parameters, function parameters
 *                            and call arguments (all empty when there are none)
 *   struct rd_unit           what one lane fetches for one unit: per source
 *                            RD_U vector loads, or RD_U x RD_VEC scalar loads
 *                            when its inner reduced stride is not its element
 *                            size
 *   rd_unit_load(u, base, e0, rin, rstr)   fill it (loads past `rin` skipped)
 *   RD_UNIT_VAL(u, j, v)     the reduced value of element v of load j
 *   struct rd_one, rd_one_load(o, ptrs), RD_ONE_VAL(o)   the same for one
 *                            element addressed by one pointer per source
 *   struct rd_cvec, rd_cvec_load(o, ptrs, nv), RD_CVEC_VAL(o, c)   the same for
 *                            RD_CV adjacent elements (redux_col)
 * RD_PV (elements per vector load) and RD_LOAD are defined first because the
 * emitted text uses them. */
#define RD_PV (RD_VEC * RD_ES)
/* every source element is read once: stream it past the caches */
#if RD_NT
#define RD_LOAD(p) __builtin_nontemporal_load(p)
#else
#define RD_LOAD(p) (*(p))
#endif

/* A use of a loaded value that no branch can skip.  The compiler waits for a
 * load where its result is first used; when every use sits under a branch that
 * some path skips, the result still counts as pending at the loop's back edge,
 * and in the next pass of the loop each load of the unit waits for the one before it
 * (their destination registers may be in flight) instead of all being issued
 * back to back.  Costs no instruction, but it makes the first use wait for
 * all of the unit's loads; redux_row leaves it out (RD_TOUCH_ROW 0) for sums
 * and the like over several sources, where the compiler orders the waits well
 * by itself and the combination starts as the first loads arrive (dot product
 * of two 2^27-float vectors: 153.6 us without it, 158.3 with). */
static __device__ inline void rd_touch(const ga_float v) { asm volatile("" ::"v"(v)); }
static __device__ inline void rd_touch(const ga_double v) { asm volatile("" ::"v"(v)); }
template <typename T>
static __device__ inline void rd_touch(const T v) {
  if (sizeof(T) > 4) asm volatile("" ::"v"((ga_ulong)v));
  else asm volatile("" ::"v"((ga_uint)v));
}

/*@RD_GENERATED@*/

/* A NaN in the first position of a floating min/max scan stays (see the
 * header): `first` is the value at that position. */
#define RD_FIRST_RULE (RD_FLT && (RD_KIND == RD_K_MAX || RD_KIND == RD_K_MIN))
static __device__ inline rd_acc rd_first_rule(rd_acc a, const RD_ACC_T first) {
#if RD_FIRST_RULE
  if (first != first) {
    a.v = first;
#if RD_ARG
    a.i = 0;
#endif
  }
#else
  (void)first;
#endif
  return a;
}

/* Write the finished value(s) of one output. */
static __device__ inline void rd_write(rd_acc a, char *d0, ga_long d0o, char *d1, ga_long d1o) {
#if RD_HAS_D0
#if RD_DST_HALF
  *(ga_half *)(d0 + d0o) = ga_float2half((float)a.v);
#else
  *(RD_DST_T *)(d0 + d0o) = (RD_DST_T)a.v;
#endif
#else
  (void)d0; (void)d0o;
#endif
#if RD_HAS_D1
  *(RD_IDX_T *)(d1 + d1o) = (RD_IDX_T)a.i;
#else
  (void)d1; (void)d1o;
#endif
}

/* The same for a caller that does not hold the scan's first value: it is
 * fetched from the row again (one element per output; the short-row kernels,
 * where that would double the traffic, pass it from their registers). */
static __device__ inline void rd_store(rd_acc a, const char *const *srow, char *d0, ga_long d0o,
                                       char *d1, ga_long d1o, ga_long rtotal RD_SCALAR_FPARAMS) {
#if RD_FIRST_RULE
  if (rtotal > 0) {
    rd_one o;
    rd_one_load(o, srow);
    a = rd_first_rule(a, (RD_ACC_T)RD_ONE_VAL(o));
  }
#else
  (void)srow; (void)rtotal;
#endif
  rd_write(a, d0, d0o, d1, d1o);
}

/* The value the first-element rule looks at, for a caller that asks for it
 * early so that the load is back by the time the result is (a second pass
 * spends most of its few microseconds waiting for loads). */
static __device__ inline RD_ACC_T rd_first_value(const char *const *srow, ga_long rtotal RD_SCALAR_FPARAMS) {
#if RD_FIRST_RULE
  if (rtotal > 0) {
    rd_one o;
    rd_one_load(o, srow);
    return (RD_ACC_T)RD_ONE_VAL(o);
  }
#else
  (void)srow; (void)rtotal;
#endif
  return RD_NEUTRAL;   /* not a NaN: the rule leaves the result alone */
}

static __device__ inline void rd_store_partial(rd_acc a, RD_ACC_T *pv, ga_long *pi, ga_long slot) {
  pv[slot] = a.v;
#if RD_ARG
  pi[slot] = a.i;
#else
  (void)pi;
#endif
}

/* ---- a split reduction finished in the same launch ---------------------------
 * Every piece of an output leaves its partial and then counts itself in with
 * an atomic add on the output's counter; the piece that brings the count to
 * nsplit knows that all partials are there, reads them, combines them in slot
 * order - so the result does not depend on which piece came last - writes the
 * output and sets the counter back to zero for the next launch.  Nobody waits
 * for anybody.
 *
 * The partials travel as device-scope atomic stores and loads (they pass the
 * per-die L2 instead of resting in it), and a piece waits for its stores to
 * be acknowledged before it counts in.  A device-scope release / acquire fence
 * pair around plain stores and loads is the textbook form, but the release
 * writes back the whole L2 once per piece: with 512 pieces a sum of 2^24
 * floats went from 14.8 to 27 us.
 *
 * Launches that share the counters must not overlap (the library issues
 * everything on one in-order stream). */
template <typename T>
static __device__ inline void rd_coherent_store(T *p, const T v) {
  if (sizeof(T) == 8) {
    union { T t; ga_ulong u; } x;
    x.t = v;
    __hip_atomic_store((ga_ulong *)p, x.u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  } else {
    union { T t; ga_uint u; } x;
    x.u = 0;
    x.t = v;
    __hip_atomic_store((ga_uint *)p, x.u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}
template <typename T>
static __device__ inline T rd_coherent_load(const T *p) {
  if (sizeof(T) == 8) {
    union { T t; ga_ulong u; } x;
    x.u = __hip_atomic_load((const ga_ulong *)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return x.t;
  } else {
    union { T t; ga_uint u; } x;
    x.u = __hip_atomic_load((const ga_uint *)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return x.t;
  }
}
/* the host only asks for this path when the accumulator has 4 or 8 bytes */
static __device__ inline void rd_publish_partial(rd_acc a, RD_ACC_T *pv, ga_long *pi, ga_long slot) {
  rd_coherent_store(pv + slot, a.v);
#if RD_ARG
  rd_coherent_store(pi + slot, a.i);
#else
  (void)pi;
#endif
}
static __device__ inline rd_acc rd_fetch_partial(const RD_ACC_T *pv, const ga_long *pi, ga_long slot) {
  rd_acc t;
  t.v = rd_coherent_load(pv + slot);
#if RD_ARG
  t.i = rd_coherent_load(pi + slot);
#else
  (void)pi;
#endif
  return t;
}
/* The wavefront's stores have been acknowledged when this returns (a
 * device-scope store is acknowledged once it is past the L2), and the
 * compiler moves no memory access across either of the two. */
static __device__ inline void rd_stores_done() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
static __device__ inline void rd_before_loads() { asm volatile("" ::: "memory"); }
/* true for the caller that completes the count */
static __device__ inline bool rd_count_in(ga_uint *counter, ga_uint total) {
  const ga_uint before = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return before + 1u == total;
}
static __device__ inline void rd_count_reset(ga_uint *counter) {
  __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

/* ---- redux_row ------------------------------------------------------------- */

/* One "unit" = RD_U loads per lane over LN lanes (RD_G in redux_row, RD_L
 * in redux_wrows): elements
 * e0 + j*LN*RD_VEC + v of the inner reduced dim, j < RD_U, v < RD_VEC, where
 * e0 = (first element of the unit) + lane*RD_VEC.
 *
 * Combination of the lane's elements of one unit.  ib, rml: index of element
 * 0 of the inner dim and index step per element. */
#if RD_TAIL
/* elements a row starts before its first one, and the pointer moved back by that */
#define RD_SHIFT(ptr) ((ga_long)(((ga_size)(ptr) / RD_ELSZ0) % RD_VEC))
#else
#define RD_SHIFT(ptr) ((ga_long)0)
#endif

/* `rin` is the end of the row in the lane's coordinates (extent + sh), `sh`
 * its start (0 unless RD_TAIL). */
template <int LN>
static __device__ inline rd_acc rd_unit_combine(const rd_unit &x, ga_long e0, ga_long rin,
                                                ga_long ib, ga_long rml, ga_long sh RD_SCALAR_FPARAMS) {
  (void)sh;
#if RD_KIND == RD_K_MAX || RD_KIND == RD_K_MIN
#if RD_TAIL
  /* A unit that touches an end of the row: the lane's first valid element can
   * be anywhere.  No branch around a use of the loaded registers, here or
   * below: a path that skips every use leaves the loads pending at the loop's
   * back edge, and the next unit's loads then wait for one another. */
  if (e0 < sh || e0 + (ga_long)(RD_U - 1) * LN * RD_VEC + RD_VEC > rin) {
    RD_ACC_T bv = RD_NEUTRAL;
    ga_int bp = 0;
    bool found = false;
#pragma unroll
    for (int j = 0; j < RD_U; j++) {
      const ga_long e = e0 + (ga_long)j * LN * RD_VEC;
      const ga_long dl = sh - e, dh = rin - e;
      const int lo = dl > RD_VEC ? RD_VEC : (int)dl;
      const int hi = dh < 0 ? 0 : (dh > RD_VEC ? RD_VEC : (int)dh);
#pragma unroll
      for (int v = 0; v < RD_VEC; v++) {
        const bool valid = v >= lo && v < hi;
        const RD_ACC_T val = rd_elem(RD_UNIT_VAL(x, j, v), 0).v;
#if RD_KIND == RD_K_MAX
        const bool better = valid && (!found || val > bv);
#else
        const bool better = valid && (!found || val < bv);
#endif
        bv = better ? val : bv;
        bp = better ? (j * LN * RD_VEC + v) : bp;
        found = found || valid;
      }
    }
    rd_acc r = rd_neutral();
    r.v = found ? bv : r.v;
#if RD_ARG
    r.i = found ? ib + (e0 + bp - sh) * rml : r.i;
#else
    (void)ib; (void)rml;
#endif
    return r;
  }
#endif
  /* The lane's elements are visited in rising index order, so a strict
   * compare keeps the first of equals by itself; only the position inside
   * the unit (a small int) is tracked. */
  /* (with RD_TAIL only units wholly inside the row come here) */
  /* For one-byte elements with a position to track, RD_NCH scans run side by
   * side (elements v, v + RD_NCH, ... of every load), each in rising order, so
   * that one compare does not wait for the one before it; they meet at the
   * end, the lower position winning a tie (maxandargmax of 2^28 bytes 127 ->
   * 65 us).  Wider elements, and a plain integer max, which compiles to one
   * instruction per element, measured a few percent slower that way. */
#define RD_NCH ((RD_ARG && RD_ELSZ0 == 1 && RD_VEC >= 4) ? 4 : 1)
  RD_ACC_T cv[RD_NCH];
  ga_int cp[RD_NCH];
#pragma unroll
  for (int c = 0; c < RD_NCH; c++) {
    cv[c] = rd_elem(RD_UNIT_VAL(x, 0, c), 0).v;
    cp[c] = c;
  }
#pragma unroll
  for (int j = 0; j < RD_U; j++) {
    const bool in = RD_TAIL || e0 + (ga_long)j * LN * RD_VEC < rin;
#pragma unroll
    for (int v = 0; v < RD_VEC; v++) {
      if (j == 0 && v < RD_NCH) continue;
      const int c = v % RD_NCH;
      const RD_ACC_T val = rd_later(RD_UNIT_VAL(x, j, v));
#if RD_KIND == RD_K_MAX
      const bool better = in && val > cv[c];
#else
      const bool better = in && val < cv[c];
#endif
      cv[c] = better ? val : cv[c];
      cp[c] = better ? (j * LN * RD_VEC + v) : cp[c];
    }
  }
  RD_ACC_T bv = cv[0];
  ga_int bp = cp[0];
#pragma unroll
  for (int c = 1; c < RD_NCH; c++) {
#if RD_KIND == RD_K_MAX
    const bool better = cv[c] > bv || (cv[c] == bv && cp[c] < bp);
#else
    const bool better = cv[c] < bv || (cv[c] == bv && cp[c] < bp);
#endif
    bv = better ? cv[c] : bv;
    bp = better ? cp[c] : bp;
  }
#undef RD_NCH
  rd_acc r = rd_neutral();
  const bool any = RD_TAIL || e0 < rin;
  r.v = any ? bv : r.v;
#if RD_ARG
  r.i = any ? ib + (e0 + bp - sh) * rml : r.i;
#else
  (void)bp; (void)ib; (void)rml;
#endif
  return r;
#elif RD_FAST8
  /* One-byte elements, four per 32-bit operation.  `m` has 0xff in the bytes
   * of a word that hold elements of the row (every RD_ES-th byte; none past
   * the row's end; with RD_TAIL only those inside [sh, rin)).  Sum: a dot
   * product of the word's four bytes with the 0/1 bytes of m & 0x01010101,
   * accumulated in 32 bits over the unit (at most 8 loads x 16 bytes x 255).
   * Any: the valid bytes or-ed together.  All: a zero among the valid bytes
   * shows as (v - 0x01010101) & ~v & 0x80808080 with the other bytes forced
   * to 0xff. */
  (void)ib; (void)rml;
  const ga_uint every = RD_ES == 1 ? 0xffffffffu : (RD_ES == 2 ? 0x00ff00ffu : 0x000000ffu);
  ga_uint acc32 = 0;
#pragma unroll
  for (int j = 0; j < RD_U; j++) {
    const ga_long e = e0 + (ga_long)j * LN * RD_VEC;
#pragma unroll
    for (int d = 0; d < RD_PV / 4; d++) {
      const ga_uint wd = x.x0[j][d];   /* the unit keeps bytes packed in words */
      ga_uint m = e < rin ? every : 0u;
#if RD_TAIL
      {   /* elements 4d .. 4d+3 of the load (RD_ES is 1 here) */
        const ga_long first = e + 4 * d;
        const ga_long lo = sh - first, hi = rin - first;   /* valid: lo <= byte < hi */
        const ga_uint below = lo <= 0 ? 0u : (lo >= 4 ? 0xffffffffu : (1u << (8 * (int)lo)) - 1u);
        const ga_uint upto = hi <= 0 ? 0u : (hi >= 4 ? 0xffffffffu : (1u << (8 * (int)hi)) - 1u);
        m = upto & ~below;
      }
#endif
#if RD_KIND == RD_K_SUM
#if RD_FAST8 == 2
      acc32 = (ga_uint)__builtin_amdgcn_sdot4((int)wd, (int)(m & 0x01010101u), (int)acc32, false);
#else
      acc32 = __builtin_amdgcn_udot4(wd, m & 0x01010101u, acc32, false);
#endif
#elif RD_KIND == RD_K_ANY
      acc32 |= wd & m;
#else
      const ga_uint v = wd | ~m;
      acc32 |= (v - 0x01010101u) & ~v & 0x80808080u;
#endif
    }
  }
  rd_acc r;
#if RD_KIND == RD_K_SUM
#if RD_FAST8 == 2
  r.v = (RD_ACC_T)(ga_int)acc32;
#else
  r.v = (RD_ACC_T)acc32;
#endif
#elif RD_KIND == RD_K_ANY
  r.v = acc32 != 0 ? 1 : 0;
#else
  r.v = acc32 == 0 ? 1 : 0;
#endif
  return r;
#else
  rd_acc t[RD_U];
#pragma unroll
  for (int j = 0; j < RD_U; j++) {
    const ga_long e = e0 + (ga_long)j * LN * RD_VEC;
    t[j] = rd_neutral();
#if RD_TAIL
    /* every element under a select, no branch (see above; a branch that sends
     * the lanes whose loads lie inside the row past the selects saved half a
     * microsecond of 46 on rows of 50257 floats and cost a few hundred rows of
     * a hundred floats as much of 4) */
    const ga_long dl = sh - e, dh = rin - e;
    const int lo = dl > RD_VEC ? RD_VEC : (int)dl;
    const int hi = dh < 0 ? 0 : (dh > RD_VEC ? RD_VEC : (int)dh);
#pragma unroll
    for (int v = 0; v < RD_VEC; v++) {
      const rd_acc c = rd_combine(t[j], rd_elem(RD_UNIT_VAL(x, j, v), ib + (e + v - sh) * rml));
      t[j] = (v >= lo && v < hi) ? c : t[j];
    }
#else
    if (e < rin) {
#pragma unroll
      for (int v = 0; v < RD_VEC; v++)
        t[j] = rd_combine(t[j], rd_elem(RD_UNIT_VAL(x, j, v), ib + (e + v - sh) * rml));
    }
#endif
  }
  /* pairwise over the unit */
#pragma unroll
  for (int w = 1; w < RD_U; w *= 2)
#pragma unroll
    for (int j = 0; j + w < RD_U; j += 2 * w) t[j] = rd_combine(t[j], t[j + w]);
  return t[0];
#endif
}

#if RD_WANT & 1   /* redux_row */
KERNEL void __launch_bounds__(256)
redux_row(RD_SRC_PARAMS, char *__restrict__ d0, const ga_size d0_off, char *__restrict__ d1,
          const ga_size d1_off, RD_ACC_T *__restrict__ part_v, ga_long *__restrict__ part_i, ga_uint *done,
          const rd_plan p RD_SCALAR_PARAMS) {
  const unsigned rows_per_group = 256u / RD_G;
  const unsigned lane = LID_0 % RD_G;
  const ga_long split = GID_0 % (unsigned)p.nsplit;
  const ga_long row = (ga_long)(GID_0 / (unsigned)p.nsplit) * rows_per_group + LID_0 / RD_G;
#if RD_G == 256
  __shared__ rd_acc lds[4];
#endif
  if (row >= p.nrows) return;   /* uniform per wavefront; per group when RD_G == 256 */

  const int ri = p.nr - 1;                 /* inner reduced dim */
  const ga_long rin = p.nr > 0 ? p.rdim[ri] : 1;
  const ga_long rml = p.nr > 0 ? p.rmul[ri] : 0;
  const ga_long seg = (ga_long)RD_G * RD_VEC * RD_U;

  ga_long so[RD_NSRC], d0o, d1o, rstr[RD_NSRC];
  rd_row_offsets(p, row, so, &d0o, &d1o);
  const char *srow[RD_NSRC];
  RD_SRC_BASES(srow);
#pragma unroll
  for (int k = 0; k < RD_NSRC; k++) {
    srow[k] += so[k];
    rstr[k] = p.nr > 0 ? p.rsstr[k][ri] : 0;
  }

  /* what the first-element rule looks at, asked for now and used at the end */
  RD_ACC_T first = RD_NEUTRAL;
  if (lane == 0) first = rd_first_value(srow, p.rtotal RD_SCALAR_ARGS);

  /* A split owns a contiguous range of units, or - for a single reduced dim
   * (RD_INTERLEAVE) - every nsplit-th unit, so that at any moment the splits
   * of a row read one moving window of memory. */
#if RD_INTERLEAVE
  ga_long u0 = split, u1 = p.units;
  const ga_long ustep = p.nsplit;
#else
  ga_long u0 = split * p.upb, u1 = u0 + p.upb;
  if (u1 > p.units) u1 = p.units;
  const ga_long ustep = 1;
#endif

#if RD_LO > 1
  /* The inner reduced dim is short: RD_G / RD_LO lanes cover it and RD_LO
   * outer reduced coordinates sit side by side; unit u holds the outer
   * coordinates u*RD_LO .. u*RD_LO + RD_LO - 1. */
  const unsigned li = lane % (RD_G / RD_LO), lo = lane / (RD_G / RD_LO);
  const ga_long e0 = (ga_long)li * RD_VEC;
  rd_acc acc = rd_neutral();
  for (ga_long u = u0; u < u1; u += ustep) {
    const ga_long ro = u * RD_LO + lo;
    if (ro < p.router) {
      ga_long rb[RD_NSRC], ib = 0;
      rd_outer_offsets(p, ri, ro, rb, &ib);
      rd_unit x;
      const char *ub[RD_NSRC];
#pragma unroll
      for (int s = 0; s < RD_NSRC; s++) ub[s] = srow[s] + rb[s];
      const ga_long sh = RD_SHIFT(ub[0]);
      ub[0] -= sh * RD_ELSZ0;
      rd_unit_load<RD_G / RD_LO>(x, ub, e0, rin + sh, rstr);
#if RD_TOUCH_ROW
      rd_unit_touch(x);
#endif
      acc = rd_combine(acc, rd_unit_combine<RD_G / RD_LO>(x, e0, rin + sh, ib, rml, sh RD_SCALAR_ARGS));
    }
  }
  (void)seg;
#else
  /* unit -> (outer reduced coordinate ro, segment k of the inner dim): one
   * division for the first unit, then counted up */
  ga_long ro = 0, k = u0;
  if (p.nr > 1) { ro = rd_divmod(u0, p.nseg, &k); }
  ga_long rb[RD_NSRC], ib = 0;
  rd_outer_offsets(p, ri, ro, rb, &ib);

  rd_acc acc = rd_neutral();
  for (ga_long u = u0; u < u1; u += ustep) {
    const ga_long e0 = k * seg + (ga_long)lane * RD_VEC;
    rd_unit x;
    const char *ub[RD_NSRC];
#pragma unroll
    for (int s = 0; s < RD_NSRC; s++) ub[s] = srow[s] + rb[s];
    const ga_long sh = RD_SHIFT(ub[0]);
    ub[0] -= sh * RD_ELSZ0;
    rd_unit_load<RD_G>(x, ub, e0, rin + sh, rstr);
#if RD_TOUCH_ROW
    rd_unit_touch(x);
#endif
    acc = rd_combine(acc, rd_unit_combine<RD_G>(x, e0, rin + sh, ib, rml, sh RD_SCALAR_ARGS));
#if RD_INTERLEAVE
    k += ustep;   /* single reduced dim: the unit is the segment */
#else
    if (++k == p.nseg) {
      k = 0;
      ro++;
      rd_outer_offsets(p, ri, ro, rb, &ib);
    }
#endif
  }

#endif

#if RD_G == 256
  acc = rd_block_reduce(acc, lds);
#else
  acc = rd_wave_reduce(acc);
#endif
  if (lane == 0) {
    if (p.nsplit == 1)
      rd_write(rd_first_rule(acc, first), d0 + d0_off, d0o, d1 + d1_off, d1o);
    else if (p.fused)
      rd_publish_partial(acc, part_v, part_i, row * p.nsplit + split);
    else
      rd_store_partial(acc, part_v, part_i, row * p.nsplit + split);
  }
  if (p.nsplit > 1 && p.fused) {
    /* uniform over the lanes that share the row: the group (RD_G == 256) or the wavefront */
#if RD_G == 256
    __shared__ ga_uint last_piece;
    if (lane == 0) {
      rd_stores_done();
      last_piece = rd_count_in(done + row, (ga_uint)p.nsplit) ? 1u : 0u;
    }
    local_barrier();
    if (!last_piece) return;
#else
    ga_uint last_piece = 0;
    if (lane == 0) {
      rd_stores_done();
      last_piece = rd_count_in(done + row, (ga_uint)p.nsplit) ? 1u : 0u;
    }
    if (!__builtin_amdgcn_readfirstlane(last_piece)) return;
#endif
    rd_before_loads();
    rd_acc all = rd_neutral();
    for (ga_long s = lane; s < p.nsplit; s += RD_G)
      all = rd_combine(all, rd_fetch_partial(part_v, part_i, row * p.nsplit + s));
#if RD_G == 256
    all = rd_block_reduce(all, lds);
#else
    all = rd_wave_reduce(all);
#endif
    if (lane == 0) {
      rd_write(rd_first_rule(all, first), d0 + d0_off, d0o, d1 + d1_off, d1o);
      rd_count_reset(done + row);
    }
  }
}

#endif   /* RD_WANT & 1 */

#if RD_WANT & 4
/* ---- redux_wrows -----------------------------------------------------------
 * Rows that one pass of a wavefront covers (at most one reduced dim, one
 * unit per row, no split).  Wavefront w owns rows [w*upb, (w+1)*upb) and takes
 * them RD_RB at a time: the loads of the whole batch are issued before the
 * first row is combined, so a wavefront whose row is a single load per lane
 * still has RD_RB loads in flight.  Only built for RD_G == 64. */
#if RD_G == 64
#if RD_RB == 1 && RD_L == 64 && !RD_TAIL
/* one row at a time; with upb > 1 the next row's loads are issued before the
 * current row is combined */
KERNEL void __launch_bounds__(256)
redux_wrows(RD_SRC_PARAMS, char *__restrict__ d0, const ga_size d0_off, char *__restrict__ d1,
            const ga_size d1_off, RD_ACC_T *__restrict__ part_v, ga_long *__restrict__ part_i, ga_uint *done,
            const rd_plan p RD_SCALAR_PARAMS) {
  (void)part_v; (void)part_i; (void)done;
  const unsigned lane = LID_0 & 63u;
  const ga_long wave = (ga_long)GID_0 * 4 + (LID_0 >> 6);
  ga_long row = wave * p.upb;
  ga_long row_end = row + p.upb;
  if (row_end > p.nrows) row_end = p.nrows;
  if (row >= row_end) return;

  const ga_long rin = p.nr > 0 ? p.rdim[0] : 1;
  const ga_long rml = p.nr > 0 ? p.rmul[0] : 0;
  const ga_long e0 = (ga_long)lane * RD_VEC;
  ga_long rstr[RD_NSRC];
  const char *base[RD_NSRC];
  RD_SRC_BASES(base);
#pragma unroll
  for (int k = 0; k < RD_NSRC; k++) rstr[k] = p.nr > 0 ? p.rsstr[k][0] : 0;

  ga_long so[RD_NSRC], d0o, d1o;
  const char *srow[RD_NSRC];
  rd_row_offsets(p, row, so, &d0o, &d1o);
#pragma unroll
  for (int k = 0; k < RD_NSRC; k++) srow[k] = base[k] + so[k];
  rd_unit cur;
  rd_unit_load<64>(cur, srow, e0, rin, rstr);
  for (; row < row_end; row++) {
    ga_long nso[RD_NSRC], nd0o = 0, nd1o = 0;
    const char *nrow[RD_NSRC];
    rd_unit nxt;
    if (row + 1 < row_end) {
      rd_row_offsets(p, row + 1, nso, &nd0o, &nd1o);
#pragma unroll
      for (int k = 0; k < RD_NSRC; k++) nrow[k] = base[k] + nso[k];
      rd_unit_load<64>(nxt, nrow, e0, rin, rstr);
    }
    rd_acc acc = rd_wave_reduce(rd_unit_combine<64>(cur, e0, rin, 0, rml, 0 RD_SCALAR_ARGS));
    if (lane == 0)   /* which also holds the row's first element */
      rd_write(rd_first_rule(acc, (RD_ACC_T)RD_UNIT_VAL(cur, 0, 0)), d0 + d0_off, d0o, d1 + d1_off, d1o);
    cur = nxt;
#pragma unroll
    for (int k = 0; k < RD_NSRC; k++) srow[k] = nrow[k];
    d0o = nd0o; d1o = nd1o;
  }
}
#else
/* RD_L lanes per row, 64 / RD_L rows side by side in a wavefront, RD_RB such
 * sets per batch.  Every lane computes (a lane whose row is past the end
 * works on the last row and does not store), so the cross-lane steps never
 * see a disabled lane. */
KERNEL void __launch_bounds__(256)
redux_wrows(RD_SRC_PARAMS, char *__restrict__ d0, const ga_size d0_off, char *__restrict__ d1,
            const ga_size d1_off, RD_ACC_T *__restrict__ part_v, ga_long *__restrict__ part_i, ga_uint *done,
            const rd_plan p RD_SCALAR_PARAMS) {
  (void)part_v; (void)part_i; (void)done;
  const unsigned lane = LID_0 & 63u;
  const unsigned sub = lane / RD_L, l = lane % RD_L;
  const ga_long wave = (ga_long)GID_0 * 4 + (LID_0 >> 6);
  ga_long row0 = wave * p.upb;
  ga_long row_end = row0 + p.upb;
  if (row_end > p.nrows) row_end = p.nrows;
  if (row0 >= row_end) return;

  const ga_long rin = p.nr > 0 ? p.rdim[0] : 1;
  const ga_long rml = p.nr > 0 ? p.rmul[0] : 0;
  const ga_long e0 = (ga_long)l * RD_VEC;
  ga_long rstr[RD_NSRC];
  const char *base[RD_NSRC];
  RD_SRC_BASES(base);
#pragma unroll
  for (int k = 0; k < RD_NSRC; k++) rstr[k] = p.nr > 0 ? p.rsstr[k][0] : 0;

  for (; row0 < row_end; row0 += (64 / RD_L) * RD_RB) {
    rd_unit x[RD_RB];
    ga_long d0o[RD_RB], d1o[RD_RB], sh[RD_RB];
#pragma unroll
    for (int b = 0; b < RD_RB; b++) {
      ga_long row = row0 + b * (64 / RD_L) + sub;
      if (row >= row_end) row = row_end - 1;
      ga_long so[RD_NSRC];
      rd_row_offsets(p, row, so, &d0o[b], &d1o[b]);
      const char *lp[RD_NSRC];
#pragma unroll
      for (int k = 0; k < RD_NSRC; k++) lp[k] = base[k] + so[k];
      sh[b] = RD_SHIFT(lp[0]);
      lp[0] -= sh[b] * RD_ELSZ0;
      rd_unit_load<RD_L>(x[b], lp, e0, rin + sh[b], rstr);
    }
#pragma unroll
    for (int b = RD_RB - 1; b >= 0; b--) rd_unit_touch(x[b]);
#pragma unroll
    for (int b = 0; b < RD_RB; b++) {
      const ga_long row = row0 + b * (64 / RD_L) + sub;
      rd_acc acc = rd_seg_reduce<RD_L>(
          rd_unit_combine<RD_L>(x[b], e0, rin + sh[b], 0, rml, sh[b] RD_SCALAR_ARGS));
#if RD_FIRST_RULE
      /* Lane 0 of the row holds its first element (at position sh of its first
       * load).  Where that is a NaN this lane writes the result itself, and
       * the last lane, which holds the combination, stands back. */
      RD_ACC_T first = (RD_ACC_T)RD_UNIT_VAL(x[b], 0, 0);
#if RD_TAIL
#pragma unroll
      for (int v = 1; v < RD_VEC; v++)
        if (sh[b] == v) first = (RD_ACC_T)RD_UNIT_VAL(x[b], 0, v);
#endif
      const bool first_nan = l == 0 && first != first;
      const ga_ulong nan_rows = __builtin_amdgcn_ballot_w64(first_nan);
      if (first_nan && row < row_end)
        rd_write(rd_first_rule(acc, first), d0 + d0_off, d0o[b], d1 + d1_off, d1o[b]);
      if (l == RD_L - 1 && row < row_end && !((nan_rows >> (lane - l)) & 1u))
        rd_write(acc, d0 + d0_off, d0o[b], d1 + d1_off, d1o[b]);
#else
      if (l == RD_L - 1 && row < row_end)
        rd_write(acc, d0 + d0_off, d0o[b], d1 + d1_off, d1o[b]);
#endif
    }
  }
}
#endif
#endif

#endif   /* RD_WANT & 4 */

#if RD_SROWS
/* ---- redux_srows -----------------------------------------------------------
 * Rows of a few dozen elements, one after the other in memory (one source,
 * one reduced dim, unit stride, row pitch = row length).  redux_wrows spends
 * its time on instructions per row there - address arithmetic, masks and
 * cross-lane steps for a handful of elements.  Here a group copies the
 * contiguous bytes of its p.upb <= 256 rows into LDS with 16-byte streaming
 * loads (from the 16-byte boundary at or below the first row), and after one
 * barrier lane t walks row t out of LDS: no cross-lane step, and per element
 * one LDS read and the combine.  A lane starts t elements into its row when the
 * row length is even, so that the lanes of a wavefront spread over the banks. */
typedef ga_uint rd_chunk_t __attribute__((ext_vector_type(4)));

KERNEL void __launch_bounds__(256)
redux_srows(RD_SRC_PARAMS, char *__restrict__ d0, const ga_size d0_off, char *__restrict__ d1,
            const ga_size d1_off, RD_ACC_T *__restrict__ part_v, ga_long *__restrict__ part_i, ga_uint *done,
            const rd_plan p RD_SCALAR_PARAMS) {
  (void)part_v; (void)part_i; (void)done;
  extern __shared__ rd_chunk_t rd_staged[];
  const ga_long per_group = p.upb;
  const ga_long row0 = (ga_long)GID_0 * per_group;
  ga_long nrow = p.nrows - row0;
  if (nrow > per_group) nrow = per_group;
  const ga_long rin = p.rdim[0], rml = p.rmul[0];

  const char *base[RD_NSRC];
  RD_SRC_BASES(base);
  const char *begin = base[0] + row0 * p.fsstr[0][0];
  const ga_size sh = (ga_size)begin & 15u;
  const char *from = begin - sh;
  const ga_long chunks = ((ga_long)sh + nrow * rin * RD_ELSZ0 + 15) >> 4;

  for (ga_long c0 = LID_0; c0 < chunks; c0 += 256 * 8) {
    rd_chunk_t t[8];
#pragma unroll
    for (int j = 0; j < 8; j++)
      if (c0 + j * 256 < chunks) t[j] = RD_LOAD((const rd_chunk_t *)(from + (c0 + j * 256) * 16));
#pragma unroll
    for (int j = 7; j >= 0; j--) rd_touch(t[j][0]);
#pragma unroll
    for (int j = 0; j < 8; j++)
      if (c0 + j * 256 < chunks) rd_staged[c0 + j * 256] = t[j];
  }
  local_barrier();

  if ((ga_long)LID_0 < nrow) {
    typedef decltype(rd_one::x0) elem_t;
    const elem_t *e = (const elem_t *)((const char *)rd_staged + sh) + (ga_long)LID_0 * rin;
    const ga_int n = (ga_int)rin;
    rd_acc acc = rd_neutral();
#if RD_ARG && (RD_KIND == RD_K_MAX || RD_KIND == RD_K_MIN)
    /* value and position inside the row (32 bits) while walking; the 64-bit
     * index is formed once at the end */
#if RD_KIND == RD_K_MAX
#define RD_SR_BETTER(x, y) ((x) > (y))
#else
#define RD_SR_BETTER(x, y) ((x) < (y))
#endif
    RD_ACC_T bv;
    ga_int bp;
    if (n & 1) {
      /* rising positions: a strict compare keeps the first of equals */
      rd_one o;
      o.x0 = e[0];
      bv = rd_elem(RD_ONE_VAL(o), 0).v;
      bp = 0;
#pragma unroll 4
      for (ga_int i = 1; i < n; i++) {
        o.x0 = e[i];
        const RD_ACC_T val = rd_later(RD_ONE_VAL(o));
        const bool better = RD_SR_BETTER(val, bv);
        bv = better ? val : bv;
        bp = better ? i : bp;
      }
    } else {
      ga_int pos = (ga_int)(LID_0 % (unsigned)n);
      bv = RD_NEUTRAL;
      bp = 0x7fffffff;
#pragma unroll 4
      for (ga_int i = 0; i < n; i++) {
        rd_one o;
        o.x0 = e[pos];
        const RD_ACC_T val = rd_later(RD_ONE_VAL(o));
        const bool better = RD_SR_BETTER(val, bv) || (val == bv && pos < bp);
        bv = better ? val : bv;
        bp = better ? pos : bp;
        pos = (pos + 1 == n) ? 0 : pos + 1;
      }
    }
#undef RD_SR_BETTER
    acc.v = bv;
    acc.i = (ga_long)bp * rml;
#else
    ga_int pos = (n & 1) ? 0 : (ga_int)(LID_0 % (unsigned)n);
#pragma unroll 4
    for (ga_int i = 0; i < n; i++) {
      rd_one o;
      o.x0 = e[pos];
      acc = rd_combine(acc, rd_elem(RD_ONE_VAL(o), (ga_long)pos * rml));
      pos = (pos + 1 == n) ? 0 : pos + 1;
    }
#endif
    ga_long so[RD_NSRC], d0o, d1o;
    rd_row_offsets(p, row0 + LID_0, so, &d0o, &d1o);
    rd_one first;
    first.x0 = e[0];
    rd_write(rd_first_rule(acc, (RD_ACC_T)RD_ONE_VAL(first)), d0 + d0_off, d0o, d1 + d1_off, d1o);
  }
}
#endif

#if RD_TROWS
/* ---- redux_trows -----------------------------------------------------------
 * Rows of RD_TE elements, at most 32 bytes, one after the other in memory (one
 * source, one reduced dim, unit stride, row pitch = row length, first row on
 * a 16-byte boundary).  There the time goes into instructions per row, not
 * into bytes.  A lane takes the least run of whole rows that is a whole number
 * of 16-byte chunks - RD_TR rows in RD_TC chunks, both fixed when the kernel
 * is built - into registers and walks its rows there: every element position
 * is a constant, no cross-lane step, no LDS. */
#endif   /* RD_TROWS */
#if RD_TROWS || RD_PCOLS
/* elements out of 16-byte chunks held in registers (redux_trows, redux_pcols) */
typedef ga_uint rd_tchunk_t __attribute__((ext_vector_type(4)));

template <int ES> struct rd_tbits;
template <> struct rd_tbits<1> {
  static __device__ inline ga_ulong at(const rd_tchunk_t *c, const int b) {
    return (c[b >> 4][(b >> 2) & 3] >> ((b & 3) * 8)) & 0xffu;
  }
};
template <> struct rd_tbits<2> {
  static __device__ inline ga_ulong at(const rd_tchunk_t *c, const int b) {
    return (c[b >> 4][(b >> 2) & 3] >> ((b & 2) * 8)) & 0xffffu;
  }
};
template <> struct rd_tbits<4> {
  static __device__ inline ga_ulong at(const rd_tchunk_t *c, const int b) { return c[b >> 4][(b >> 2) & 3]; }
};
template <> struct rd_tbits<8> {
  static __device__ inline ga_ulong at(const rd_tchunk_t *c, const int b) {
    return (ga_ulong)c[b >> 4][(b >> 2) & 3] | ((ga_ulong)c[b >> 4][((b >> 2) & 3) + 1] << 32);
  }
};

/* element e of the lane's registers as a one-element fetch */
static __device__ inline rd_one rd_trow_elem(const rd_tchunk_t *c, const int e) {
  typedef decltype(rd_one::x0) elem_t;
  const ga_ulong bits = rd_tbits<RD_ELSZ0>::at(c, e * RD_ELSZ0);
  rd_one o;
  __builtin_memcpy(&o.x0, &bits, sizeof(elem_t));
  return o;
}

#endif   /* RD_TROWS || RD_PCOLS */
#if RD_TROWS
#define RD_TROW_BYTES (RD_TE * RD_ELSZ0)

/* A lane's RD_TR results side by side, for the case that they lie so in
 * memory: up to 16 bytes go out as one store per lane; a longer run is handed
 * back through LDS so that the wavefront's stores are 16 bytes per lane side
 * by side again (a lane storing its own 64 bytes in four pieces would leave
 * every store instruction with 64 pieces 64 bytes apart). */
#if RD_HAS_D0 && RD_DST_HALF
typedef ga_half rd_tdst_t;
#elif RD_HAS_D0
typedef RD_DST_T rd_tdst_t;
#else
typedef ga_int rd_tdst_t;
#endif
template <typename T> struct __attribute__((aligned(sizeof(T) * RD_TR > 16 ? 16 : sizeof(T) * RD_TR))) rd_trun {
  T e[RD_TR];
};
constexpr int rd_trun0 = RD_HAS_D0 ? (int)sizeof(rd_trun<rd_tdst_t>) : 0;
constexpr int rd_trun1 = RD_HAS_D1 ? (int)sizeof(rd_trun<RD_IDX_T>) : 0;
constexpr int rd_tmax(const int a, const int b) { return a > b ? a : b; }
/* 16-byte chunks of LDS per lane: the loads' hand-out and the longer runs */
constexpr int rd_tlds = rd_tmax(RD_TC > 2 ? RD_TC : 0,
                                rd_tmax(rd_trun0 > 16 ? rd_trun0 / 16 : 0, rd_trun1 > 16 ? rd_trun1 / 16 : 0));

static __device__ inline void rd_twave_sync() {
  /* LDS operations of one wavefront run in the order they were issued; this
   * keeps the compiler from moving them across */
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

/* `dst`: where the wavefront's first result goes; `area`: its 64 * rd_tlds chunks of LDS */
template <typename RUN>
static __device__ inline void rd_twave_store(char *dst, const RUN &o, rd_tchunk_t *area, const unsigned lane) {
  ((RUN *)area)[lane] = o;
  rd_twave_sync();
#pragma unroll
  for (int k = 0; k < (int)sizeof(RUN) / 16; k++) ((rd_tchunk_t *)dst)[k * 64 + lane] = area[k * 64 + lane];
  rd_twave_sync();
}

KERNEL void __launch_bounds__(256)
redux_trows(RD_SRC_PARAMS, char *__restrict__ d0, const ga_size d0_off, char *__restrict__ d1,
            const ga_size d1_off, RD_ACC_T *__restrict__ part_v, ga_long *__restrict__ part_i, ga_uint *done,
            const rd_plan p RD_SCALAR_PARAMS) {
  (void)part_v; (void)part_i; (void)done;
  __shared__ rd_tchunk_t rd_tstage[256 * (rd_tlds ? rd_tlds : 1)];
  const ga_long unit = (ga_long)GID_0 * 256 + LID_0;
  const ga_long row0 = unit * RD_TR;
  const ga_long rml = p.rmul[0];
  const unsigned lane = LID_0 & 63u;
  rd_tchunk_t *area = rd_tstage + (LID_0 - lane) * rd_tlds;   /* the wavefront's own part */
  const char *base[RD_NSRC];
  RD_SRC_BASES(base);
  const rd_tchunk_t *src = (const rd_tchunk_t *)base[0];
  /* chunks that hold part of the array: the last lanes' runs may end past it */
  const ga_long total = (p.nrows * RD_TROW_BYTES + 15) >> 4;
  rd_tchunk_t c[RD_TC];
#if RD_TC > 2
  /* A lane's chunks lie RD_TC * 16 bytes from its neighbour's: fetched by the
   * lane itself, every load of a wavefront would touch 64 separate pieces of
   * memory.  The wavefront fetches its RD_TC * 64 chunks side by side
   * instead and hands them out through LDS. */
  {
    const ga_long cw = (unit - lane) * RD_TC;   /* the wavefront's first chunk */
    rd_tchunk_t t[RD_TC];
#pragma unroll
    for (int j = 0; j < RD_TC; j++) {
      const ga_long ci = cw + j * 64 + lane;
      if (ci < total) t[j] = RD_LOAD(src + ci);
      else t[j] = (rd_tchunk_t)(0u);
    }
#pragma unroll
    for (int j = 0; j < RD_TC; j++) area[j * 64 + lane] = t[j];
    rd_twave_sync();
#pragma unroll
    for (int j = 0; j < RD_TC; j++) c[j] = area[lane * RD_TC + j];
    rd_twave_sync();
  }
#else
#pragma unroll
  for (int j = 0; j < RD_TC; j++) {
    if (unit * RD_TC + j < total) c[j] = RD_LOAD(src + unit * RD_TC + j);
    else c[j] = (rd_tchunk_t)(0u);
  }
#endif
  if (row0 >= p.nrows) return;

  rd_acc res[RD_TR];
#pragma unroll
  for (int r = 0; r < RD_TR; r++) {
    rd_acc acc = rd_neutral();
#if RD_ARG && (RD_KIND == RD_K_MAX || RD_KIND == RD_K_MIN)
    /* value and position inside the row while walking up the row (a strict
     * compare keeps the first of equals); the index is formed at the end */
    RD_ACC_T bv = rd_elem(RD_ONE_VAL(rd_trow_elem(c, r * RD_TE)), 0).v;
    ga_int bp = 0;
#pragma unroll
    for (int i = 1; i < RD_TE; i++) {
      const RD_ACC_T val = rd_later(RD_ONE_VAL(rd_trow_elem(c, r * RD_TE + i)));
#if RD_KIND == RD_K_MAX
      const bool better = val > bv;
#else
      const bool better = val < bv;
#endif
      bv = better ? val : bv;
      bp = better ? i : bp;
    }
    acc.v = bv;
    acc.i = (ga_long)bp * rml;
#else
#pragma unroll
    for (int i = 0; i < RD_TE; i++)
      acc = rd_combine(acc, rd_elem(RD_ONE_VAL(rd_trow_elem(c, r * RD_TE + i)), (ga_long)i * rml));
#endif
    res[r] = rd_first_rule(acc, (RD_ACC_T)RD_ONE_VAL(rd_trow_elem(c, r * RD_TE)));
  }

  /* p.upb bit 0 / 1: the values / the indices of a lane's rows lie side by
   * side in memory, the first of them on the boundary of one store.  A lane
   * whose run is cut short by the end of the array, and for the longer runs
   * every lane of that last wavefront, writes row by row. */
  const bool whole = row0 + RD_TR <= p.nrows;
  const ga_long wrow0 = (unit - lane) * RD_TR;
  const bool wave_whole = wrow0 + 64 * RD_TR <= p.nrows;
  (void)wave_whole; (void)area;
  bool v_done = !RD_HAS_D0, i_done = !RD_HAS_D1;
#if RD_HAS_D0
  if (p.upb & 1) {
    rd_trun<rd_tdst_t> o;
#pragma unroll
    for (int r = 0; r < RD_TR; r++) {
#if RD_DST_HALF
      o.e[r] = ga_float2half((float)res[r].v);
#else
      o.e[r] = (RD_DST_T)res[r].v;
#endif
    }
    if constexpr (rd_trun0 > 16) {
      if (wave_whole) {
        rd_twave_store(d0 + d0_off + wrow0 * (ga_long)sizeof(rd_tdst_t), o, area, lane);
        v_done = true;
      }
    } else if (whole) {
      *(rd_trun<rd_tdst_t> *)(d0 + d0_off + row0 * (ga_long)sizeof(rd_tdst_t)) = o;
      v_done = true;
    }
  }
#endif
#if RD_HAS_D1
  if (p.upb & 2) {
    rd_trun<RD_IDX_T> o;
#pragma unroll
    for (int r = 0; r < RD_TR; r++) o.e[r] = (RD_IDX_T)res[r].i;
    if constexpr (rd_trun1 > 16) {
      if (wave_whole) {
        rd_twave_store(d1 + d1_off + wrow0 * (ga_long)sizeof(RD_IDX_T), o, area, lane);
        i_done = true;
      }
    } else if (whole) {
      *(rd_trun<RD_IDX_T> *)(d1 + d1_off + row0 * (ga_long)sizeof(RD_IDX_T)) = o;
      i_done = true;
    }
  }
#endif
  if (v_done && i_done) return;
#pragma unroll
  for (int r = 0; r < RD_TR; r++) {
    const ga_long row = row0 + r;
    if (row < p.nrows) {
      ga_long so[RD_NSRC], d0o, d1o;
      rd_row_offsets(p, row, so, &d0o, &d1o);
#if RD_HAS_D0
      if (!v_done) {
#if RD_DST_HALF
        *(ga_half *)(d0 + d0_off + d0o) = ga_float2half((float)res[r].v);
#else
        *(RD_DST_T *)(d0 + d0_off + d0o) = (RD_DST_T)res[r].v;
#endif
      }
#endif
#if RD_HAS_D1
      if (!i_done) *(RD_IDX_T *)(d1 + d1_off + d1o) = (RD_IDX_T)res[r].i;
#endif
    }
  }
}
#endif   /* RD_TROWS */

#if RD_PCOLS
/* ---- redux_pcols -----------------------------------------------------------
 * Reducing the leading dims of a dense array whose kept rows are short - the
 * sum over a batch of rows of 10 floats: p.nrows outputs (the kept row, F
 * elements), p.rtotal rows, all F * rtotal elements one after the other in
 * memory, the first on a 16-byte boundary (one source).  The array is walked
 * as one run of 16-byte chunks, like a full reduction; which output an
 * element belongs to is its position modulo F.  L = p.upb lanes of a group
 * are active, L chosen so that L chunks hold a whole number of kept rows:
 * the lane's next chunk, L further on, then holds the same outputs at the
 * same places, and a lane keeps one accumulator per element of a chunk
 * without ever computing a position.  Group g owns the chunks from g L J on
 * (J = p.units chunks per lane).  At the end the L * 16 / size accumulators
 * of a group meet in LDS, F of them come out per group, and the group that
 * counts in last (p.nsplit groups, one counter) combines the groups'
 * partials and writes the outputs: one launch.  For operations whose result
 * does not depend on how the elements are grouped.
 * With p.router > 1 the source is that many such arrays one behind the other
 * (slabs: a middle run of reduced dims under kept ones), whole chunks each;
 * with one group per slab (p.nsplit == 1) a group's F values are the slab's
 * outputs, and nothing is left or counted. */
#define RD_PVN (16 / RD_ELSZ0)
static __device__ inline rd_acc rd_pacc(const RD_ACC_T v) {
  rd_acc a = rd_neutral();
  a.v = v;
  return a;
}

/* The L * RD_PVN (or nsplit * F) values at stage[i * F + k] combined per
 * column k: lane t < S F takes column t mod F and every S-th copy, S = 256 / F
 * lane subsets, which then meet; with more than 256 columns a lane walks its
 * columns alone.  `out(k, a)` receives each column once. */
template <typename FETCH, typename OUT>
static __device__ inline void rd_pcols_fold(const unsigned F, const unsigned copies, RD_ACC_T *meet,
                                            FETCH fetch, OUT out) {
  if (F <= 256u) {
    const unsigned S = 256u / F, s = LID_0 / F, k = LID_0 - s * F;
    rd_acc a = rd_neutral();
    if (s < S) {
      /* eight fetches go out before the first is combined: one at a time each
       * would wait for the one before it */
      unsigned i = s;
      for (; i + 7 * S < copies; i += 8 * S) {
        RD_ACC_T t[8];
#pragma unroll
        for (int j = 0; j < 8; j++) t[j] = fetch((i + j * S) * F + k);
#pragma unroll
        for (int j = 0; j < 8; j++) a = rd_combine(a, rd_pacc(t[j]));
      }
      for (; i < copies; i += S) a = rd_combine(a, rd_pacc(fetch(i * F + k)));
    }
    meet[LID_0] = a.v;
    local_barrier();
    if (LID_0 < F) {
      for (unsigned q = 1; q < S; q++) a = rd_combine(a, rd_pacc(meet[q * F + LID_0]));
      out(LID_0, a);
    }
  } else {
    for (unsigned k = LID_0; k < F; k += 256u) {
      rd_acc a = rd_neutral();
      for (unsigned i = 0; i < copies; i++) a = rd_combine(a, rd_pacc(fetch(i * F + k)));
      out(k, a);
    }
  }
}

KERNEL void __launch_bounds__(256)
redux_pcols(RD_SRC_PARAMS, char *__restrict__ d0, const ga_size d0_off, char *__restrict__ d1,
            const ga_size d1_off, RD_ACC_T *__restrict__ part_v, ga_long *__restrict__ part_i, ga_uint *done,
            const rd_plan p RD_SCALAR_PARAMS) {
  __shared__ RD_ACC_T stage[256 * RD_PVN];
  __shared__ RD_ACC_T meet[256];
  __shared__ ga_uint last_piece;
  const unsigned F = (unsigned)p.nrows, L = (unsigned)p.upb, G = (unsigned)p.nsplit;
  const ga_long J = p.units;
  const ga_long bytes = p.nrows * p.rtotal * RD_ELSZ0;
  const ga_long full = bytes >> 4;                          /* whole chunks */
  const int rem = (int)((bytes & 15) / RD_ELSZ0);           /* elements of a last, partial chunk */
  const char *base[RD_NSRC];
  RD_SRC_BASES(base);
  /* p.router > 1: that many dense arrays (slabs) of p.rtotal rows one behind
   * the other, whole chunks each, G groups per slab; the outputs of slab s are
   * the rows s F ... s F + F - 1 of the result */
  const ga_long slab = p.router > 1 ? (ga_long)(GID_0 / G) : 0;
  const unsigned gi = (unsigned)((ga_long)GID_0 - slab * G);
  const rd_tchunk_t *src = (const rd_tchunk_t *)base[0] + slab * full;

  rd_acc acc[RD_PVN];
#pragma unroll
  for (int v = 0; v < RD_PVN; v++) acc[v] = rd_neutral();
  if (LID_0 < L) {
    const ga_long c0 = (ga_long)gi * L * J + LID_0;
    for (ga_long j = 0; j < J; j += RD_U) {
      rd_tchunk_t c[RD_U];
      if (j + RD_U <= J && c0 + (j + RD_U - 1) * L < full) {
        /* all of the batch inside the array: the loads go out together */
#pragma unroll
        for (int u = 0; u < RD_U; u++) c[u] = RD_LOAD(src + c0 + (j + u) * L);
#pragma unroll
        for (int u = 0; u < RD_U; u++)
#pragma unroll
          for (int v = 0; v < RD_PVN; v++)
            acc[v] = rd_combine(acc[v], rd_elem(RD_ONE_VAL(rd_trow_elem(&c[u], v)), 0));
      } else {
#pragma unroll
        for (int u = 0; u < RD_U; u++) {
          const ga_long ci = c0 + (j + u) * L;
          const bool in = j + u < J && (ci < full || (ci == full && rem > 0));
          c[u] = (rd_tchunk_t)(0u);
          if (in) c[u] = RD_LOAD(src + ci);
#pragma unroll
          for (int v = 0; v < RD_PVN; v++)
            if (in && (ci < full || v < rem))
              acc[v] = rd_combine(acc[v], rd_elem(RD_ONE_VAL(rd_trow_elem(&c[u], v)), 0));
        }
      }
    }
  }
#pragma unroll
  for (int v = 0; v < RD_PVN; v++) stage[LID_0 * RD_PVN + v] = acc[v].v;   /* idle lanes: neutral */
  local_barrier();
  /* a group's chunks start at a multiple of L chunks, a whole number of kept
   * rows: accumulator v of lane l belongs to output (l RD_PVN + v) mod F */
  if (G == 1u) {
    /* one group per slab: its F values are the slab's outputs (no partials, no counter) */
    rd_pcols_fold(F, L * RD_PVN / F, meet,
                  [&](const unsigned at) { return stage[at]; },
                  [&](const unsigned k, const rd_acc a) {
                    ga_long so[RD_NSRC], d0o, d1o;
                    rd_row_offsets(p, slab * F + k, so, &d0o, &d1o);
                    rd_write(a, d0 + d0_off, d0o, d1 + d1_off, d1o);
                  });
    return;
  }
  rd_pcols_fold(F, L * RD_PVN / F, meet,
                [&](const unsigned at) { return stage[at]; },
                [&](const unsigned k, const rd_acc a) { rd_publish_partial(a, part_v, part_i, (ga_long)GID_0 * F + k); });
  rd_stores_done();   /* every lane that left partials */
  local_barrier();
  if (LID_0 == 0) last_piece = rd_count_in(done + slab, G) ? 1u : 0u;
  local_barrier();
  if (!last_piece) return;
  rd_before_loads();
  rd_pcols_fold(F, G, meet,
                [&](const unsigned at) { return rd_fetch_partial(part_v, part_i, slab * G * F + (ga_long)at).v; },
                [&](const unsigned k, const rd_acc a) {
                  ga_long so[RD_NSRC], d0o, d1o;
                  rd_row_offsets(p, slab * F + k, so, &d0o, &d1o);
                  rd_write(a, d0 + d0_off, d0o, d1 + d1_off, d1o);
                });
  if (LID_0 == 0) rd_count_reset(done + slab);
}
#endif   /* RD_PCOLS */

/* ---- helpers of redux_col ------------------------------------------------- */

/* Position j of the flattened reduced range: byte offset in every source and
 * flattened index in the caller's axis order.  32-bit divisions when the
 * range allows it. */
static __device__ inline void rd_col_at(const rd_plan &p, const ga_long j, ga_long *off, ga_long *ix) {
  if (p.nr == 1) {
#pragma unroll
    for (int k = 0; k < RD_NSRC; k++) off[k] = j * p.rsstr[k][0];
    *ix = j * p.rmul[0];
    return;
  }
#pragma unroll
  for (int k = 0; k < RD_NSRC; k++) off[k] = 0;
  *ix = 0;
  if (p.rtotal <= 0x7fffffffLL) {
    ga_uint r = (ga_uint)j;
    for (int d = p.nr - 1; d >= 0; d--) {
      ga_uint c = r;
      if (d > 0) {
        const ga_uint n = (ga_uint)p.rdim[d];
        const ga_uint qd = r / n;
        c = r - qd * n;
        r = qd;
      }
#pragma unroll
      for (int k = 0; k < RD_NSRC; k++) off[k] += (ga_long)c * p.rsstr[k][d];
      *ix += (ga_long)c * p.rmul[d];
    }
  } else {
    ga_long r = j;
    for (int d = p.nr - 1; d >= 0; d--) {
      ga_long c = r;
      if (d > 0) { r = rd_divmod(r, p.rdim[d], &c); }
#pragma unroll
      for (int k = 0; k < RD_NSRC; k++) off[k] += c * p.rsstr[k][d];
      *ix += c * p.rmul[d];
    }
  }
}

static __device__ inline ga_long rd_col_index(const rd_plan &p, const ga_long j) {
  ga_long off[RD_NSRC], ix;
  rd_col_at(p, j, off, &ix);
  return ix;
}

/* A lane's RD_CV adjacent elements at position j of the reduced range. */
static __device__ inline void rd_col_fetch(const rd_plan &p, const char *const *srow, const ga_long j,
                                           rd_cvec &x, const int nv) {
  ga_long off[RD_NSRC], ix;
  rd_col_at(p, j, off, &ix);
  const char *ep[RD_NSRC];
#pragma unroll
  for (int k = 0; k < RD_NSRC; k++) ep[k] = srow[k] + off[k];
  rd_cvec_load(x, ep, nv);
}

/* Arg-min/max and floating min/max scan a lane's elements in rising order
 * with a strict compare when the plan says the index rises with them
 * (RD_RISING: decided per variant, so that a text holds one of the two scans). */
#define RD_COL_SCAN (RD_RISING && RD_ARG && (RD_KIND == RD_K_MAX || RD_KIND == RD_K_MIN))
#if RD_KIND == RD_K_MAX
#define RD_COL_BETTER(a, b) ((a) > (b))
#else
#define RD_COL_BETTER(a, b) ((a) < (b))
#endif

#define RD_CX (256 / RD_CY)   /* lanes along the free dim; RD_CY lane rows share the reduced range */

#if RD_WANT & 2   /* redux_col */
/* ---- redux_col -------------------------------------------------------------
 * Lanes along the fastest free dim; a lane owns RD_CV adjacent outputs and
 * fetches them with one load (RD_CV > 1 needs that dim to be contiguous in
 * every source and everything aligned to the load). */

KERNEL void __launch_bounds__(256)
redux_col(RD_SRC_PARAMS, char *d0, const ga_size d0_off, char *d1, const ga_size d1_off,
          RD_ACC_T *part_v, ga_long *part_i, ga_uint *done, const rd_plan p RD_SCALAR_PARAMS) {
  __shared__ rd_acc lds[RD_CY][RD_CV][RD_CX];
  const unsigned tx = LID_0 % RD_CX, ty = LID_0 / RD_CX;
#if RD_XCD
  /* Groups g and g + 8 run on the same of the 8 dies, each with a cache of its
   * own.  Here the groups that are neighbours along the inner free dim (same
   * rows, same piece of the reduced range) follow one another on one die:
   * their pieces of a row share the lines that the pieces straddle when rows
   * do not start on 128-byte lines, and a line is then fetched from memory
   * once, not once per die (sum over the middle axis of (64, 1000, 1000)
   * floats read 1.38 times the array in the plain order). */
  unsigned gid = GID_0;
  {
    const unsigned whole = (unsigned)p.units;   /* the launch's groups, down to a multiple of 8 */
    if (gid < whole) gid = (gid % 8u) * (whole / 8u) + gid / 8u;
  }
  /* a launch has fewer than 2^31 groups: 32-bit divisions */
  const unsigned gxs = (unsigned)p.gx, tq = gid / gxs;
  const ga_long bx = (ga_long)(gid - tq * gxs);
  const ga_long fo = (ga_long)(tq / (unsigned)p.nsplit);        /* flat index over the outer free dims */
  const ga_long split = (ga_long)(tq - (unsigned)fo * (unsigned)p.nsplit);
  ga_long t = fo * p.gx + bx;                                   /* the tile of outputs (its counter) */
#else
  const unsigned gid = GID_0;
  const ga_long split = gid % (unsigned)p.nsplit;
  ga_long t = gid / (unsigned)p.nsplit;
  ga_long bx;
  const ga_long fo = rd_divmod(t, p.gx, &bx);   /* flat index over the outer free dims */
#endif
  const int fi_d = p.nf - 1;
  const ga_long fin = p.fdim[fi_d];
  const ga_long fi = (bx * RD_CX + tx) * RD_CV;   /* first of the lane's outputs */
  const bool live = fi < fin;
  /* how many of the lane's RD_CV outputs exist (RD_CLOOSE: the inner free
   * dim need not be a multiple of RD_CV; else all of them do) */
#if RD_CLOOSE
  const int nv = fin - fi >= RD_CV ? RD_CV : (int)(fin - fi);
#else
  const int nv = RD_CV;
#endif

  /* offsets of this lane's first output */
  ga_long so[RD_NSRC], d0o = 0, d1o = 0;
#pragma unroll
  for (int k = 0; k < RD_NSRC; k++) so[k] = 0;
  {
    ga_long r = fo;
    for (int d = fi_d - 1; d >= 0; d--) {
      ga_long c;
      if (d > 0) { r = rd_divmod(r, p.fdim[d], &c); } else { c = r; }
#pragma unroll
      for (int k = 0; k < RD_NSRC; k++) so[k] += c * p.fsstr[k][d];
      d0o += c * p.fd0str[d];
      d1o += c * p.fd1str[d];
    }
#pragma unroll
    for (int k = 0; k < RD_NSRC; k++) so[k] += fi * p.fsstr[k][fi_d];
    d0o += fi * p.fd0str[fi_d];
    d1o += fi * p.fd1str[fi_d];
  }
  const char *srow[RD_NSRC];
  RD_SRC_BASES(srow);
#pragma unroll
  for (int k = 0; k < RD_NSRC; k++) srow[k] += so[k];

  ga_long r0 = split * p.upb, r1 = r0 + p.upb;
  if (r1 > p.rtotal) r1 = p.rtotal;

  rd_acc acc[RD_CV];
#pragma unroll
  for (int c = 0; c < RD_CV; c++) acc[c] = rd_neutral();
#if RD_COL_SCAN
  if (live) {
    /* The index grows with j and j fits 31 bits: a lane meets its elements in
     * rising order, so a strict compare keeps the first of equals, and what
     * it carries per output is the value and a 32-bit j. */
    RD_ACC_T bv[RD_CV];
    ga_int bj[RD_CV];
#pragma unroll
    for (int c = 0; c < RD_CV; c++) { bv[c] = RD_NEUTRAL; bj[c] = 0x7fffffff; }
    ga_long j0 = r0 + ty;
    for (; j0 + RD_CY * (RD_U - 1) < r1; j0 += RD_CY * RD_U) {
      rd_cvec x[RD_U];
#pragma unroll
      for (int q = 0; q < RD_U; q++) rd_col_fetch(p, srow, j0 + RD_CY * q, x[q], nv);
#pragma unroll
      for (int q = 0; q < RD_U; q++) {
#pragma unroll
        for (int c = 0; c < RD_CV; c++) {
          const RD_ACC_T val = rd_later(RD_CVEC_VAL(x[q], c));
          const bool better = RD_COL_BETTER(val, bv[c]);
          bv[c] = better ? val : bv[c];
          bj[c] = better ? (ga_int)(j0 + RD_CY * q) : bj[c];
        }
      }
    }
    if (j0 < r1) {   /* the last, partial batch: its loads go out together too */
      rd_cvec x[RD_U];
#pragma unroll
      for (int q = 0; q < RD_U; q++)
        if (j0 + RD_CY * q < r1) rd_col_fetch(p, srow, j0 + RD_CY * q, x[q], nv);
#pragma unroll
      for (int q = 0; q < RD_U; q++)
        if (j0 + RD_CY * q < r1) {
#pragma unroll
          for (int c = 0; c < RD_CV; c++) {
            const RD_ACC_T val = rd_later(RD_CVEC_VAL(x[q], c));
            const bool better = RD_COL_BETTER(val, bv[c]);
            bv[c] = better ? val : bv[c];
            bj[c] = better ? (ga_int)(j0 + RD_CY * q) : bj[c];
          }
        }
    }
    if (r0 + ty < r1) {
#pragma unroll
      for (int c = 0; c < RD_CV; c++) {
        /* nothing beat the neutral value: every element equals it, the first stays */
        const ga_long j = bj[c] == 0x7fffffff ? r0 + ty : (ga_long)bj[c];
        acc[c].v = bv[c];
        acc[c].i = rd_col_index(p, j);
      }
    }
  }
#elif RD_COL_FAST8
  if (live) {
    /* any / all over bytes: bit 8c+7 of word c/4 of `seen` says that byte c of
     * some load was non-zero (any) or zero (all); exact per byte (the sum of
     * the low seven bits and 0x7f carries into bit 7 and no further) */
    ga_uint seen[RD_CV / 4];
#pragma unroll
    for (int d = 0; d < RD_CV / 4; d++) seen[d] = 0;
#define RD_COL_BYTES_SEEN(xx)                                                              \
  _Pragma("unroll") for (int d = 0; d < RD_CV / 4; d++) {                                  \
    const ga_uint wd = RD_CVEC_WORD(xx, d);                                                \
    const ga_uint nz = (((wd & 0x7f7f7f7fu) + 0x7f7f7f7fu) | wd) & 0x80808080u;            \
    seen[d] |= RD_KIND == RD_K_ANY ? nz : (nz ^ 0x80808080u);                              \
  }
    ga_long j0 = r0 + ty;
    for (; j0 + RD_CY * (RD_U - 1) < r1; j0 += RD_CY * RD_U) {
      rd_cvec x[RD_U];
#pragma unroll
      for (int q = 0; q < RD_U; q++) rd_col_fetch(p, srow, j0 + RD_CY * q, x[q], nv);
#pragma unroll
      for (int q = 0; q < RD_U; q++) { RD_COL_BYTES_SEEN(x[q]) }
    }
    if (j0 < r1) {   /* the last, partial batch */
      rd_cvec x[RD_U];
#pragma unroll
      for (int q = 0; q < RD_U; q++)
        if (j0 + RD_CY * q < r1) rd_col_fetch(p, srow, j0 + RD_CY * q, x[q], nv);
#pragma unroll
      for (int q = 0; q < RD_U; q++)
        if (j0 + RD_CY * q < r1) { RD_COL_BYTES_SEEN(x[q]) }
    }
#undef RD_COL_BYTES_SEEN
#pragma unroll
    for (int c = 0; c < RD_CV; c++) {
      const ga_uint bit = (seen[c / 4] >> (8 * (c % 4) + 7)) & 1u;
      acc[c].v = RD_KIND == RD_K_ANY ? bit : (bit ^ 1u);
    }
  }
#else
  if (live) {
    ga_long j0 = r0 + ty;
    /* all RD_U loads of a batch lie inside the range: no test per load */
    for (; j0 + RD_CY * (RD_U - 1) < r1; j0 += RD_CY * RD_U) {
      rd_cvec x[RD_U];
      ga_long idx[RD_U];
#pragma unroll
      for (int q = 0; q < RD_U; q++) {
        rd_col_fetch(p, srow, j0 + RD_CY * q, x[q], nv);
        idx[q] = RD_ARG ? rd_col_index(p, j0 + RD_CY * q) : 0;
      }
#pragma unroll
      for (int q = 0; q < RD_U; q++) {
#pragma unroll
        for (int c = 0; c < RD_CV; c++)
          acc[c] = rd_combine(acc[c], rd_elem(RD_CVEC_VAL(x[q], c), idx[q]));
      }
    }
    if (j0 < r1) {   /* the last, partial batch: its loads go out together too */
      rd_cvec x[RD_U];
      ga_long idx[RD_U];
#pragma unroll
      for (int q = 0; q < RD_U; q++)
        if (j0 + RD_CY * q < r1) {
          rd_col_fetch(p, srow, j0 + RD_CY * q, x[q], nv);
          idx[q] = RD_ARG ? rd_col_index(p, j0 + RD_CY * q) : 0;
        }
#pragma unroll
      for (int q = 0; q < RD_U; q++)
        if (j0 + RD_CY * q < r1) {
#pragma unroll
          for (int c = 0; c < RD_CV; c++)
            acc[c] = rd_combine(acc[c], rd_elem(RD_CVEC_VAL(x[q], c), idx[q]));
        }
    }
  }
#endif
#if RD_CY > 1
#pragma unroll
  for (int c = 0; c < RD_CV; c++) lds[ty][c][tx] = acc[c];
  local_barrier();
#else
  (void)lds;
#endif
  if (ty == 0 && live) {
#pragma unroll
    for (int c = 0; c < RD_CV; c++) {
      if (RD_CLOOSE && c >= nv) break;
      rd_acc a = acc[c];
#pragma unroll
      for (int y = 1; y < RD_CY; y++) a = rd_combine(a, lds[y][c][tx]);
      const ga_long row = fo * fin + fi + c;
      if (p.nsplit == 1) {
        /* element 0 of the scan is at the start of the output's reduced range */
        const char *sc[RD_NSRC];
#pragma unroll
        for (int k = 0; k < RD_NSRC; k++) sc[k] = srow[k] + c * p.fsstr[k][fi_d];
        rd_store(a, sc, d0 + d0_off, d0o + c * p.fd0str[fi_d], d1 + d1_off,
                 d1o + c * p.fd1str[fi_d], p.rtotal RD_SCALAR_ARGS);
      } else {
        /* with many outputs the partials lie split-major (adjacent lanes write
         * adjacent slots, redux_final_cols reads them); else output-major */
        if (p.fused)
          rd_publish_partial(a, part_v, part_i, split * p.nrows + row);
        else
          rd_store_partial(a, part_v, part_i,
                           p.split_major ? split * p.nrows + row : row * p.nsplit + split);
      }
    }
  }
  if (p.nsplit > 1 && p.fused) {
    /* one counter per tile of outputs (the groups that differ in `split` only);
     * the partials lie split-major here */
    __shared__ ga_uint last_piece;
    rd_stores_done();   /* every lane that left partials */
    local_barrier();
    if (LID_0 == 0) last_piece = rd_count_in(done + t, (ga_uint)p.nsplit) ? 1u : 0u;
    local_barrier();
    if (!last_piece) return;
    rd_before_loads();
#pragma unroll
    for (int c = 0; c < RD_CV; c++) acc[c] = rd_neutral();
    if (live) {
      /* a lane row's partials four or eight splits at a time, all their loads issued
       * before the first is combined (one at a time, the 256 partials of 64
       * outputs took 12 of the 16 us of a sum over axis 0 of (16384, 64));
       * combined in the order of the splits either way */
      const ga_long at = fo * fin + fi;
      ga_long s = ty;
#if RD_ARG || RD_CV > 4
#define RD_FIN_BATCH 4
#else
#define RD_FIN_BATCH 8
#endif
      for (; s + (RD_FIN_BATCH - 1) * RD_CY < p.nsplit; s += RD_FIN_BATCH * RD_CY) {
        rd_acc t[RD_FIN_BATCH][RD_CV];
#pragma unroll
        for (int j = 0; j < RD_FIN_BATCH; j++)
#pragma unroll
          for (int c = 0; c < RD_CV; c++)
            t[j][c] = (RD_CLOOSE && c >= nv) ? rd_neutral()
                                              : rd_fetch_partial(part_v, part_i, (s + j * RD_CY) * p.nrows + at + c);
#pragma unroll
        for (int j = 0; j < RD_FIN_BATCH; j++)
#pragma unroll
          for (int c = 0; c < RD_CV; c++) acc[c] = rd_combine(acc[c], t[j][c]);
      }
#undef RD_FIN_BATCH
      for (; s < p.nsplit; s += RD_CY)
#pragma unroll
        for (int c = 0; c < RD_CV; c++)
          if (!RD_CLOOSE || c < nv)
            acc[c] = rd_combine(acc[c], rd_fetch_partial(part_v, part_i, s * p.nrows + at + c));
    }
#if RD_CY > 1
#pragma unroll
    for (int c = 0; c < RD_CV; c++) lds[ty][c][tx] = acc[c];
    local_barrier();
#endif
    if (ty == 0 && live) {
#pragma unroll
      for (int c = 0; c < RD_CV; c++) {
        if (RD_CLOOSE && c >= nv) break;
        rd_acc a = acc[c];
#pragma unroll
        for (int y = 1; y < RD_CY; y++) a = rd_combine(a, lds[y][c][tx]);
        const char *sc[RD_NSRC];
#pragma unroll
        for (int k = 0; k < RD_NSRC; k++) sc[k] = srow[k] + c * p.fsstr[k][fi_d];
        rd_store(a, sc, d0 + d0_off, d0o + c * p.fd0str[fi_d], d1 + d1_off,
                 d1o + c * p.fd1str[fi_d], p.rtotal RD_SCALAR_ARGS);
      }
    }
    if (LID_0 == 0) rd_count_reset(done + t);
  }
}

#endif   /* RD_WANT & 2 */

#if RD_WANT & 8
/* ---- redux_final ------------------------------------------------------------
 * One wavefront per output: combine its nsplit partials and write the result. */
KERNEL void __launch_bounds__(256)
redux_final(RD_SRC_PARAMS, char *d0, const ga_size d0_off, char *d1, const ga_size d1_off,
            RD_ACC_T *part_v, ga_long *part_i, ga_uint *done, const rd_plan p RD_SCALAR_PARAMS) {
  const unsigned lane = LID_0 & 63u;
  const ga_long row = (ga_long)GID_0 * 4 + (LID_0 >> 6);
  if (row >= p.nrows) return;
  ga_long so[RD_NSRC], d0o, d1o;
  rd_row_offsets(p, row, so, &d0o, &d1o);
  const char *srow[RD_NSRC];
  RD_SRC_BASES(srow);
#pragma unroll
  for (int k = 0; k < RD_NSRC; k++) srow[k] += so[k];
  RD_ACC_T first = RD_NEUTRAL;
  if (lane == 0) first = rd_first_value(srow, p.rtotal RD_SCALAR_ARGS);
  rd_acc acc = rd_neutral();
  for (ga_long s = lane; s < p.nsplit; s += 64) {
    rd_acc t;
    t.v = part_v[row * p.nsplit + s];
#if RD_ARG
    t.i = part_i[row * p.nsplit + s];
#endif
    acc = rd_combine(acc, t);
  }
  acc = rd_wave_reduce(acc);
  if (lane == 0) rd_write(rd_first_rule(acc, first), d0 + d0_off, d0o, d1 + d1_off, d1o);
}

#endif   /* RD_WANT & 8 */

#if (RD_WANT & 10) == 10
/* The second pass after redux_col, whose partials lie split-major
 * (slot = split * nrows + output): 64 adjacent outputs per group, lanes along
 * the outputs so that every load of a wavefront is one contiguous run, the 4
 * lane rows share the splits and meet in LDS. */
KERNEL void __launch_bounds__(256)
redux_final_cols(RD_SRC_PARAMS, char *d0, const ga_size d0_off, char *d1, const ga_size d1_off,
                 RD_ACC_T *part_v, ga_long *part_i, ga_uint *done, const rd_plan p RD_SCALAR_PARAMS) {
  __shared__ rd_acc meet[4][64];
  const unsigned tx = LID_0 & 63u, ty = LID_0 >> 6;
  const ga_long row = (ga_long)GID_0 * 64 + tx;
  const bool live = row < p.nrows;
  rd_acc acc = rd_neutral();
  if (live) {
    for (ga_long s = ty; s < p.nsplit; s += 4) {
      rd_acc t;
      t.v = part_v[s * p.nrows + row];
#if RD_ARG
      t.i = part_i[s * p.nrows + row];
#endif
      acc = rd_combine(acc, t);
    }
  }
  meet[ty][tx] = acc;
  local_barrier();
  if (ty == 0 && live) {
    acc = rd_combine(acc, meet[1][tx]);
    acc = rd_combine(acc, meet[2][tx]);
    acc = rd_combine(acc, meet[3][tx]);
    ga_long so[RD_NSRC], d0o, d1o;
    rd_row_offsets(p, row, so, &d0o, &d1o);
    const char *srow[RD_NSRC];
    RD_SRC_BASES(srow);
#pragma unroll
    for (int k = 0; k < RD_NSRC; k++) srow[k] += so[k];
    rd_store(acc, srow, d0 + d0_off, d0o, d1 + d1_off, d1o, p.rtotal RD_SCALAR_ARGS);
  }
}
#endif   /* RD_WANT & 2 and & 8 */
