// Tuning knobs of the planners.
//
// Every knob is an environment variable GPUARRAY_<NAME> holding a number.  The
// environment is read when a context is made (and again when the caller asks
// through the "hip_reload_tuning" hook), never on the path of a call: a call
// looks a knob up in its context's table, which is one load and one test.
// A knob that is not set leaves the planner's own choice (the default given at
// the place of use, often computed from the call) in force.
#pragma once

#include <cstdint>
#include <cstdlib>

#define GA_KNOBS(X) \
  X(ALLOW_OTHER_ISA) X(ELEMWISE_BAND) X(ELEMWISE_FLAT_NT_MASK) X(ELEMWISE_GROUPS_PER_CU) \
  X(ELEMWISE_MIXED_ALIGN) X(ELEMWISE_NARROW) X(ELEMWISE_NARROW_CHUNKS) X(ELEMWISE_NARROW_LDS) X(ELEMWISE_NARROW_MIN) X(ELEMWISE_NARROW_MIN_PLANE) X(ELEMWISE_NARROW_NT) X(ELEMWISE_NARROW_QUADS) X(ELEMWISE_NARROW_STAGED) X(ELEMWISE_NARROW_STAGED_WIDE) X(ELEMWISE_NT) X(ELEMWISE_NT_LINES) X(ELEMWISE_NT_MASK) X(ELEMWISE_PAIRS) \
  X(ELEMWISE_PANEL) X(ELEMWISE_PERIODIC) X(ELEMWISE_PERIODIC_ROWLOAD) X(ELEMWISE_PERIODIC_VEC) X(ELEMWISE_LOOSE) X(ELEMWISE_LOOSE_MIN_BYTES) X(ELEMWISE_QUADS) X(ELEMWISE_RECORDS) X(ELEMWISE_RECORDS_MIN) X(ELEMWISE_RECORDS_NT) X(ELEMWISE_RECORDS_SKEW) X(ELEMWISE_RECORDS_TILE) X(ELEMWISE_RECORDS_YMAJOR) X(ELEMWISE_SKEW) \
  X(ELEMWISE_TILE) X(ELEMWISE_TMIN) X(ELEMWISE_TTILE) X(ELEMWISE_TTILE_FILL) X(ELEMWISE_TTILE_MIN) X(ELEMWISE_UNROLL) X(ELEMWISE_VEC4) \
  X(ELEMWISE_ZMASK) X(FILL_KERNEL_MIN) X(MARK_EVENT_FLAGS) X(MOVE_KERNEL_MIN) X(REDUX_BALANCE) X(REDUX_COLVEC) \
  X(REDUX_COL_BALANCE) X(REDUX_COL_CVMAX) X(REDUX_COL_FAR) X(REDUX_COL_IDLE) X(REDUX_COL_LOOSE) X(REDUX_COL_LOOSE_MIN_BYTES) X(REDUX_COL_ROWS) X(REDUX_COL_U) X(REDUX_FAST8) \
  X(REDUX_FOLD) X(REDUX_FOLD_BYTES) X(REDUX_FOLD_MIN_BYTES) X(REDUX_FOLD_SLAB_MIN_BYTES) X(REDUX_FUSED) \
  X(REDUX_FUSED_COL_FEW) X(REDUX_FUSED_COL_PIECE) X(REDUX_FUSED_COL_SPLITS) \
  X(REDUX_FUSED_FEW) X(REDUX_FUSED_PIECE) X(REDUX_G) X(REDUX_GROUPS_PER_CU) X(REDUX_INFLIGHT) X(REDUX_INTERLEAVE) \
  X(REDUX_L) X(REDUX_LANE_BYTES) X(REDUX_LIGHT) X(REDUX_LO) X(REDUX_MIN_PER_CU) X(REDUX_MEMO) X(REDUX_PCOLS) X(REDUX_PCOLS_PER_CU) X(REDUX_PSLABS) X(REDUX_PSLABS_MAX_BYTES) X(REDUX_PSLABS_MIN_SLABS) X(REDUX_PCOLS_COL_BYTES) X(REDUX_PCOLS_MAX_PARTIALS) X(ELEMWISE_MEMO) X(ELEMWISE_TPAIRS) \
  X(REDUX_MIN_UNITS) X(REDUX_NT) X(REDUX_NT_LINES) X(REDUX_OUTER_FIRST) X(REDUX_RB) X(REDUX_RPW) X(REDUX_SPLIT_MAJOR_MIN) \
  X(REDUX_SROWS) X(REDUX_SROWS_MAX_BYTES) X(REDUX_SROWS_MIN_BYTES) X(REDUX_SROWS_MIN_ROWS) \
  X(REDUX_TAIL) X(REDUX_TOUCH) X(REDUX_TROWS) X(REDUX_TROWS_DIRECT) X(REDUX_TROWS_MAX_BYTES) \
  X(REDUX_TROWS_MAX_CHUNKS) X(REDUX_TROWS_MIN_ROWS) X(REDUX_U) X(REDUX_WROWS) X(REDUX_XCD) \
  X(TAKE1_SHORT_ROWS)

enum ga_knob : unsigned {
#define X(name) KNOB_##name,
  GA_KNOBS(X)
#undef X
  GA_NKNOBS
};

struct ga_tuning {
  bool set[GA_NKNOBS];
  unsigned long val[GA_NKNOBS];
  unsigned long generation;   // differs between any two fillings of any table in the process
  char redux_family[16];   // GPUARRAY_REDUX_FAMILY ("row" / "col"), empty = the planner's choice
  unsigned long get(ga_knob k, unsigned long dflt) const { return set[k] ? val[k] : dflt; }
  bool is_set(ga_knob k) const { return set[k]; }
};

// Fills `t` from the environment.
void ga_tuning_read(ga_tuning *t);
// A table read from the environment on first use, for code that runs without a context.
const ga_tuning *ga_tuning_default();

struct _gpucontext;
// The table of a context; of no context (ctx == NULL: operators made only to
// show their kernel text), the table read from the environment on first use.
const ga_tuning *ga_hip_tuning(_gpucontext *ctx);
