/* GpuReduction: reductions over any subset of the axes of a strided array.
 *
 * The reference snapshot has no such header: its only C reduction is
 * GpuArray_maxandargmax (src/gpuarray/array.h:607-644,
 * src/gpuarray_reduction.c:100-124) and sum/prod/any/all exist only in its
 * Python layer (pygpu/reduction.py:137-319, pygpu/_array.py:238-294).  This
 * header gives those semantics, plus min, max, arg-min/max and bitwise, one C entry
 * point.  GpuArray_maxandargmax is a wrapper around GA_REDUCE_MAXANDARGMAX.
 */
#ifndef GPUARRAY_REDUCTION_H
#define GPUARRAY_REDUCTION_H

#include <gpuarray/array.h>
#include <gpuarray/buffer.h>
#include <gpuarray/elemwise.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum _ga_reduce_op {
  /*                               d0 (value)        d1 (index)          */
  GA_REDUCE_SUM = 0,            /* sum                 -                  */
  GA_REDUCE_PROD,               /* product             -                  */
  GA_REDUCE_PRODNZ,             /* product of non-zero elements           */
  GA_REDUCE_MIN,                /* minimum             -                  */
  GA_REDUCE_MAX,                /* maximum             -                  */
  GA_REDUCE_ARGMIN,             /* -                   index of minimum   */
  GA_REDUCE_ARGMAX,             /* -                   index of maximum   */
  GA_REDUCE_MINANDARGMIN,       /* minimum             index of minimum   */
  GA_REDUCE_MAXANDARGMAX,       /* maximum             index of maximum   */
  GA_REDUCE_AND,                /* bitwise and         -                  */
  GA_REDUCE_OR,                 /* bitwise or          -                  */
  GA_REDUCE_XOR,                /* bitwise xor         -                  */
  GA_REDUCE_ALL,                /* 1 if all non-zero   -                  */
  GA_REDUCE_ANY,                /* 1 if any non-zero   -                  */
  GA_REDUCE_CUSTOM,             /* caller's expression (GpuReduction_new_map only) */
  GA_REDUCE_ENDSUPPORTED
} ga_reduce_op;

typedef struct _GpuReduction GpuReduction;

/* Create a reduction operator.
 *   ndf, ndr    expected numbers of free and reduced axes; hints only, any
 *               rank is accepted by GpuReduction_call.
 *   s0Typecode  element type of the source.
 * Returns GA_NO_ERROR and *gr, or an error code with *gr == NULL. */
GPUARRAY_PUBLIC int GpuReduction_new(GpuReduction **gr, gpucontext *ctx,
                                     ga_reduce_op op, unsigned ndf,
                                     unsigned ndr, int s0Typecode, int flags);
GPUARRAY_PUBLIC void GpuReduction_free(GpuReduction *gr);

/* Reduce s0 over the axes in reduxList.
 *
 *   d0  value result (NULL for ARGMIN/ARGMAX), d1 index result (NULL unless
 *       the op has one).  Each has the shape of s0 with the reduced axes
 *       removed, in ascending axis order, and is written through its own
 *       strides; GA_VALUE_ERROR on a shape mismatch.
 *   accumulation type = d0's element type: SUM/PROD of int32 into an int64
 *       d0 accumulates in 64 bits (the rule of pygpu/_array.py:250-293);
 *       half sources are widened to float and accumulated in float whatever
 *       d0 is (float or half).  Integer sums wrap modulo 2^bits, so they are
 *       exact and order-independent.  Floating sums use a fixed tree order:
 *       the same call gives the same bits every time.
 *   ALL/ANY test `element != 0` and write 0/1 (pygpu/_array.py:238-248).
 *   MIN/MAX/ARG*: d0 must have s0's type, d1 a 64-bit integer type
 *       (GA_LONG, GA_ULONG).  The index is flattened over the reduced axes
 *       in reduxList order (see GpuArray_maxandargmax); ties resolve to the
 *       lowest index; NaN is ignored unless it is element 0 of the scan.
 *   empty reduction (a reduced axis of length 0): d0 gets the neutral
 *       element (0, 1, all-ones, ...); MIN/MAX/ARG* give GA_VALUE_ERROR.
 *   reduxLen == 0 is GA_INVALID_ERROR, as are repeated or out-of-range axes.
 */
GPUARRAY_PUBLIC int GpuReduction_call(const GpuReduction *gr, GpuArray *d0,
                                      GpuArray *d1, const GpuArray *s0,
                                      unsigned reduxLen, const int *reduxList,
                                      int flags);

/* GpuReduction_call for callers that cannot allocate device memory: code
 * under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  It has no counterpart in the reference.
 *
 * Same arguments, rules and results as GpuReduction_call (operators made by
 * GpuReduction_new only).  Where GpuReduction_call keeps the partial results
 * of a split reduction in a buffer the context allocates and grows, this
 * entry point keeps them in a device array that is part of the library
 * itself, GA_REDUCTION_NOALLOC_SCRATCH bytes on every GPU the library runs
 * on, looked up once when the context is made; it calls no allocating
 * routine, and a split reduction always ends in a second launch (the one
 * exception: the leading dims of a dense array over short kept rows keep
 * their single launch, whose counter an earlier GpuReduction_call has made).
 * Every layout takes the route GpuReduction_call takes for it, so that one
 * such call is the warm-up this entry point needs.
 *   GA_UNSUPPORTED_ERROR  the kernels for this layout are not built yet
 *                         (building loads a code object, which allocates):
 *                         call GpuReduction_call once on arrays of the same
 *                         types and layout first.
 *   GA_XLARGE_ERROR       the partials (outputs x pieces x 12 or 16 bytes)
 *                         would not fit GA_REDUCTION_NOALLOC_SCRATCH.
 * All calls on one GPU share that GPU's array: calls issued on one context
 * run in order on its stream; calls on different contexts of the same GPU
 * that overlap in time race, and must be ordered by the caller. */
#define GA_REDUCTION_NOALLOC_SCRATCH ((size_t)4 << 20)
GPUARRAY_PUBLIC int GpuReduction_call_noalloc(const GpuReduction *gr,
                                              GpuArray *d0, GpuArray *d1,
                                              const GpuArray *s0,
                                              unsigned reduxLen,
                                              const int *reduxList, int flags);

/* A reduction fed by an elementwise expression over several arguments, in one
 * pass over memory: the C counterpart of the reference's
 * ReductionKernel(map_expr=..., arguments=...) (pygpu/reduction.py:137-291,
 * used as in pygpu/tests/test_reduction.py:57-84), which exists there only in
 * Python.
 *
 *   op           any ga_reduce_op.  GA_REDUCE_CUSTOM combines with the caller's
 *                `reduce_expr`, an expression in `a` and `b` (the reference's
 *                REDUCE(a, b) macro, pygpu/reduction.py:38), starting from
 *                `neutral`; the expression must be associative and
 *                commutative and `neutral` its identity.  Both are NULL for
 *                the other operations.
 *   accTypecode  type the expression's value is converted to, the operation
 *                runs in, and the value result d0 has (ALL/ANY: any integer
 *                d0).  GA_HALF accumulates in float and stores a half.
 *   preamble     device code placed before the expression (may be NULL).
 *   map_expr     expression over the argument names, e.g. "a*b"; an array
 *                argument's name stands for its element (half elements are
 *                seen as float), a scalar's for its value.
 *   args         n descriptors as for GpuElemwise_new; GE_SCALAR marks
 *                scalars, GE_WRITE is refused.  At least one array, at most 8.
 */
GPUARRAY_PUBLIC int GpuReduction_new_map(GpuReduction **gr, gpucontext *ctx,
                                         ga_reduce_op op,
                                         const char *reduce_expr,
                                         const char *neutral, int accTypecode,
                                         const char *preamble,
                                         const char *map_expr, unsigned int n,
                                         const gpuelemwise_arg *args,
                                         int flags);

/* Run an operator made by GpuReduction_new_map.
 *   args   n pointers in descriptor order: GpuArray* for arrays, pointer to a
 *          host value of the declared type for scalars (the convention of
 *          GpuElemwise_call).
 *   flags  GE_BROADCAST: an extent of 1 stretches to the other arrays' extent.
 *          All arrays must have the same number of dimensions.
 * d0, d1, reduxLen, reduxList and every rule on values, indices, ties, NaN and
 * empty axes are those of GpuReduction_call, applied to the expression's
 * values over the common (broadcast) shape. */
GPUARRAY_PUBLIC int GpuReduction_call_map(const GpuReduction *gr, GpuArray *d0,
                                          GpuArray *d1, void **args,
                                          unsigned reduxLen,
                                          const int *reduxList, int flags);

#ifdef __cplusplus
}
#endif
#endif
