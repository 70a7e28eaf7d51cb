/* Function-pointer types of the hooks returned by gpuarray_get_extension()
 * on the "hip" backend.  Counterpart of the reference's CUDA hook list
 * (src/gpuarray/ext_cuda.h:1-46); only what a caller of the elementwise and
 * reduction path needs is published. */
#ifndef GPUARRAY_EXT_HIP_H
#define GPUARRAY_EXT_HIP_H

#include <gpuarray/buffer.h>

#ifdef __cplusplus
extern "C" {
#endif

/* "hip_get_stream": the context's single stream as a hipStream_t. */
typedef void *(*ga_hip_get_stream_fn)(gpucontext *ctx);
/* "hip_get_ptr": raw device address of a buffer. */
typedef void *(*ga_hip_get_ptr_fn)(gpudata *b);
/* "hip_get_sz": byte size of a buffer. */
typedef size_t (*ga_hip_get_sz_fn)(gpudata *b);
/* "hip_make_buf": wrap caller-owned device memory (not freed on release). */
typedef gpudata *(*ga_hip_make_buf_fn)(gpucontext *ctx, void *devptr,
                                       size_t sz);
/* "hip_compile_only": compile kernel source for gfx950 without a device and
 * return GA_NO_ERROR or GA_IMPL_ERROR; *log (if not NULL) gets a malloc'd
 * compiler log.  Lets host-only checks see that generated kernels build. */
typedef int (*ga_hip_compile_only_fn)(unsigned int count, const char **strs,
                                      const size_t *lens, char **log);
/* "hip_time_begin"/"hip_time_end": bracket queued work with events on the
 * context's stream; end waits and returns elapsed milliseconds (< 0 on
 * error). */
typedef int (*ga_hip_time_begin_fn)(gpucontext *ctx);
typedef float (*ga_hip_time_end_fn)(gpucontext *ctx);

/* "hip_event_record": put timing mark number `slot` on the context's stream
 * (marks are created on first use and reused); does not wait.  The marks'
 * events are made without the system-scope fence (hipEventDisableSystemFence):
 * they time the stream and publish nothing to the host.
 * "hip_event_elapsed": milliseconds from mark a to mark b; waits for b;
 * < 0 on error. */
typedef int (*ga_hip_event_record_fn)(gpucontext *ctx, unsigned int slot);
typedef float (*ga_hip_event_elapsed_fn)(gpucontext *ctx, unsigned int a, unsigned int b);
/* "hip_kernel_timing": on != 0 drops earlier records and gives every kernel
 * launch of the context from now on its own start and stop event (the
 * distance between them is the kernel's duration on the device, without the
 * gap between a mark on the stream and the kernel's start); on == 0 returns to
 * plain launches.  "hip_kernel_times": waits for the last recorded launch and
 * writes the durations, in milliseconds and in launch order, to out[0..max);
 * returns the number of launches recorded, < 0 on error. */
typedef int (*ga_hip_kernel_timing_fn)(gpucontext *ctx, int on);
typedef int (*ga_hip_kernel_times_fn)(gpucontext *ctx, float *out, unsigned int max);
/* "hip_kernel_hashes": the text hashes (as "hip_last_launch_hash" gives for the
 * last launch) of the launches recorded since hip_kernel_timing was turned
 * on, in launch order, to out[0..max); returns the number recorded.  A call
 * made of several kernels is identified by all of them. */
typedef int (*ga_hip_kernel_hashes_fn)(gpucontext *ctx, unsigned long long *out, unsigned int max);
/* "hip_last_launch_hash": 64-bit FNV-1a hash of the source text, followed by
 * the entry point's name, of the kernel the context launched last (0 before
 * the first launch): ties a measurement to the generated kernel it was made
 * on. */
typedef unsigned long long (*ga_hip_last_launch_hash_fn)(gpucontext *ctx);
/* "hip_reload_tuning": the planners' tuning knobs (environment variables
 * GPUARRAY_<NAME>, numbers) are read once, when a context is made, and looked
 * up in the context's table from then on; this reads the environment into
 * that table again.  For tests and sweeps that change a knob between calls. */
typedef int (*ga_hip_reload_tuning_fn)(gpucontext *ctx);
/* "hip_take1_source": kernel text of GpuArray_take1 for result/source/index
 * typecodes and `tnd` collapsed trailing dims; chunks != 0: the variant that
 * moves dense aligned rows as 16-byte chunks. */
typedef char *(*ga_hip_take1_source_fn)(int chunks, int a_typecode, int v_typecode,
                                        int i_typecode, unsigned int tnd);
/* "hip_module_cache_stats": out[0..2] = entries in the hot, warm and cold
 * lists of the context's loaded-module cache (the reference's 2Q policy,
 * src/cache/twoq.c), out[3] = code objects currently loaded. */
typedef int (*ga_hip_module_cache_stats_fn)(gpucontext *ctx, size_t out[4]);
/* "hip_elemwise_source" / "hip_reduction_source": the kernel text the
 * generators would compile for a given variant, as a malloc'd string the
 * caller frees.  For host-side checks of the generated code. */
/* strided: 0 flat kernel, 1 strided kernel with one element per lane,
 * 2 strided kernel with four elements per lane (tmask bits 0..15: arrays
 * staged through LDS; bits 16..: arrays with unit stride along x), 3 the
 * same with the streaming hint on every array's 16-byte accesses, 4 as 3
 * with 128 x 128 transposed tiles (1024 lanes), 5 / 6 the flat kernel with 2 /
 * 4 adjacent chunks per lane, 7 as 4 with every array in neither mask taken
 * as constant along x (one load for a lane's four elements), 8 as 4 with
 * every read-only array outside the LDS mask taken as constant along y (one
 * load for a lane's four rows), 9 the flat kernel with the arrays in tmask
 * (read-only, broadcast against the dense ones) read through the coordinates
 * of the flat index in nd = 2 or 3 dims (idx64 then carries the mask of those
 * among them that are fetched a whole aligned chunk at a time in bits 0..15,
 * and in bits 16.. the mask of those whose chunks inside one row of the inner
 * dim are fetched with one load on four-byte boundaries), 10 as 3 with
 * one group of two elements per lane (8-byte types, no transposed operand),
 * 11 to 13 variants of 4 and 3 for rows off the 64-byte blocks and for
 * four-byte elements on any layout, 14 a plane of two dims with a short
 * extent held in registers: nd carries the short extent (2 to 16; plus 256
 * for three dims, planes one after the other), idx64 the
 * width of the offsets in bit 0, which of the two dims is the short one in bit
 * 1, the streaming hint in bit 2, the LDS for the first kind of arrays in bit
 * 3, four-byte boundaries for the second kind in bit 4 and the arrays of
 * neither kind taken as constant along the long dim in bit 5; tmask bits 0..15
 * the arrays with the short dim innermost, bits 16.. those with the long one;
 * 15 the same arguments for a short extent of 17 to 64, whole through the LDS;
 * 16 tiles of short records: nd carries the record's elements (plus 256 for
 * four dims), idx64 the width of the offsets in bit 0 and the streaming hint
 * in bit 2, windows moved onto the last array's 64-byte blocks in bit 3 and
 * tiles numbered along Y first in bit 4,
 * tmask bits 0..15 the arrays whose records follow one another
 * along Y, bits 16.. those laid out like the result. */
typedef char *(*ga_hip_elemwise_source_fn)(const char *preamble, const char *expr,
                                           unsigned int n, void *args, int flags,
                                           int strided, unsigned int nd, int idx64,
                                           unsigned int tmask);
/* vec: elements used per load in bits 0..7, element step of the inner
 * reduced dim (1, 2 or 4; 0 means 1) in bits 8..15, adjacent outputs per lane
 * of the column kernel in bits 16..23 (0 means 1); bit 24: the column kernel
 * numbers its groups so that neighbours along the inner kept dim run on one die.
 * lanes_per_output: 64 or 256 in bits 0..15; lanes per row of the short-row
 * kernel in bits 16 and up (0 means 64).
 * unroll: loads in flight per lane in bits 0..7; rows per batch of the
 * short-row kernel in bits 8..15 (0 means 1); outer reduced coordinates the
 * row kernel handles side by side in bits 16..23 (0 means 1); bit 24: rows
 * read from the 16-byte boundary below their start, both ends masked; bit 25:
 * also the kernel that stages short contiguous rows in LDS; bit 26: the column
 * kernel of min / max scans in rising index order; bit 27: the kernel for rows
 * that one pass of a wavefront covers in place of the general row kernel
 * (64 lanes per output only); bit 28: every count of the call is below 2^31
 * (32-bit divisions); bit 29: also the kernel that walks rows of at most 32
 * bytes in registers, with bits 0..7 of vec as the row length in elements;
 * bit 30: also the kernel that reduces the leading dims of a dense array over
 * short kept rows in one launch; bit 31: the column kernel's loads assume the
 * elements' own alignment only, and the inner free dim need not be a multiple
 * of the outputs per lane. */
typedef char *(*ga_hip_reduction_source_fn)(int op, int src_typecode, int d0_typecode,
                                            int d1_typecode, unsigned int lanes_per_output,
                                            unsigned int vec, unsigned int unroll);
/* "hip_mapreduce_source": the same for an operator of GpuReduction_new_map
 * (same leading arguments); vecmask bit k: array argument k is fetched with
 * vector loads, the others element by element. */
typedef char *(*ga_hip_mapreduce_source_fn)(int op, const char *reduce_expr, const char *neutral,
                                            int acc_typecode, const char *preamble,
                                            const char *map_expr, unsigned int n, const void *args,
                                            int d0_typecode, unsigned int lanes_per_output,
                                            unsigned int vec, unsigned int unroll,
                                            unsigned int vecmask);

#ifdef __cplusplus
}
#endif
#endif
