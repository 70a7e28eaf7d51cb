/* Device prelude: what `#include "cluda.h"` resolves to when a kernel is
 * compiled for gfx950.  It gives kernel text written against the reference's
 * preludes (src/cluda_cuda.h:3-171, src/cluda_opencl.h:3-187) the same
 * vocabulary: KERNEL / WITHIN_KERNEL / GLOBAL_MEM / LOCAL_MEM, LID_n / LDIM_n /
 * GID_n / GDIM_n, the ga_* scalar types, ga_half with conversions, the
 * atom_add_* / atom_xchg_* family, and the usual math constants.
 * Wavefronts are 64 lanes wide. */
#ifndef CLUDA_H
#define CLUDA_H

#define local_barrier() __syncthreads()
#define WITHIN_KERNEL extern "C" __device__
#define KERNEL extern "C" __global__
#define GLOBAL_MEM /* flat address space */
#define LOCAL_MEM __shared__
#define LOCAL_MEM_ARG /* flat address space */

#define LID_0 threadIdx.x
#define LID_1 threadIdx.y
#define LID_2 threadIdx.z
#define LDIM_0 blockDim.x
#define LDIM_1 blockDim.y
#define LDIM_2 blockDim.z
#define GID_0 blockIdx.x
#define GID_1 blockIdx.y
#define GID_2 blockIdx.z
#define GDIM_0 gridDim.x
#define GDIM_1 gridDim.y
#define GDIM_2 gridDim.z

typedef unsigned char ga_bool;
typedef signed char ga_byte;
typedef unsigned char ga_ubyte;
typedef short ga_short;
typedef unsigned short ga_ushort;
typedef int ga_int;
typedef unsigned int ga_uint;
typedef long long ga_long;
typedef unsigned long long ga_ulong;
typedef float ga_float;
typedef double ga_double;
typedef __SIZE_TYPE__ ga_size;
typedef __PTRDIFF_TYPE__ ga_ssize;

#define GA_WARP_SIZE 64
/* Dynamic local memory arrives CUDA-style: declared in the body, sized at
 * launch. */
#define GA_DECL_SHARED_PARAM(type, name)
#define GA_DECL_SHARED_BODY(type, name) extern __shared__ type name[];

#ifdef NAN
#undef NAN
#endif
#define NAN __builtin_nanf("")
#ifdef INFINITY
#undef INFINITY
#endif
#define INFINITY __builtin_inff()
#ifndef MAXFLOAT
#define MAXFLOAT 3.402823466E+38F
#endif
#ifndef HUGE_VALF
#define HUGE_VALF __builtin_inff()
#endif
#ifndef HUGE_VAL
#define HUGE_VAL __builtin_inf()
#endif
#ifndef M_E
#define M_E 2.7182818284590452354
#define M_LOG2E 1.4426950408889634074
#define M_LOG10E 0.43429448190325182765
#define M_LN2 0.69314718055994530942
#define M_LN10 2.30258509299404568402
#define M_PI 3.14159265358979323846
#define M_PI_2 1.57079632679489661923
#define M_PI_4 0.78539816339744830962
#define M_1_PI 0.31830988618379067154
#define M_2_PI 0.63661977236758134308
#define M_2_SQRTPI 1.12837916709551257390
#define M_SQRT2 1.41421356237309504880
#define M_SQRT1_2 0.70710678118654752440
#endif

/* IEEE binary16 carried as raw bits; conversions use the hardware
 * converters (float->half rounds to nearest even). */
struct ga_half {
  ga_ushort data;
};

static __device__ inline float ga_half2float(ga_half h) {
  return (float)__builtin_bit_cast(_Float16, h.data);
}
static __device__ inline ga_half ga_float2half(float f) {
  ga_half r;
  r.data = __builtin_bit_cast(ga_ushort, (_Float16)f);
  return r;
}

/* atom_{add,xchg}_<type><space>: type i/I/l/L/f/d/e = int/uint/long/ulong/
 * float/double/half, space g/l = global/local.  Flat addressing makes the
 * two spaces one implementation. */
#define atom_add_ig(a, b) atomicAdd(a, b)
#define atom_add_il(a, b) atomicAdd(a, b)
#define atom_xchg_ig(a, b) atomicExch(a, b)
#define atom_xchg_il(a, b) atomicExch(a, b)
#define atom_add_Ig(a, b) atomicAdd(a, b)
#define atom_add_Il(a, b) atomicAdd(a, b)
#define atom_xchg_Ig(a, b) atomicExch(a, b)
#define atom_xchg_Il(a, b) atomicExch(a, b)
static __device__ inline ga_long atom_add_lg(ga_long *addr, ga_long val) {
  return (ga_long)atomicAdd((ga_ulong *)addr, (ga_ulong)val);
}
#define atom_add_ll(a, b) atom_add_lg(a, b)
static __device__ inline ga_long atom_xchg_lg(ga_long *addr, ga_long val) {
  return (ga_long)atomicExch((ga_ulong *)addr, (ga_ulong)val);
}
#define atom_xchg_ll(a, b) atom_xchg_lg(a, b)
#define atom_add_Lg(a, b) atomicAdd(a, b)
#define atom_add_Ll(a, b) atomicAdd(a, b)
#define atom_xchg_Lg(a, b) atomicExch(a, b)
#define atom_xchg_Ll(a, b) atomicExch(a, b)
#define atom_add_fg(a, b) atomicAdd(a, b)
#define atom_add_fl(a, b) atomicAdd(a, b)
#define atom_xchg_fg(a, b) atomicExch(a, b)
#define atom_xchg_fl(a, b) atomicExch(a, b)
#define atom_add_dg(a, b) atomicAdd(a, b)
#define atom_add_dl(a, b) atomicAdd(a, b)
static __device__ inline ga_double atom_xchg_dg(ga_double *addr, ga_double val) {
  ga_ulong old = atomicExch((ga_ulong *)addr, __builtin_bit_cast(ga_ulong, val));
  return __builtin_bit_cast(ga_double, old);
}
#define atom_xchg_dl(a, b) atom_xchg_dg(a, b)

/* A half shares a 32-bit word with its neighbour: compare-and-swap the word. */
static __device__ inline ga_half atom_add_eg(ga_half *addr, ga_half val) {
  ga_size a = (ga_size)addr;
  ga_uint *word = (ga_uint *)(a & ~(ga_size)2);
  const int hi = (a & 2) != 0;
  ga_uint old = *word, seen;
  ga_half cur;
  do {
    seen = old;
    cur.data = hi ? (ga_ushort)(seen >> 16) : (ga_ushort)(seen & 0xffffu);
    ga_uint s = ga_float2half(ga_half2float(val) + ga_half2float(cur)).data;
    ga_uint repl = hi ? ((seen & 0x0000ffffu) | (s << 16)) : ((seen & 0xffff0000u) | s);
    old = atomicCAS(word, seen, repl);
  } while (old != seen);
  cur.data = hi ? (ga_ushort)(old >> 16) : (ga_ushort)(old & 0xffffu);
  return cur;
}
#define atom_add_el(a, b) atom_add_eg(a, b)
static __device__ inline ga_half atom_xchg_eg(ga_half *addr, ga_half val) {
  ga_size a = (ga_size)addr;
  ga_uint *word = (ga_uint *)(a & ~(ga_size)2);
  const int hi = (a & 2) != 0;
  ga_uint old = *word, seen;
  do {
    seen = old;
    ga_uint repl = hi ? ((seen & 0x0000ffffu) | ((ga_uint)val.data << 16))
                      : ((seen & 0xffff0000u) | val.data);
    old = atomicCAS(word, seen, repl);
  } while (old != seen);
  ga_half r;
  r.data = hi ? (ga_ushort)(old >> 16) : (ga_ushort)(old & 0xffffu);
  return r;
}
#define atom_xchg_el(a, b) atom_xchg_eg(a, b)

#endif /* CLUDA_H */
