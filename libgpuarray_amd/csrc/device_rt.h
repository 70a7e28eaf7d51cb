/* Device-side runtime for kernels compiled at run time for gfx950.
 *
 * Kernel text is compiled as HIP by the code-object manager with the
 * toolchain's own headers left out (-nogpuinc): parsing those costs a quarter
 * of a second per kernel, more than compiling most kernels does.  This file
 * is put in front of every kernel instead and supplies what kernel text may
 * rely on without including anything:
 *   - __global__ / __device__ / __shared__ / __launch_bounds__,
 *     threadIdx / blockIdx / blockDim / gridDim, __syncthreads();
 *   - atomicAdd / atomicSub / atomicExch / atomicCAS / atomicMin / atomicMax /
 *     atomicAnd / atomicOr / atomicXor (relaxed, device scope) on int, unsigned
 *     int, unsigned long and unsigned long long (add and exchange on float, add
 *     on double, min and max on long long as well);
 *   - the C math library for float and double under its C names (expf, exp,
 *     ...), its C++ overloads on the unsuffixed names (exp(float) is the float
 *     function; integers promote to double; mixed arguments to the wider type),
 *     abs / min / max, isnan / isinf / isfinite / signbit, and a few integer
 *     intrinsics (__popc, __clz, __ffs, __brev, __mulhi, __umulhi).
 * Math functions resolve to compiler builtins where the compiler expands them
 * itself and to the device library (ocml) otherwise, the same split the
 * toolchain's HIP headers make, so results are those of a hipcc build. */
#ifndef GA_DEVICE_RT_H
#define GA_DEVICE_RT_H

#define __host__ __attribute__((host))
#define __device__ __attribute__((device))
#define __global__ __attribute__((global))
#define __shared__ __attribute__((shared))
#define __constant__ __attribute__((constant))
#define __noinline__ __attribute__((noinline))
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...) __attribute__((launch_bounds(__VA_ARGS__)))
#define GA_RT_FN static __device__ inline __attribute__((always_inline))

extern "C" __device__ __attribute__((const)) __SIZE_TYPE__ __ockl_get_num_groups(unsigned int);

struct ga_rt_uint3 {
  unsigned int x, y, z;
};
#define threadIdx                                                          \
  (ga_rt_uint3{__builtin_amdgcn_workitem_id_x(), __builtin_amdgcn_workitem_id_y(), \
               __builtin_amdgcn_workitem_id_z()})
#define blockIdx                                                             \
  (ga_rt_uint3{__builtin_amdgcn_workgroup_id_x(), __builtin_amdgcn_workgroup_id_y(), \
               __builtin_amdgcn_workgroup_id_z()})
#define blockDim                                                                 \
  (ga_rt_uint3{__builtin_amdgcn_workgroup_size_x(), __builtin_amdgcn_workgroup_size_y(), \
               __builtin_amdgcn_workgroup_size_z()})
#define gridDim                                                                      \
  (ga_rt_uint3{(unsigned int)__ockl_get_num_groups(0), (unsigned int)__ockl_get_num_groups(1), \
               (unsigned int)__ockl_get_num_groups(2)})
#define warpSize 64

GA_RT_FN void __syncthreads() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}
GA_RT_FN void __threadfence() { __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "agent"); }
GA_RT_FN void __threadfence_block() { __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup"); }

/* ---- atomics: relaxed, device scope, returning the old value -------------- */
#define GA_RT_ATOMIC(name, builtin, T)                                               \
  GA_RT_FN T name(T *p, T v) {                                                       \
    return builtin(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);                \
  }
#define GA_RT_ATOMIC_INTS(name, builtin) \
  GA_RT_ATOMIC(name, builtin, int)       \
  GA_RT_ATOMIC(name, builtin, unsigned int) \
  GA_RT_ATOMIC(name, builtin, unsigned long) \
  GA_RT_ATOMIC(name, builtin, unsigned long long)
GA_RT_ATOMIC_INTS(atomicAdd, __hip_atomic_fetch_add)
GA_RT_ATOMIC(atomicAdd, __hip_atomic_fetch_add, float)
GA_RT_ATOMIC(atomicAdd, __hip_atomic_fetch_add, double)
GA_RT_ATOMIC_INTS(atomicSub, __hip_atomic_fetch_sub)
GA_RT_ATOMIC_INTS(atomicExch, __hip_atomic_exchange)
GA_RT_ATOMIC(atomicExch, __hip_atomic_exchange, float)
GA_RT_ATOMIC_INTS(atomicMin, __hip_atomic_fetch_min)
GA_RT_ATOMIC(atomicMin, __hip_atomic_fetch_min, long long)
GA_RT_ATOMIC_INTS(atomicMax, __hip_atomic_fetch_max)
GA_RT_ATOMIC(atomicMax, __hip_atomic_fetch_max, long long)
GA_RT_ATOMIC_INTS(atomicAnd, __hip_atomic_fetch_and)
GA_RT_ATOMIC_INTS(atomicOr, __hip_atomic_fetch_or)
GA_RT_ATOMIC_INTS(atomicXor, __hip_atomic_fetch_xor)
#define GA_RT_CAS(T)                                                                        \
  GA_RT_FN T atomicCAS(T *p, T expected, T desired) {                                       \
    __hip_atomic_compare_exchange_strong(p, &expected, desired, __ATOMIC_RELAXED,           \
                                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);       \
    return expected;                                                                        \
  }
GA_RT_CAS(int)
GA_RT_CAS(unsigned int)
GA_RT_CAS(unsigned long)
GA_RT_CAS(unsigned long long)

/* ---- integer helpers -------------------------------------------------------- */
GA_RT_FN int abs(int x) { return __builtin_abs(x); }
GA_RT_FN long labs(long x) { return __builtin_labs(x); }
GA_RT_FN long long llabs(long long x) { return __builtin_llabs(x); }
GA_RT_FN long abs(long x) { return __builtin_labs(x); }
GA_RT_FN long long abs(long long x) { return __builtin_llabs(x); }
GA_RT_FN int __popc(unsigned int x) { return __builtin_popcount(x); }
GA_RT_FN int __popcll(unsigned long long x) { return __builtin_popcountll(x); }
GA_RT_FN int __clz(int x) { return x == 0 ? 32 : __builtin_clz((unsigned int)x); }
GA_RT_FN int __clzll(long long x) { return x == 0 ? 64 : __builtin_clzll((unsigned long long)x); }
GA_RT_FN int __ffs(int x) { return __builtin_ffs(x); }
GA_RT_FN int __ffsll(long long x) { return __builtin_ffsll(x); }
GA_RT_FN unsigned int __brev(unsigned int x) { return __builtin_bitreverse32(x); }
GA_RT_FN unsigned long long __brevll(unsigned long long x) { return __builtin_bitreverse64(x); }
GA_RT_FN int __mulhi(int a, int b) { return (int)(((long long)a * b) >> 32); }
GA_RT_FN unsigned int __umulhi(unsigned int a, unsigned int b) {
  return (unsigned int)(((unsigned long long)a * b) >> 32);
}
#define GA_RT_MINMAX(T)                              \
  GA_RT_FN T min(T a, T b) { return b < a ? b : a; } \
  GA_RT_FN T max(T a, T b) { return a < b ? b : a; }
GA_RT_MINMAX(int)
GA_RT_MINMAX(unsigned int)
GA_RT_MINMAX(long)
GA_RT_MINMAX(unsigned long)
GA_RT_MINMAX(long long)
GA_RT_MINMAX(unsigned long long)

/* ---- math ------------------------------------------------------------------- */
/* device library entry points used below */
#define GA_RT_PRIVATE __attribute__((opencl_private))
#define GA_RT_OCML1(NAME)                                                        \
  extern "C" __device__ __attribute__((const)) float __ocml_##NAME##_f32(float); \
  extern "C" __device__ __attribute__((const)) double __ocml_##NAME##_f64(double);
#define GA_RT_OCML2(NAME)                                                               \
  extern "C" __device__ __attribute__((const)) float __ocml_##NAME##_f32(float, float); \
  extern "C" __device__ __attribute__((const)) double __ocml_##NAME##_f64(double, double);
GA_RT_OCML1(acos) GA_RT_OCML1(acosh) GA_RT_OCML1(asin) GA_RT_OCML1(asinh) GA_RT_OCML1(atan)
GA_RT_OCML1(atanh) GA_RT_OCML1(cbrt) GA_RT_OCML1(cos) GA_RT_OCML1(cosh) GA_RT_OCML1(cospi)
GA_RT_OCML1(erf) GA_RT_OCML1(erfc) GA_RT_OCML1(erfcinv) GA_RT_OCML1(erfcx) GA_RT_OCML1(erfinv)
GA_RT_OCML1(expm1) GA_RT_OCML1(lgamma) GA_RT_OCML1(log1p) GA_RT_OCML1(logb) GA_RT_OCML1(ncdf)
GA_RT_OCML1(ncdfinv) GA_RT_OCML1(rcbrt) GA_RT_OCML1(rsqrt) GA_RT_OCML1(sin) GA_RT_OCML1(sinh)
GA_RT_OCML1(sinpi) GA_RT_OCML1(tan) GA_RT_OCML1(tanh) GA_RT_OCML1(tgamma) GA_RT_OCML1(i0)
GA_RT_OCML1(i1) GA_RT_OCML1(j0) GA_RT_OCML1(j1) GA_RT_OCML1(y0) GA_RT_OCML1(y1)
GA_RT_OCML2(atan2) GA_RT_OCML2(fdim) GA_RT_OCML2(fmod) GA_RT_OCML2(hypot) GA_RT_OCML2(nextafter)
GA_RT_OCML2(pow) GA_RT_OCML2(remainder) GA_RT_OCML2(rhypot)
extern "C" __device__ __attribute__((const)) double __ocml_exp_f64(double);
extern "C" __device__ __attribute__((const)) double __ocml_exp2_f64(double);
extern "C" __device__ __attribute__((const)) double __ocml_exp10_f64(double);
extern "C" __device__ __attribute__((const)) double __ocml_log_f64(double);
extern "C" __device__ __attribute__((const)) double __ocml_log2_f64(double);
extern "C" __device__ __attribute__((const)) double __ocml_log10_f64(double);
extern "C" __device__ __attribute__((const)) int __ocml_ilogb_f32(float);
extern "C" __device__ __attribute__((const)) int __ocml_ilogb_f64(double);
extern "C" __device__ __attribute__((const)) float __ocml_pown_f32(float, int);
extern "C" __device__ __attribute__((const)) double __ocml_pown_f64(double, int);
extern "C" __device__ float __ocml_modf_f32(float, GA_RT_PRIVATE float *);
extern "C" __device__ double __ocml_modf_f64(double, GA_RT_PRIVATE double *);
extern "C" __device__ float __ocml_remquo_f32(float, float, GA_RT_PRIVATE int *);
extern "C" __device__ double __ocml_remquo_f64(double, double, GA_RT_PRIVATE int *);
extern "C" __device__ float __ocml_sincos_f32(float, GA_RT_PRIVATE float *);
extern "C" __device__ double __ocml_sincos_f64(double, GA_RT_PRIVATE double *);

/* one argument, float name NAMEf and double name NAME */
#define GA_RT_M1(NAME, impl32, impl64)                     \
  GA_RT_FN float NAME##f(float x) { return impl32(x); }    \
  GA_RT_FN double NAME(double x) { return impl64(x); }     \
  GA_RT_FN float NAME(float x) { return impl32(x); }       \
  template <class T>                                       \
  GA_RT_FN typename ga_rt_if_int<T>::type NAME(T x) {      \
    return impl64((double)x);                              \
  }
#define GA_RT_M1L(NAME) GA_RT_M1(NAME, __ocml_##NAME##_f32, __ocml_##NAME##_f64)
#define GA_RT_M1B(NAME) GA_RT_M1(NAME, __builtin_##NAME##f, __builtin_##NAME)
/* two arguments; mixed arithmetic arguments promote as in <cmath> */
#define GA_RT_M2(NAME, impl32, impl64)                                   \
  GA_RT_FN float NAME##f(float x, float y) { return impl32(x, y); }      \
  GA_RT_FN double NAME(double x, double y) { return impl64(x, y); }      \
  GA_RT_FN float NAME(float x, float y) { return impl32(x, y); }         \
  template <class A, class B>                                            \
  GA_RT_FN typename ga_rt_if_mixed<A, B>::type NAME(A x, B y) {          \
    return impl64((double)x, (double)y);                                 \
  }
#define GA_RT_M2L(NAME) GA_RT_M2(NAME, __ocml_##NAME##_f32, __ocml_##NAME##_f64)
#define GA_RT_M2B(NAME) GA_RT_M2(NAME, __builtin_##NAME##f, __builtin_##NAME)

template <class T, bool = __is_integral(T)>
struct ga_rt_if_int {};
template <class T>
struct ga_rt_if_int<T, true> {
  typedef double type;
};
template <class A, class B>
struct ga_rt_same {
  static const bool value = false;
};
template <class A>
struct ga_rt_same<A, A> {
  static const bool value = true;
};
/* two arithmetic arguments that are not (float, float) or (double, double) */
template <class A, class B,
          bool = __is_arithmetic(A) && __is_arithmetic(B) &&
                 !(ga_rt_same<A, B>::value && (ga_rt_same<A, float>::value || ga_rt_same<A, double>::value))>
struct ga_rt_if_mixed {};
template <class A, class B>
struct ga_rt_if_mixed<A, B, true> {
  typedef double type;
};

GA_RT_M1L(acos) GA_RT_M1L(acosh) GA_RT_M1L(asin) GA_RT_M1L(asinh) GA_RT_M1L(atan)
GA_RT_M1L(atanh) GA_RT_M1L(cbrt) GA_RT_M1L(cos) GA_RT_M1L(cosh) GA_RT_M1L(cospi)
GA_RT_M1L(erf) GA_RT_M1L(erfc) GA_RT_M1L(erfcinv) GA_RT_M1L(erfcx) GA_RT_M1L(erfinv)
GA_RT_M1L(expm1) GA_RT_M1L(lgamma) GA_RT_M1L(log1p) GA_RT_M1L(logb) GA_RT_M1L(rcbrt)
GA_RT_M1L(rsqrt) GA_RT_M1L(sin) GA_RT_M1L(sinh) GA_RT_M1L(sinpi) GA_RT_M1L(tan)
GA_RT_M1L(tanh) GA_RT_M1L(tgamma) GA_RT_M1L(j0) GA_RT_M1L(j1) GA_RT_M1L(y0) GA_RT_M1L(y1)
GA_RT_M1(normcdf, __ocml_ncdf_f32, __ocml_ncdf_f64)
GA_RT_M1(normcdfinv, __ocml_ncdfinv_f32, __ocml_ncdfinv_f64)
GA_RT_M1(cyl_bessel_i0, __ocml_i0_f32, __ocml_i0_f64)
GA_RT_M1(cyl_bessel_i1, __ocml_i1_f32, __ocml_i1_f64)
GA_RT_M1B(ceil) GA_RT_M1B(fabs) GA_RT_M1B(floor) GA_RT_M1B(nearbyint) GA_RT_M1B(rint)
GA_RT_M1B(round) GA_RT_M1B(sqrt) GA_RT_M1B(trunc)
GA_RT_M1(exp, __builtin_expf, __ocml_exp_f64)
GA_RT_M1(exp2, __builtin_exp2f, __ocml_exp2_f64)
GA_RT_M1(exp10, __builtin_exp10f, __ocml_exp10_f64)
GA_RT_M1(log, __builtin_logf, __ocml_log_f64)
GA_RT_M1(log2, __builtin_log2f, __ocml_log2_f64)
GA_RT_M1(log10, __builtin_log10f, __ocml_log10_f64)
GA_RT_M2L(atan2) GA_RT_M2L(fdim) GA_RT_M2L(fmod) GA_RT_M2L(hypot) GA_RT_M2L(nextafter)
GA_RT_M2L(remainder) GA_RT_M2L(rhypot)
GA_RT_M2B(copysign) GA_RT_M2B(fmax) GA_RT_M2B(fmin)
GA_RT_M2(pow, __ocml_pow_f32, __ocml_pow_f64)
GA_RT_FN float powif(float x, int n) { return __ocml_pown_f32(x, n); }
GA_RT_FN double powi(double x, int n) { return __ocml_pown_f64(x, n); }
GA_RT_FN float pow(float x, int n) { return __ocml_pown_f32(x, n); }
GA_RT_FN double pow(double x, int n) { return __ocml_pown_f64(x, n); }

GA_RT_FN float fmaf(float x, float y, float z) { return __builtin_fmaf(x, y, z); }
GA_RT_FN double fma(double x, double y, double z) { return __builtin_fma(x, y, z); }
GA_RT_FN float fma(float x, float y, float z) { return __builtin_fmaf(x, y, z); }
GA_RT_FN float fdividef(float x, float y) { return x / y; }
GA_RT_FN float ldexpf(float x, int e) { return __builtin_amdgcn_ldexpf(x, e); }
GA_RT_FN double ldexp(double x, int e) { return __builtin_amdgcn_ldexp(x, e); }
GA_RT_FN float ldexp(float x, int e) { return __builtin_amdgcn_ldexpf(x, e); }
GA_RT_FN float scalbnf(float x, int e) { return __builtin_amdgcn_ldexpf(x, e); }
GA_RT_FN double scalbn(double x, int e) { return __builtin_amdgcn_ldexp(x, e); }
GA_RT_FN float scalbn(float x, int e) { return __builtin_amdgcn_ldexpf(x, e); }
GA_RT_FN float frexpf(float x, int *e) { return __builtin_frexpf(x, e); }
GA_RT_FN double frexp(double x, int *e) { return __builtin_frexp(x, e); }
GA_RT_FN float frexp(float x, int *e) { return __builtin_frexpf(x, e); }
GA_RT_FN int ilogbf(float x) { return __ocml_ilogb_f32(x); }
GA_RT_FN int ilogb(double x) { return __ocml_ilogb_f64(x); }
GA_RT_FN int ilogb(float x) { return __ocml_ilogb_f32(x); }
GA_RT_FN long lrintf(float x) { return (long)__builtin_rintf(x); }
GA_RT_FN long lrint(double x) { return (long)__builtin_rint(x); }
GA_RT_FN long lrint(float x) { return (long)__builtin_rintf(x); }
GA_RT_FN long long llrintf(float x) { return (long long)__builtin_rintf(x); }
GA_RT_FN long long llrint(double x) { return (long long)__builtin_rint(x); }
GA_RT_FN long long llrint(float x) { return (long long)__builtin_rintf(x); }
GA_RT_FN long lroundf(float x) { return (long)__builtin_roundf(x); }
GA_RT_FN long lround(double x) { return (long)__builtin_round(x); }
GA_RT_FN long lround(float x) { return (long)__builtin_roundf(x); }
GA_RT_FN long long llroundf(float x) { return (long long)__builtin_roundf(x); }
GA_RT_FN long long llround(double x) { return (long long)__builtin_round(x); }
GA_RT_FN long long llround(float x) { return (long long)__builtin_roundf(x); }
GA_RT_FN float modff(float x, float *ip) {
  float t;
  float r = __ocml_modf_f32(x, (GA_RT_PRIVATE float *)&t);
  *ip = t;
  return r;
}
GA_RT_FN double modf(double x, double *ip) {
  double t;
  double r = __ocml_modf_f64(x, (GA_RT_PRIVATE double *)&t);
  *ip = t;
  return r;
}
GA_RT_FN float modf(float x, float *ip) { return modff(x, ip); }
GA_RT_FN float remquof(float x, float y, int *q) {
  int t;
  float r = __ocml_remquo_f32(x, y, (GA_RT_PRIVATE int *)&t);
  *q = t;
  return r;
}
GA_RT_FN double remquo(double x, double y, int *q) {
  int t;
  double r = __ocml_remquo_f64(x, y, (GA_RT_PRIVATE int *)&t);
  *q = t;
  return r;
}
GA_RT_FN float remquo(float x, float y, int *q) { return remquof(x, y, q); }
GA_RT_FN void sincosf(float x, float *s, float *c) {
  float t;
  *s = __ocml_sincos_f32(x, (GA_RT_PRIVATE float *)&t);
  *c = t;
}
GA_RT_FN void sincos(double x, double *s, double *c) {
  double t;
  *s = __ocml_sincos_f64(x, (GA_RT_PRIVATE double *)&t);
  *c = t;
}
GA_RT_FN void sincos(float x, float *s, float *c) { sincosf(x, s, c); }

GA_RT_FN float abs(float x) { return __builtin_fabsf(x); }
GA_RT_FN double abs(double x) { return __builtin_fabs(x); }
GA_RT_FN float min(float a, float b) { return __builtin_fminf(a, b); }
GA_RT_FN float max(float a, float b) { return __builtin_fmaxf(a, b); }
GA_RT_FN double min(double a, double b) { return __builtin_fmin(a, b); }
GA_RT_FN double max(double a, double b) { return __builtin_fmax(a, b); }
#define GA_RT_CLASSIFY(T)                                            \
  GA_RT_FN bool isnan(T x) { return __builtin_isnan(x); }            \
  GA_RT_FN bool isinf(T x) { return __builtin_isinf(x); }            \
  GA_RT_FN bool isfinite(T x) { return __builtin_isfinite(x); }      \
  GA_RT_FN bool signbit(T x) { return __builtin_signbit(x); }
GA_RT_CLASSIFY(float)
GA_RT_CLASSIFY(double)

#endif /* GA_DEVICE_RT_H */
