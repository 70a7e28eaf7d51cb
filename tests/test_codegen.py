"""Generated kernel text compiles for gfx950 (the compiler needs no device), and the
device prelude offers the vocabulary kernels written for the reference use.
No kernel is launched here."""
import ctypes as C

import pytest

from libgpuarray_amd import _lib

gen_elemwise = _lib.extension("hip_elemwise_source", C.c_void_p,
                              [C.c_char_p, C.c_char_p, C.c_uint, C.POINTER(_lib.ElemwiseArg),
                               C.c_int, C.c_int, C.c_uint, C.c_int, C.c_uint])
gen_reduction = _lib.extension("hip_reduction_source", C.c_void_p,
                               [C.c_int, C.c_int, C.c_int, C.c_int, C.c_uint, C.c_uint, C.c_uint])
compile_only = _lib.extension("hip_compile_only", C.c_int,
                              [C.c_uint, C.POINTER(C.c_char_p), C.POINTER(C.c_size_t),
                               C.POINTER(C.c_char_p)])
libc = C.CDLL(None)
libc.free.argtypes = [C.c_void_p]


def take_string(p):
    assert p, "generator returned NULL"
    s = C.string_at(p)
    libc.free(p)
    return s


def compile_src(src):
    arr = (C.c_char_p * 1)(src)
    log = C.c_char_p()
    err = compile_only(1, arr, None, C.byref(log))
    return err, (log.value or b"").decode(errors="replace")


def args_of(spec):
    arr = (_lib.ElemwiseArg * len(spec))()
    keep = []
    for i, (name, tc, fl) in enumerate(spec):
        keep.append(name.encode())
        arr[i].name, arr[i].typecode, arr[i].flags = keep[-1], tc, fl
    arr._keep = keep
    return arr


R, W, S = _lib.GE_READ, _lib.GE_WRITE, _lib.GE_SCALAR | _lib.GE_READ
F32 = [("a", _lib.GA_FLOAT, R), ("b", _lib.GA_FLOAT, R), ("c", _lib.GA_FLOAT, W)]


def test_flat_kernel_text_shape():
    src = take_string(gen_elemwise(b"", b"c = a*b + 0.5f", 3, args_of(F32), 0, 0, 0, 0, 0)).decode()
    # same argument order as the reference's flat kernel
    # (src/gpuarray_elemwise.c:472-488): n, then data+offset per array
    assert "elem(const ga_size n, GLOBAL_MEM ga_float *a_p, const ga_size a_offset" in src
    assert "ga_chunk16" in src and "__builtin_nontemporal_load" in src
    assert "c = a*b + 0.5f;" in src
    err, log = compile_src(src.encode())
    assert err == 0, log


@pytest.mark.parametrize("nd,idx64,tmask", [(1, 0, 0), (2, 0, 0), (4, 1, 0), (2, 0, 1), (3, 1, 5)])
def test_strided_variants_compile(nd, idx64, tmask):
    src = take_string(gen_elemwise(b"", b"c = a*b + 0.5f", 3, args_of(F32), 0, 1, nd, idx64, tmask))
    err, log = compile_src(src)
    assert err == 0, log


@pytest.mark.parametrize("nd,idx64,tmask,umask", [(1, 0, 0, 0b101), (2, 0, 0b001, 0b110),
                                                  (3, 1, 0b100, 0b011), (2, 0, 0, 0b100)])
def test_four_elements_per_lane_variants_compile(nd, idx64, tmask, umask):
    src = take_string(gen_elemwise(b"", b"c = a*b + 0.5f", 3, args_of(F32), 0, 2, nd, idx64,
                                   tmask | (umask << 16)))
    assert b"ga_chunk16" in src
    err, log = compile_src(src)
    assert err == 0, log


@pytest.mark.parametrize("f,planes,flags", [(3, 0, 0b00100), (11, 0, 0b01111), (5, 1, 0b11110), (8, 1, 0b101100)])
def test_narrow_planes_in_registers_compile(f, planes, flags):
    """Variant 14: (N, f) against its transpose with a lane holding a chunk of
    positions by the whole short dim; arrays with the short dim innermost direct or
    through the LDS, the others as chunks, an operand constant along the long dim."""
    src = take_string(gen_elemwise(b"", b"c = a*b + 0.5f", 3, args_of(F32), 0, 14, f | (planes << 8), flags,
                                   0b001 | (0b100 << 16)))
    text = src.decode()
    assert "union { ga_chunk16 c[%d]; ga_float e[%d]; } a_r;" % (f, 4 * f) in text     # a lane's 4 f elements of a
    assert ("LOCAL_MEM ga_chunk16 a_s[%d];" % (256 * f) in text) == bool(flags & 8)      # staged or not
    assert ("ga_float b_z[%d];" % f in text) == bool(flags & 32)                        # fetched once per row
    assert text.count("c = a*b + 0.5f;") == 4 * f
    err, log = compile_src(src)
    assert err == 0, log


def test_narrow_planes_of_mixed_element_sizes_compile():
    """Bytes with the short dim innermost and floats in planes: 16 positions per lane,
    four chunks of floats per row."""
    spec = [("a", _lib.GA_UBYTE, R), ("c", _lib.GA_FLOAT, W)]
    src = take_string(gen_elemwise(b"", b"c = a", 2, args_of(spec), 0, 14, 3, 0b00100, 0b01 | (0b10 << 16)))
    text = src.decode()
    assert "union { ga_chunk16 c[3]; ga_ubyte e[48]; } a_r;" in text
    assert "union { ga_chunk16 c[4]; ga_float e[16]; } c_r[3];" in text
    err, log = compile_src(src)
    assert err == 0, log


@pytest.mark.parametrize("f,planes,flags", [(17, 0, 0b00100), (33, 1, 0b10111), (64, 0, 0b00000)])
def test_narrow_planes_through_the_lds_compile(f, planes, flags):
    """Variant 15: short extents of 17 to 64, a group's piece whole through the LDS."""
    src = take_string(gen_elemwise(b"", b"c = a*b + 0.5f", 3, args_of(F32), 0, 15, f | (planes << 8), flags,
                                   0b001 | (0b110 << 16)))
    assert ("LOCAL_MEM ga_float a_s[%d];" % (260 * (f | 1))).encode() in src
    err, log = compile_src(src)
    assert err == 0, log


@pytest.mark.parametrize("f,planes,flags,tc", [(3, 0, 0b00100, "GA_FLOAT"), (20, 1, 0b01001, "GA_FLOAT"),
                                               (3, 0, 0b11100, "GA_UBYTE"), (2, 1, 0b00100, "GA_DOUBLE")])
def test_tiles_of_records_compile(f, planes, flags, tc):
    """Variant 16: matrices of short records against their transposes; rectangular
    tiles and windows moved onto the result's 64-byte blocks, tiles numbered along Y
    first, element sizes of 1, 4 and 8 bytes."""
    t = getattr(_lib, tc)
    spec = [("a", t, R), ("b", t, R), ("c", t, W)]
    src = take_string(gen_elemwise(b"", b"c = a + b", 3, args_of(spec), 0, 16, f | (planes << 8), flags,
                                   0b001 | (0b110 << 16)))
    text = src.decode()
    assert "LOCAL_MEM" in text and "a_s[" in text and "b_s[" not in text      # only the transposed operand is staged
    assert ("ga_sh" in text) == bool(flags & 8)
    assert ("GDIM_0 & ~7u" in text) == bool(flags & 16)
    err, log = compile_src(src)
    assert err == 0, log


def test_mixed_types_scalars_and_half_compile():
    spec = [("x", _lib.GA_HALF, R), ("k", _lib.GA_DOUBLE, S), ("m", _lib.GA_UBYTE, R),
            ("y", _lib.GA_HALF, R | W), ("z", _lib.GA_LONG, W)]
    expr = b"y = x * (ga_float)k + y; z = (ga_long)m + (ga_long)y"
    for strided, nd, tm in [(0, 0, 0), (1, 2, 0), (1, 2, 0b1001)]:
        src = take_string(gen_elemwise(b"", expr, 5, args_of(spec), _lib.GE_CONVERT_F16, strided,
                                       nd, 0, tm))
        err, log = compile_src(src)
        assert err == 0, log


def test_preamble_and_prelude_vocabulary():
    # pygpu/tests/test_elemwise.py:310-346 uses INFINITY from a preamble
    pre = (b"WITHIN_KERNEL ga_float clampinf(ga_float v) { return v > 1e30f ? INFINITY : v; }\n"
           b"#define TWO_PI (2 * M_PI)\n")
    expr = b"c = clampinf(a) + (ga_float)TWO_PI * b + (isnan(a) ? NAN : 0.0f)"
    src = take_string(gen_elemwise(pre, expr, 3, args_of(F32), 0, 0, 0, 0, 0))
    err, log = compile_src(src)
    assert err == 0, log
    # a hand-written kernel in the reference's dialect
    user = b"""#include "cluda.h"
KERNEL void k(GLOBAL_MEM ga_float *x, ga_size n, GLOBAL_MEM ga_half *h, GLOBAL_MEM ga_int *cnt,
              GLOBAL_MEM ga_long *lc, GLOBAL_MEM ga_double *dc) {
  GA_DECL_SHARED_BODY(ga_float, tile)
  LOCAL_MEM ga_uint hits[GA_WARP_SIZE];
  ga_size i = GID_0 * LDIM_0 + LID_0;
  tile[LID_0] = i < n ? x[i] : 0;
  hits[LID_0 % GA_WARP_SIZE] = 0;
  local_barrier();
  if (i < n) {
    h[i] = ga_float2half(ga_half2float(h[i]) + tile[LID_0]);
    atom_add_ig(cnt, 1); atom_add_lg(lc, 1); atom_add_dg(dc, 1.0); atom_add_fg(x, 1.0f);
    atom_add_Il(&hits[0], 1u); atom_xchg_ig(cnt, 2); atom_add_eg(h, h[i]); atom_xchg_eg(h, h[i]);
  }
  if (GDIM_0 > 1 && LID_1 + LID_2 + GID_1 + GID_2 + LDIM_1 + LDIM_2 + GDIM_1 + GDIM_2 > 1000) x[0] = MAXFLOAT;
}
"""
    err, log = compile_src(user)
    assert err == 0, log


def test_device_runtime_vocabulary_without_toolchain_headers():
    """Kernel text is compiled without the toolchain's HIP headers; the
    library's own device runtime supplies what kernels may use: the HIP
    spelling of kernels and indices, atomics, and the C math library with
    <cmath>-style overloads (float stays float, integers go to double)."""
    user = b"""#include <hip/hip_runtime.h>
template <class A, class B> struct same_t { static const bool v = false; };
template <class A> struct same_t<A, A> { static const bool v = true; };
static_assert(same_t<decltype(exp(1.0f)), float>::v, "exp(float) is the float function");
static_assert(same_t<decltype(exp(1)), double>::v, "integers promote to double");
static_assert(same_t<decltype(pow(2.0f, 3.0f)), float>::v, "pow(float, float)");
static_assert(same_t<decltype(pow(2.0f, 3)), float>::v, "pow(float, int)");
static_assert(same_t<decltype(pow(2.0f, 3.0)), double>::v, "mixed arguments promote");
static_assert(same_t<decltype(fmod(2.0f, 3)), double>::v, "mixed arguments promote");
static_assert(same_t<decltype(fabs(-1.0f)), float>::v, "fabs(float)");
static_assert(same_t<decltype(abs(-1.0f)), float>::v, "abs(float)");
static_assert(same_t<decltype(abs(-1LL)), long long>::v, "abs(long long)");
static_assert(same_t<decltype(min(1u, 2u)), unsigned>::v, "min(unsigned, unsigned)");
extern "C" __global__ void __launch_bounds__(256) k(float *x, double *d, int *cnt, unsigned long long *big, int n) {
  __shared__ float tile[256];
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  tile[threadIdx.x] = i < n ? x[i] : 0.0f;
  __syncthreads();
  if (i >= n) return;
  float v = tile[threadIdx.x ^ 1];
  v = expf(v) + logf(v) + log2(v) + log10(v) + log1p(v) + expm1(v) + exp2(v) + exp10(v);
  v += sin(v) + cos(v) + tan(v) + asin(v) + acos(v) + atan(v) + atan2(v, 2.0f) + sinh(v) + cosh(v) + tanh(v);
  v += asinh(v) + acosh(v) + atanh(v) + sqrt(v) + rsqrt(v) + cbrt(v) + hypot(v, 1.0f) + pow(v, 1.5f);
  v += floor(v) + ceil(v) + trunc(v) + round(v) + rint(v) + nearbyint(v) + fmod(v, 3.0f) + remainder(v, 3.0f);
  v += fmin(v, 1.0f) + fmax(v, 1.0f) + fdim(v, 1.0f) + copysign(v, -1.0f) + fma(v, v, v) + ldexp(v, 2);
  v += erf(v) + erfc(v) + lgamma(v) + tgamma(v) + nextafter(v, 0.0f) + logb(v) + (float)ilogb(v);
  float ip, sn, cs; int e, q;
  v += modf(v, &ip) + ip + frexp(v, &e) + (float)e + remquo(v, 3.0f, &q) + (float)q;
  sincos(v, &sn, &cs);
  v += sn + cs + (isnan(v) || isinf(v) || !isfinite(v) || signbit(v) ? 1.0f : 0.0f);
  v += (float)(lrint(v) + llrint(v) + lround(v) + llround(v));
  d[i] = exp((double)v) + pow((double)v, 2) + sqrt(i) + erf((double)v) + fmod((double)v, 2.0) + fabs((double)v);
  x[i] = v + (float)min(i, n) + (float)max(i, 3) + (float)abs(i - 7) + (float)(__popc(i) + __clz(i) + __ffs(i));
  atomicAdd(cnt, 1); atomicAdd(x, 1.0f); atomicAdd(d, 1.0); atomicAdd(big, 1ull);
  atomicMax(cnt, i); atomicMin(cnt, i); atomicExch(cnt, 2); atomicCAS(cnt, 2, 3); atomicOr(cnt, 1); atomicAnd(cnt, 7);
  if (gridDim.x > 1000000 && blockIdx.y + blockIdx.z + threadIdx.y + threadIdx.z + blockDim.y + gridDim.z > 5) __threadfence();
}
"""
    err, log = compile_src(user)
    assert err == 0, log


def test_bad_expression_is_a_compile_error_with_a_log():
    src = take_string(gen_elemwise(b"", b"c = a +* undefined_name", 3, args_of(F32), 0, 0, 0, 0, 0))
    err, log = compile_src(src)
    assert err == _lib.GA_IMPL_ERROR
    assert "undefined_name" in log or "error" in log


@pytest.mark.parametrize("cfg", [
    # op, src, d0, d1, G, V, U
    (_lib.GA_REDUCE_SUM, _lib.GA_FLOAT, _lib.GA_FLOAT, _lib.GA_LONG, 256, 4, 4),
    (_lib.GA_REDUCE_SUM, _lib.GA_HALF, _lib.GA_FLOAT, _lib.GA_LONG, 256, 1, 2),
    (_lib.GA_REDUCE_SUM, _lib.GA_INT, _lib.GA_LONG, _lib.GA_LONG, 256, 1, 4),
    (_lib.GA_REDUCE_MAXANDARGMAX, _lib.GA_FLOAT, _lib.GA_FLOAT, _lib.GA_ULONG, 64, 4, 4),
    (_lib.GA_REDUCE_ARGMIN, _lib.GA_DOUBLE, _lib.GA_DOUBLE, _lib.GA_LONG, 64, 2, 4),
    (_lib.GA_REDUCE_ANY, _lib.GA_UBYTE, _lib.GA_BOOL, _lib.GA_LONG, 64, 1, 4),
    (_lib.GA_REDUCE_ALL, _lib.GA_HALF, _lib.GA_BOOL, _lib.GA_LONG, 64, 8, 1),
    (_lib.GA_REDUCE_XOR, _lib.GA_USHORT, _lib.GA_USHORT, _lib.GA_LONG, 256, 8, 2),
    (_lib.GA_REDUCE_PRODNZ, _lib.GA_BYTE, _lib.GA_HALF, _lib.GA_LONG, 64, 16, 1),
])
def test_reduction_variants_compile(cfg):
    src = take_string(gen_reduction(*cfg))
    assert b"redux_row" in src and b"redux_col" in src and b"redux_final" in src
    err, log = compile_src(src)
    assert err == 0, log


def test_reduction_plan_struct_matches_the_kernel_side():
    # 7 arrays of 8 x int64 + 6 x int64 + 4 x int32
    import re
    src = take_string(gen_reduction(0, _lib.GA_FLOAT, _lib.GA_FLOAT, _lib.GA_LONG, 64, 1, 1)).decode()
    body = re.search(r"struct rd_plan \{(.*?)\};", src, re.S).group(1)
    assert body.count("[RD_MAXD]") == 7 and "#define RD_MAXD 8" in src


def test_text_that_needs_the_toolchain_headers_gets_a_second_compile():
    """The library's device runtime covers what its own generators use; a
    caller's kernel may use more of HIP.  What fails on a missing header or
    identifier is compiled once more through hipRTC (needs no device)."""
    plain = b'#include "cluda.h"\nKERNEL void k(GLOBAL_MEM float *a) { a[LID_0] = 1.0f; }'
    err, log = compile_src(plain)
    assert err == 0 and "second try" not in log
    rich = (b'#include <hip/hip_fp16.h>\n'
            b'extern "C" __global__ void k(__half *a, float4 *b) {\n'
            b'  a[threadIdx.x] = __float2half(1.0f); b[0] = make_float4(1, 2, 3, 4);\n'
            b'  a[1] = __float2half((float)__shfl(5, 0)); printf("%d", (int)clock64()); }')
    err, log = compile_src(rich)
    assert err == 0, log[-800:]
    # the atomics callers most often reach for on 64-bit words are in the small runtime itself
    words = (b'#include "cluda.h"\nKERNEL void k(GLOBAL_MEM unsigned long *a, GLOBAL_MEM long long *b) {\n'
             b'  atomicAdd(a, 1ul); atomicMax(b, 3ll); atomicCAS(a, 1ul, 2ul); }')
    err, log = compile_src(words)
    assert err == 0 and log == "", log[-400:]
    err, log = compile_src(b'extern "C" __global__ void k(int *p) { p[0] = no_such_thing(3); }')
    assert err != 0 and "no_such_thing" in log and "second try" in log
