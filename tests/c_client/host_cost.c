/* Host side of a call, per call, with launches that return at once (the
 * stand-in runtime of tests/mock_runtime): what the library itself spends
 * between the caller and hipModuleLaunchKernel.  Prints one line per entry
 * point: name and microseconds per call. */
#include <stdio.h>
#include <stdlib.h>
#include <time.h>
#include <gpuarray/array.h>
#include <gpuarray/buffer.h>
#include <gpuarray/elemwise.h>
#include <gpuarray/error.h>
#include <gpuarray/reduction.h>

static double now_us(void) {
  struct timespec t;
  clock_gettime(CLOCK_MONOTONIC, &t);
  return t.tv_sec * 1e6 + t.tv_nsec * 1e-3;
}

#define CHECK(call)                                               \
  do {                                                            \
    if ((call) != GA_NO_ERROR) {                                  \
      fprintf(stderr, "%s failed (line %d)\n", #call, __LINE__);  \
      return 1;                                                   \
    }                                                             \
  } while (0)

int main(void) {
  gpucontext_props *p;
  gpucontext *ctx;
  CHECK(gpucontext_props_new(&p));
  CHECK(gpucontext_props_hip_dev(p, 0));
  CHECK(gpucontext_init(&ctx, "hip", p));
  GpuArray a, b, c, m, o, x, y, z;
  size_t d1[1] = {1024}, d2[2] = {64, 64}, d3[1] = {64};
  CHECK(GpuArray_zeros(&a, ctx, GA_FLOAT, 1, d1, GA_C_ORDER));
  CHECK(GpuArray_zeros(&b, ctx, GA_FLOAT, 1, d1, GA_C_ORDER));
  CHECK(GpuArray_zeros(&c, ctx, GA_FLOAT, 1, d1, GA_C_ORDER));
  CHECK(GpuArray_zeros(&m, ctx, GA_FLOAT, 2, d2, GA_C_ORDER));
  CHECK(GpuArray_zeros(&o, ctx, GA_FLOAT, 1, d3, GA_C_ORDER));
  CHECK(GpuArray_zeros(&x, ctx, GA_FLOAT, 2, d2, GA_C_ORDER));
  CHECK(GpuArray_zeros(&y, ctx, GA_FLOAT, 2, d2, GA_F_ORDER));   /* a transposed operand */
  CHECK(GpuArray_zeros(&z, ctx, GA_FLOAT, 2, d2, GA_C_ORDER));
  gpuelemwise_arg args[3] = {{"a", GA_FLOAT, GE_READ}, {"b", GA_FLOAT, GE_READ}, {"c", GA_FLOAT, GE_WRITE}};
  GpuElemwise *ge = GpuElemwise_new(ctx, "", "c = a*b + 0.5f", 3, args, 0, 0);
  if (ge == NULL) return 1;
  GpuReduction *gr;
  CHECK(GpuReduction_new(&gr, ctx, GA_REDUCE_SUM, 1, 1, GA_FLOAT, 0));
  void *flat[3] = {&a, &b, &c}, *strided[3] = {&x, &y, &z};
  int axis[1] = {1};
  const int N = 200000;
  double t;
  for (int i = 0; i < 100; i++) CHECK(GpuElemwise_call(ge, flat, 0));
  t = now_us();
  for (int i = 0; i < N; i++) GpuElemwise_call(ge, flat, 0);
  printf("GpuElemwise_call_contiguous %.4f\n", (now_us() - t) / N);
  for (int i = 0; i < 100; i++) CHECK(GpuElemwise_call(ge, strided, 0));
  t = now_us();
  for (int i = 0; i < N; i++) GpuElemwise_call(ge, strided, 0);
  printf("GpuElemwise_call_strided %.4f\n", (now_us() - t) / N);
  for (int i = 0; i < 100; i++) CHECK(GpuReduction_call(gr, &o, NULL, &m, 1, axis, 0));
  t = now_us();
  for (int i = 0; i < N; i++) GpuReduction_call(gr, &o, NULL, &m, 1, axis, 0);
  printf("GpuReduction_call %.4f\n", (now_us() - t) / N);
  /* two layouts in turn: both plans are kept */
  void *alt[3] = {&y, &x, &z};
  t = now_us();
  for (int i = 0; i < N; i++) GpuElemwise_call(ge, (i & 1) ? alt : strided, 0);
  printf("GpuElemwise_call_two_layouts_in_turn %.4f\n", (now_us() - t) / N);
  return 0;
}
