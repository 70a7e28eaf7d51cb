/* A C program written against the reference's headers alone, the way its own
 * C tests are (tests/device.c:58-70, tests/check_elemwise.c:39-93,
 * tests/check_reduction.c:85-160, tests/check_array.c:252-279): it only
 * includes <gpuarray/...> and links libgpuarray.  The one change from the
 * reference's set-up is the backend name ("hip") and its device setter.
 * Exit status 0 means every check passed; each failure prints its line. */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <gpuarray/array.h>
#include <gpuarray/buffer.h>
#include <gpuarray/elemwise.h>
#include <gpuarray/error.h>
#include <gpuarray/kernel.h>
#include <gpuarray/reduction.h>
#include <gpuarray/types.h>
#include <gpuarray/util.h>

static int failures = 0;
#define CHECK(cond) do { if (!(cond)) { printf("FAILED line %d: %s\n", __LINE__, #cond); failures++; } } while (0)
#define OK(call) do { int e_ = (call); if (e_ != GA_NO_ERROR) { printf("FAILED line %d: %s -> %d (%s)\n", __LINE__, #call, e_, gpucontext_error(ctx, e_)); failures++; } } while (0)

static gpucontext *ctx;

static void contig_simple(void) {                      /* check_elemwise.c:39-93 */
  GpuArray a, b, c;
  GpuElemwise *ge;
  static const uint32_t data1[3] = {1, 2, 3};
  static const uint32_t data2[3] = {4, 5, 6};
  uint32_t data3[3] = {0};
  size_t dims[1];
  gpuelemwise_arg args[3];
  void *rargs[3];

  memset(args, 0, sizeof(args));
  dims[0] = 3;
  OK(GpuArray_empty(&a, ctx, GA_UINT, 1, dims, GA_C_ORDER));
  OK(GpuArray_write(&a, data1, sizeof(data1)));
  OK(GpuArray_empty(&b, ctx, GA_UINT, 1, dims, GA_C_ORDER));
  OK(GpuArray_write(&b, data2, sizeof(data2)));
  OK(GpuArray_empty(&c, ctx, GA_UINT, 1, dims, GA_C_ORDER));
  args[0].name = "a"; args[0].typecode = GA_UINT; args[0].flags = GE_READ;
  args[1].name = "b"; args[1].typecode = GA_UINT; args[1].flags = GE_READ;
  args[2].name = "c"; args[2].typecode = GA_UINT; args[2].flags = GE_WRITE;
  ge = GpuElemwise_new(ctx, "", "c = a + b", 3, args, 1, 0);
  CHECK(ge != NULL);
  if (ge == NULL) return;
  rargs[0] = &a; rargs[1] = &b; rargs[2] = &c;
  OK(GpuElemwise_call(ge, rargs, GE_NOCOLLAPSE));
  OK(GpuArray_read(data3, sizeof(data3), &c));
  CHECK(data3[0] == 5 && data3[1] == 7 && data3[2] == 9);
  GpuElemwise_free(ge);
  GpuArray_clear(&a); GpuArray_clear(&b); GpuArray_clear(&c);
}

static void reduction(void) {                          /* check_reduction.c:85-160 */
  enum { D0 = 32, D1 = 50, D2 = 79 };
  static float src[D0 * D1 * D2];
  static float got_max[D1];
  static uint64_t got_arg[D1];
  GpuArray gs, gmax, garg, gsum;
  GpuReduction *gr = NULL;
  size_t dims[3], odims[1];
  const unsigned redux[2] = {0, 2};
  const int iredux[2] = {0, 2};
  size_t i, j, k;
  uint32_t state = 12345u;
  static float got_sum[D1];

  for (i = 0; i < D0 * D1 * D2; i++) {
    state = state * 1664525u + 1013904223u;
    src[i] = (float)(state >> 8) / 16777216.0f;
  }
  dims[0] = D0; dims[1] = D1; dims[2] = D2;
  odims[0] = D1;
  OK(GpuArray_empty(&gs, ctx, GA_FLOAT, 3, dims, GA_C_ORDER));
  OK(GpuArray_empty(&gmax, ctx, GA_FLOAT, 1, odims, GA_C_ORDER));
  OK(GpuArray_empty(&garg, ctx, GA_ULONG, 1, odims, GA_C_ORDER));
  OK(GpuArray_empty(&gsum, ctx, GA_FLOAT, 1, odims, GA_C_ORDER));
  OK(GpuArray_write(&gs, src, sizeof(src)));
  OK(GpuArray_maxandargmax(&gmax, &garg, &gs, 2, redux));
  OK(GpuArray_read(got_max, sizeof(got_max), &gmax));
  OK(GpuArray_read(got_arg, sizeof(got_arg), &garg));
  OK(GpuReduction_new(&gr, ctx, GA_REDUCE_SUM, 1, 2, GA_FLOAT, 0));
  OK(GpuReduction_call(gr, &gsum, NULL, &gs, 2, iredux, 0));
  OK(GpuArray_read(got_sum, sizeof(got_sum), &gsum));
  for (j = 0; j < D1; j++) {
    uint64_t arg = 0;
    float max = src[j * D2];
    double sum = 0.0;
    for (i = 0; i < D0; i++)
      for (k = 0; k < D2; k++) {
        float v = src[(i * D1 + j) * D2 + k];
        if (v > max) { max = v; arg = i * D2 + k; }
        sum += v;
      }
    CHECK(got_max[j] == max);
    CHECK(got_arg[j] == arg);
    CHECK(got_sum[j] > sum * (1 - 1e-5) && got_sum[j] < sum * (1 + 1e-5));
  }
  GpuReduction_free(gr);
  GpuArray_clear(&gs); GpuArray_clear(&gmax); GpuArray_clear(&garg); GpuArray_clear(&gsum);
}

static void take1_offset(void) {                       /* check_array.c:252-279 */
  const uint32_t data[4] = {0, 1, 2, 3};
  const size_t data_dims[1] = {4};
  const size_t out_dims[1] = {2};
  const uint32_t idx[4] = {20, 3, 3, 2};
  uint32_t out[2] = {0, 0};
  GpuArray v, i, r;
  OK(GpuArray_empty(&v, ctx, GA_UINT, 1, data_dims, GA_C_ORDER));
  OK(GpuArray_write(&v, data, sizeof(data)));
  OK(GpuArray_empty(&i, ctx, GA_UINT, 1, data_dims, GA_C_ORDER));
  OK(GpuArray_write(&i, idx, sizeof(idx)));
  OK(GpuArray_empty(&r, ctx, GA_UINT, 1, out_dims, GA_C_ORDER));
  i.offset += 8;
  i.dimensions[0] = 2;
  GpuArray_fix_flags(&i);
  OK(GpuArray_take1(&r, &v, &i, 1));
  OK(GpuArray_read(out, sizeof(out), &r));
  CHECK(out[0] == 3 && out[1] == 2);
  GpuArray_clear(&v); GpuArray_clear(&i); GpuArray_clear(&r);
}

static void raw_kernel(void) {
  static const char *src =
      "#include \"cluda.h\"\n"
      "KERNEL void twice(GLOBAL_MEM ga_float *x, ga_size n) {\n"
      "  ga_size i = (ga_size)GID_0 * LDIM_0 + LID_0;\n"
      "  if (i < n) x[i] = 2.0f * x[i];\n"
      "}\n";
  GpuKernel k;
  GpuArray x;
  float host[1000];
  size_t dims[1] = {1000}, n = 1000, gs = 0, ls = 0, len;
  int types[2] = {GA_BUFFER, GA_SIZE};
  char *err_str = NULL;
  size_t i;
  for (i = 0; i < 1000; i++) host[i] = (float)i;
  len = strlen(src);
  OK(GpuArray_empty(&x, ctx, GA_FLOAT, 1, dims, GA_C_ORDER));
  OK(GpuArray_write(&x, host, sizeof(host)));
  OK(GpuKernel_init(&k, ctx, 1, &src, &len, "twice", 2, types, 0, &err_str));
  free(err_str);
  OK(GpuKernel_sched(&k, n, &gs, &ls));
  CHECK(gs * ls >= n);
  OK(GpuKernel_setarg(&k, 0, x.data));
  OK(GpuKernel_setarg(&k, 1, &n));
  OK(GpuKernel_call(&k, 1, &gs, &ls, 0, NULL));
  OK(GpuArray_read(host, sizeof(host), &x));
  for (i = 0; i < 1000; i++) CHECK(host[i] == 2.0f * (float)i);
  GpuKernel_clear(&k);
  GpuArray_clear(&x);
}

int main(void) {
  gpucontext_props *p = NULL;
  if (gpucontext_props_new(&p) != GA_NO_ERROR) return 2;
  if (gpucontext_props_hip_dev(p, 0) != GA_NO_ERROR) return 2;
  if (gpucontext_init(&ctx, "hip", p) != GA_NO_ERROR) {
    printf("no context: %s\n", gpucontext_error(NULL, 0));
    return 2;
  }
  setvbuf(stdout, NULL, _IONBF, 0);
  contig_simple();
  reduction();
  take1_offset();
  raw_kernel();
  gpucontext_deref(ctx);
  printf(failures ? "%d checks failed\n" : "all checks passed\n", failures);
  return failures ? 1 : 0;
}
