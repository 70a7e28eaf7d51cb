// TEST INFRASTRUCTURE ONLY: host-memory stand-ins for the HIP runtime calls the
// backend makes, preloaded by tests that exercise the library's HOST logic where
// there is no device (argument checks, buffer bookkeeping, the memory cache,
// compile errors, context teardown).  Buffers are host allocations,
// copies are memcpy, a kernel launch does nothing: no result of a kernel means
// anything here, and nothing the library ships may link or load this file.
#include <hip/hip_runtime_api.h>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <cstdio>
extern "C" {
// calls that allocate or free memory on the device or pinned host side, or load code onto the device
unsigned long mock_allocating_calls = 0;
// kernel launches so far (a planner's choice between one launch and two shows here)
unsigned long mock_kernel_launches = 0;
hipError_t hipGetDeviceCount(int *n) { *n = 1; return hipSuccess; }
hipError_t hipSetDevice(int) { return hipSuccess; }
hipError_t hipGetDevice(int *d) { *d = 0; return hipSuccess; }
hipError_t hipGetDevicePropertiesR0600(hipDeviceProp_t *p, int) {
  memset(p, 0, sizeof(*p));
  strcpy(p->name, "mock"); strcpy(p->gcnArchName, "gfx950:sramecc+:xnack-");
  p->multiProcessorCount = 256; p->sharedMemPerBlock = 65536; p->maxThreadsPerBlock = 1024;
  p->maxThreadsDim[0] = 1024; p->maxThreadsDim[1] = 1024; p->maxThreadsDim[2] = 1024;
  p->maxGridSize[0] = 2147483647; p->maxGridSize[1] = 65535; p->maxGridSize[2] = 65535;
  p->totalGlobalMem = 1ull << 34; p->warpSize = 64;
  return hipSuccess;
}
hipError_t hipGetLastError() { return hipSuccess; }
const char *hipGetErrorString(hipError_t) { return "mock"; }
hipError_t hipMalloc(void **p, size_t n) { mock_allocating_calls++; *p = malloc(n ? n : 1); return *p ? hipSuccess : hipErrorOutOfMemory; }
hipError_t hipFree(void *p) { mock_allocating_calls++; free(p); return hipSuccess; }
hipError_t hipHostMalloc(void **p, size_t n, unsigned) { mock_allocating_calls++; *p = malloc(n ? n : 1); return *p ? hipSuccess : hipErrorOutOfMemory; }
hipError_t hipHostFree(void *p) { mock_allocating_calls++; free(p); return hipSuccess; }
hipError_t hipMemGetInfo(size_t *f, size_t *t) { *f = 1ull << 33; *t = 1ull << 34; return hipSuccess; }
hipError_t hipStreamCreateWithFlags(hipStream_t *s, unsigned) { *s = (hipStream_t)0x10; return hipSuccess; }
hipError_t hipStreamDestroy(hipStream_t) { return hipSuccess; }
hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
hipError_t hipEventCreate(hipEvent_t *e) { mock_allocating_calls++; *e = (hipEvent_t)0x20; return hipSuccess; }
hipError_t hipEventCreateWithFlags(hipEvent_t *e, unsigned) { mock_allocating_calls++; *e = (hipEvent_t)0x20; return hipSuccess; }
hipError_t hipEventDestroy(hipEvent_t) { return hipSuccess; }
hipError_t hipEventRecord(hipEvent_t, hipStream_t) { return hipSuccess; }
hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
hipError_t hipEventElapsedTime(float *ms, hipEvent_t, hipEvent_t) { *ms = 1; return hipSuccess; }
hipError_t hipMemcpyHtoDAsync(hipDeviceptr_t d, const void *s, size_t n, hipStream_t) { memcpy(d, s, n); return hipSuccess; }
hipError_t hipMemcpyDtoHAsync(void *d, hipDeviceptr_t s, size_t n, hipStream_t) { memcpy(d, s, n); return hipSuccess; }
hipError_t hipMemcpyDtoDAsync(hipDeviceptr_t d, hipDeviceptr_t s, size_t n, hipStream_t) { memmove(d, s, n); return hipSuccess; }
hipError_t hipMemcpyPeerAsync(void *d, int, const void *s, int, size_t n, hipStream_t) { memmove(d, s, n); return hipSuccess; }
hipError_t hipMemsetD8Async(hipDeviceptr_t d, unsigned char v, size_t n, hipStream_t) { memset(d, v, n); return hipSuccess; }
hipError_t hipStreamIsCapturing(hipStream_t, hipStreamCaptureStatus *s) { *s = hipStreamCaptureStatusNone; return hipSuccess; }
hipError_t hipGetSymbolAddress(void **p, const void *) { static char buf[4 << 20]; *p = buf; return hipSuccess; }
hipError_t hipModuleLoadData(hipModule_t *m, const void *) { mock_allocating_calls++; *m = (hipModule_t)malloc(8); return hipSuccess; }
hipError_t hipModuleUnload(hipModule_t m) { free(m); return hipSuccess; }
hipError_t hipModuleGetFunction(hipFunction_t *f, hipModule_t, const char *) { *f = (hipFunction_t)0x30; return hipSuccess; }
hipError_t hipFuncGetAttribute(int *v, hipFunction_attribute, hipFunction_t) { *v = 1024; return hipSuccess; }
hipError_t hipExtModuleLaunchKernel(hipFunction_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, size_t, hipStream_t, void **, void **, hipEvent_t, hipEvent_t, uint32_t) { mock_kernel_launches++; return hipSuccess; }
hipError_t hipModuleLaunchKernel(hipFunction_t, unsigned gx, unsigned, unsigned, unsigned bx, unsigned, unsigned, unsigned, hipStream_t, void **params, void **) {
  (void)gx; (void)bx; (void)params; mock_kernel_launches++; return hipSuccess; }
}
