// Device scratch memory that exists without any allocation call: the partials
// of split reductions launched through GpuReduction_call_noalloc live here.
//
// The array is part of the library's code object, so every GPU the library
// runs on holds its own copy, at its own address, from the first lookup until
// the process ends.  In host code the array's name is only a handle for the
// lookup below, never a device address: kernels receive the address that
// hipGetSymbolAddress returned for the current device.
#include <hip/hip_runtime.h>

#include <mutex>

#include "private.hpp"

static __device__ __align__(256) unsigned char scratch[ga_static_scratch_bytes];

namespace {
constexpr int MAXDEV = 64;
std::mutex mu;
void *ptr_of[MAXDEV];      // address of `scratch` on device d, once looked up
int err_of[MAXDEV];        // HIP error code of a failed lookup
bool tried[MAXDEV];
}  // namespace

int ga_static_scratch_setup(int dev, void **out) {
  *out = nullptr;
  if (dev < 0 || dev >= MAXDEV) return (int)hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lk(mu);
  if (!tried[dev]) {
    // the caller has made `dev` the current device
    void *ptr = nullptr;
    hipError_t e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) {
      (void)hipGetLastError();
      ptr = nullptr;
    } else if (ptr == nullptr) {
      e = hipErrorInvalidSymbol;
    }
    tried[dev] = true;
    ptr_of[dev] = ptr;
    err_of[dev] = (int)e;
  }
  *out = ptr_of[dev];
  return err_of[dev];
}
