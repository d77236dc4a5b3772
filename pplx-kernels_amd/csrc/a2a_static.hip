// The library's own scratch memory for pplx_a2a_static_step, the entry point that allocates
// nothing: a fixed array in device memory that every GPU the library runs on holds from the
// moment the code object is loaded until the process ends.
//
// The array's name is a host-side stand-in, not a device address.  The address of a device's
// copy is looked up once per device with hipGetSymbolAddress, with that device current, and
// kept; host code uses only that pointer (as kernel argument), never the name.
#include <hip/hip_runtime.h>

#include <mutex>

#include "a2a_device.h"

namespace pplx_amd {
namespace {

static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_of_device[kMaxDevices] = {};

}  // namespace

// `device` must be the calling thread's current device.  Returns a hipError_t as int.
int static_scratch_address(int device, void **out) {
  *out = nullptr;
  if (device < 0 || device >= kMaxDevices) return (int)hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_of_device[device]) {
    int current = -1;
    hipError_t err = hipGetDevice(&current);
    if (err != hipSuccess) return (int)err;
    if (current != device) return (int)hipErrorInvalidDevice;
    void *ptr = nullptr;
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess) return (int)err;
    if (!ptr) return (int)hipErrorInvalidSymbol;
    g_scratch_of_device[device] = ptr;
  }
  *out = g_scratch_of_device[device];
  return (int)hipSuccess;
}

bool static_scratch_known(int device) {
  if (device < 0 || device >= kMaxDevices) return false;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  return g_scratch_of_device[device] != nullptr;
}

}  // namespace pplx_amd
