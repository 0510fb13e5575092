// Device-resident scratch memory for the entry point that allocates nothing
// (cutile_launch_fmha_decode_gqa_noalloc, include/cutile_hip.h).
//
// This is the only source of the package that hipcc compiles for host AND
// device: the array below lives in the device image of this file, and the HIP
// runtime that registers that image is the one the process already runs
// (libcutile_hip.so loads this file's library, libcutile_hip_scratch.so, with
// dlopen after it has bound the runtime, so the soname resolves to that copy).
//
// Every GPU holds its own copy of the array, at its own address, from the first
// call on that GPU until the process ends.  In host code the name `scratch` is a
// host-side handle for the runtime's symbol table, never a device address: the
// only host use of the name is the HIP_SYMBOL() lookup below, and everything
// else (kernel arguments, copies) takes the pointer that lookup returned.
#include <hip/hip_runtime.h>

#include <mutex>

#include "scratch.h"

static __device__ __align__(256) unsigned char scratch[CUTILE_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_mutex;
void* g_ptr[kMaxDevices] = {};
}  // namespace

// The device address of the calling thread's current GPU's copy of the array.
// Looked up once per device, with that device current (it is: the lookup asks the
// runtime for the current device and resolves the symbol there).  Returns the
// hipError_t of the failing runtime call, 0 on success.
extern "C" int cutile_scratch_lookup(void** device_ptr, size_t* bytes, int* device_ordinal) {
  int dev = -1;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return (int)err;
  if (dev < 0 || dev >= kMaxDevices) return (int)hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_mutex);
  if (!g_ptr[dev]) {
    void* p = nullptr;
    err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (err != hipSuccess) return (int)err;
    if (!p) return (int)hipErrorInvalidSymbol;
    size_t n = 0;
    err = hipGetSymbolSize(&n, HIP_SYMBOL(scratch));
    if (err != hipSuccess) return (int)err;
    if (n != (size_t)CUTILE_SCRATCH_BYTES) return (int)hipErrorInvalidSymbol;
    g_ptr[dev] = p;
  }
  *device_ptr = g_ptr[dev];
  *bytes = (size_t)CUTILE_SCRATCH_BYTES;
  if (device_ordinal) *device_ordinal = dev;
  return 0;
}
