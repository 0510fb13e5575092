// Lazily bound HIP runtime entry points.
//
// The library never links libamdhip64: it binds the few dozen runtime calls it
// needs with dlopen/dlsym on first use, the way the reference binds libcuda
// (cuda-bindings/src/dyn_load.rs:63-78,121-143).  Two reasons: the library then
// loads (and its host-side logic is testable) on machines without a GPU stack,
// and inside a process that already mapped a HIP runtime (PyTorch ships its own
// copy) it binds to THAT copy instead of starting a second runtime.
#pragma once
#include <hip/hip_runtime_api.h>

namespace cutile {

// name, return type, parameter list
#define CUTILE_HIP_FUNCTIONS(X)                                                                        \
  X(hipInit, hipError_t, (unsigned int))                                                               \
  X(hipGetDeviceCount, hipError_t, (int*))                                                             \
  X(hipSetDevice, hipError_t, (int))                                                                   \
  X(hipGetDevice, hipError_t, (int*))                                                                  \
  X(hipDeviceSynchronize, hipError_t, (void))                                                          \
  X(hipDeviceGetAttribute, hipError_t, (int*, hipDeviceAttribute_t, int))                              \
  X(hipDeviceGetName, hipError_t, (char*, int, hipDevice_t))                                           \
  X(hipDeviceTotalMem, hipError_t, (size_t*, hipDevice_t))                                             \
  X(hipGetDevicePropertiesR0600, hipError_t, (hipDeviceProp_tR0600*, int))                             \
  X(hipGetErrorString, const char*, (hipError_t))                                                      \
  X(hipStreamCreateWithFlags, hipError_t, (hipStream_t*, unsigned int))                                \
  X(hipStreamSynchronize, hipError_t, (hipStream_t))                                                   \
  X(hipStreamQuery, hipError_t, (hipStream_t))                                                         \
  X(hipLaunchHostFunc, hipError_t, (hipStream_t, hipHostFn_t, void*))                                  \
  X(hipStreamBeginCapture, hipError_t, (hipStream_t, hipStreamCaptureMode))                            \
  X(hipStreamEndCapture, hipError_t, (hipStream_t, hipGraph_t*))                                       \
  X(hipStreamWriteValue32, hipError_t, (hipStream_t, void*, uint32_t, unsigned int))                   \
  X(hipEventCreateWithFlags, hipError_t, (hipEvent_t*, unsigned int))                                  \
  X(hipEventRecord, hipError_t, (hipEvent_t, hipStream_t))                                             \
  X(hipEventSynchronize, hipError_t, (hipEvent_t))                                                     \
  X(hipEventElapsedTime, hipError_t, (float*, hipEvent_t, hipEvent_t))                                 \
  X(hipEventDestroy, hipError_t, (hipEvent_t))                                                         \
  X(hipModuleLoadData, hipError_t, (hipModule_t*, const void*))                                        \
  X(hipModuleUnload, hipError_t, (hipModule_t))                                                        \
  X(hipModuleGetFunction, hipError_t, (hipFunction_t*, hipModule_t, const char*))                      \
  X(hipModuleLaunchKernel, hipError_t,                                                                 \
    (hipFunction_t, unsigned int, unsigned int, unsigned int, unsigned int, unsigned int,              \
     unsigned int, unsigned int, hipStream_t, void**, void**))                                         \
  X(hipMallocAsync, hipError_t, (void**, size_t, hipStream_t))                                         \
  X(hipMallocFromPoolAsync, hipError_t, (void**, size_t, hipMemPool_t, hipStream_t))                   \
  X(hipFreeAsync, hipError_t, (void*, hipStream_t))                                                    \
  X(hipMemsetD8Async, hipError_t, (hipDeviceptr_t, unsigned char, size_t, hipStream_t))                \
  X(hipMemcpyHtoDAsync, hipError_t, (hipDeviceptr_t, const void*, size_t, hipStream_t))                      \
  X(hipMemcpyDtoHAsync, hipError_t, (void*, hipDeviceptr_t, size_t, hipStream_t))                      \
  X(hipMemcpyDtoDAsync, hipError_t, (hipDeviceptr_t, hipDeviceptr_t, size_t, hipStream_t))             \
  X(hipHostMalloc, hipError_t, (void**, size_t, unsigned int))                                         \
  X(hipHostGetDevicePointer, hipError_t, (void**, void*, unsigned int))                                \
  X(hipHostFree, hipError_t, (void*))                                                                  \
  X(hipMemPoolCreate, hipError_t, (hipMemPool_t*, const hipMemPoolProps*))                             \
  X(hipDeviceGetDefaultMemPool, hipError_t, (hipMemPool_t*, int))                                      \
  X(hipMemPoolDestroy, hipError_t, (hipMemPool_t))                                                     \
  X(hipMemPoolSetAttribute, hipError_t, (hipMemPool_t, hipMemPoolAttr, void*))                         \
  X(hipMemPoolGetAttribute, hipError_t, (hipMemPool_t, hipMemPoolAttr, void*))                         \
  X(hipGraphInstantiateWithFlags, hipError_t, (hipGraphExec_t*, hipGraph_t, unsigned long long))       \
  X(hipGraphUpload, hipError_t, (hipGraphExec_t, hipStream_t))                                         \
  X(hipGraphLaunch, hipError_t, (hipGraphExec_t, hipStream_t))                                         \
  X(hipGraphExecDestroy, hipError_t, (hipGraphExec_t))                                                 \
  X(hipGraphDestroy, hipError_t, (hipGraph_t))

struct HipApi {
#define X(name, ret, params) ret(*name) params = nullptr;
  CUTILE_HIP_FUNCTIONS(X)
#undef X
};

// Returns the bound table, or nullptr (with the thread's error message set) when
// no HIP runtime can be loaded.  Thread-safe, binds once.
const HipApi* hip();

// Test hook: installs a replacement table (a recording fake) before first use,
// or swaps it later.  nullptr restores the real runtime on next use.
void install_hip_api(const HipApi* table);

}  // namespace cutile
