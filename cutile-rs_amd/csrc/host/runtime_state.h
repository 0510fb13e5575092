// Process-global runtime objects behind the opaque C handles.
#pragma once
#include <cstdint>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "common.h"

struct cutile_module {
  struct cutile_device* device = nullptr;
  hipModule_t handle = nullptr;
};

// One per device ordinal, created on first use and kept for the life of the
// process (cuda-core/src/runtime.rs:126-139 keeps one Device per ordinal).
struct cutile_device {
  int ordinal = 0;
  std::mutex mutex;
  std::vector<hipStream_t> idle_streams;  // released streams, reused before creating new ones
  uint64_t streams_created = 0;
  int compute_units = 0;  // filled on first use by compute_units()
  // Code objects of the kernel table loaded on this device: image id -> module.
  std::map<int, cutile_module*> table_modules;
  // Resolved functions: symbol -> hipFunction_t.
  std::map<std::string, hipFunction_t> functions;
};

namespace cutile {

cutile_status_t ensure_init();
void count_module_load();
void reset_runtime_for_testing();
void reset_async_runtime_for_testing();
// Device the calling thread is bound to (hipGetDevice), as a handle.
cutile_status_t current_device(cutile_device_t* device);
// Compute units of the device (cached).
cutile_status_t compute_units(cutile_device_t device, int* count);

}  // namespace cutile
