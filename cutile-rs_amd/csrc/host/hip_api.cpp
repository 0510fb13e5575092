// Binds the HIP runtime at first use (see hip_api.h).
#include "hip_api.h"

#include <dlfcn.h>

#include <atomic>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>

#include "common.h"

namespace cutile {
namespace {

thread_local std::string g_error;
thread_local char g_error_buf[2048];

std::mutex g_bind_mutex;
std::atomic<const HipApi*> g_api{nullptr};
HipApi g_real;
bool g_bind_failed = false;
std::string g_bind_error;

void* open_runtime(std::string* err) {
  // A runtime that is already mapped (for instance the copy PyTorch ships) wins:
  // two HIP runtimes in one process would not share streams or allocations.
  static const char* kNames[] = {"libamdhip64.so.7", "libamdhip64.so.6", "libamdhip64.so"};
  for (const char* n : kNames)
    if (void* h = dlopen(n, RTLD_NOW | RTLD_NOLOAD)) return h;
  static const char* kPaths[] = {"libamdhip64.so.7",          "libamdhip64.so.6",
                                 "libamdhip64.so",            "/opt/rocm/lib/libamdhip64.so.7",
                                 "/opt/rocm/lib/libamdhip64.so.6", "/opt/rocm/lib/libamdhip64.so"};
  for (const char* p : kPaths) {
    if (void* h = dlopen(p, RTLD_NOW | RTLD_GLOBAL)) return h;
    const char* e = dlerror();
    if (e && err->size() < 1024) {
      *err += e;
      *err += "; ";
    }
  }
  return nullptr;
}

}  // namespace

cutile_status_t fail(cutile_status_t status, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error_buf, sizeof(g_error_buf), fmt, ap);
  va_end(ap);
  g_error = g_error_buf;
  return status;
}

cutile_status_t from_hip(hipError_t err, const char* what) {
  if (err == hipSuccess) return CUTILE_SUCCESS;
  const HipApi* api = g_api.load(std::memory_order_acquire);
  const char* msg = (api && api->hipGetErrorString) ? api->hipGetErrorString(err) : "unknown";
  snprintf(g_error_buf, sizeof(g_error_buf), "DriverError(%d): %s in %s", (int)err, msg ? msg : "unknown", what);
  g_error = g_error_buf;
  return (cutile_status_t)err;
}

void clear_error() { g_error.clear(); }

const HipApi* hip() {
  const HipApi* api = g_api.load(std::memory_order_acquire);
  if (api) return api;
  std::lock_guard<std::mutex> lock(g_bind_mutex);
  api = g_api.load(std::memory_order_acquire);
  if (api) return api;
  if (g_bind_failed) {
    fail(CUTILE_ERR_LIBRARY_INIT, "%s", g_bind_error.c_str());
    return nullptr;
  }
  std::string err;
  void* h = open_runtime(&err);
  if (!h) {
    g_bind_failed = true;
    g_bind_error = "shared object init failed: cannot load libamdhip64: " + err;
    fail(CUTILE_ERR_LIBRARY_INIT, "%s", g_bind_error.c_str());
    return nullptr;
  }
#define X(name, ret, params)                                                    \
  g_real.name = reinterpret_cast<ret(*) params>(dlsym(h, #name));               \
  if (!g_real.name) {                                                           \
    g_bind_failed = true;                                                       \
    g_bind_error = "shared object init failed: libamdhip64 lacks symbol " #name; \
    fail(CUTILE_ERR_LIBRARY_INIT, "%s", g_bind_error.c_str());                  \
    return nullptr;                                                             \
  }
  CUTILE_HIP_FUNCTIONS(X)
#undef X
  g_api.store(&g_real, std::memory_order_release);
  return &g_real;
}

void install_hip_api(const HipApi* table) {
  std::lock_guard<std::mutex> lock(g_bind_mutex);
  g_bind_failed = false;
  g_api.store(table, std::memory_order_release);
}

}  // namespace cutile

extern "C" const char* cutile_last_error_message(void) { return cutile::g_error.c_str(); }

extern "C" const char* cutile_status_name(cutile_status_t s) {
  switch (s) {
    case CUTILE_SUCCESS: return "CUTILE_SUCCESS";
    case CUTILE_ERR_LIBRARY_INIT: return "CUTILE_ERR_LIBRARY_INIT";
    case CUTILE_ERR_INVALID_ARGUMENT: return "CUTILE_ERR_INVALID_ARGUMENT";
    case CUTILE_ERR_KERNEL_NOT_FOUND: return "CUTILE_ERR_KERNEL_NOT_FOUND";
    case CUTILE_ERR_KERNEL_LAUNCH: return "CUTILE_ERR_KERNEL_LAUNCH";
    case CUTILE_ERR_TENSOR: return "CUTILE_ERR_TENSOR";
    case CUTILE_ERR_STATE: return "CUTILE_ERR_STATE";
    case CUTILE_ERR_OUT_OF_SLOTS: return "CUTILE_ERR_OUT_OF_SLOTS";
    default: return s > 0 ? "DriverError" : "CUTILE_ERR_UNKNOWN";
  }
}

extern "C" const char* cutile_version(void) { return "0.1.0-gfx950"; }
