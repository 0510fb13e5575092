// Part A of the C ABI: the driver layer over the HIP runtime.
//
// Mirrors the RAII layer of the reference (cuda-core/src/runtime.rs, api.rs) as
// flat calls.  Devices are process-global handles, one per ordinal
// (runtime.rs:126-139); streams are non-blocking, pooled per device and never
// destroyed (runtime.rs:249-266,504-509,613-631) because destroying a stream
// that a still-running callback references is the teardown race the reference
// avoids the same way.
#include <cstdio>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <vector>

#include "common.h"
#include "runtime_state.h"

using namespace cutile;

namespace cutile {

namespace {
std::mutex g_devices_mutex;
std::map<int, std::unique_ptr<cutile_device>> g_devices;
std::once_flag g_init_once;
cutile_status_t g_init_status = CUTILE_SUCCESS;
std::string g_init_error;
}  // namespace

cutile_status_t ensure_init() {
  CUTILE_API_OR_RETURN(api);
  // hipInit is cheap and idempotent; call it every time a fake/real table swap
  // may have happened instead of caching across tables.
  hipError_t e = api->hipInit(0);
  if (e != hipSuccess) return from_hip(e, "hipInit(0)");
  return CUTILE_SUCCESS;
}

void reset_runtime_for_testing() {
  reset_async_runtime_for_testing();
  std::lock_guard<std::mutex> lock(g_devices_mutex);
  g_devices.clear();
}

}  // namespace cutile

extern "C" {

cutile_status_t cutile_init(void) { return ensure_init(); }

cutile_status_t cutile_device_count(int32_t* count) {
  CUTILE_REQUIRE(count, CUTILE_ERR_INVALID_ARGUMENT, "count is null");
  if (cutile_status_t s = ensure_init()) return s;
  CUTILE_API_OR_RETURN(api);
  int n = 0;
  CUTILE_HIP_OR_RETURN(api, hipGetDeviceCount(&n));
  *count = n;
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_device_get(int32_t ordinal, cutile_device_t* device) {
  CUTILE_REQUIRE(device, CUTILE_ERR_INVALID_ARGUMENT, "device is null");
  int32_t n = 0;
  if (cutile_status_t s = cutile_device_count(&n)) return s;
  // An ordinal outside the device list is the driver's invalid-device error,
  // like Device::new on a bad ordinal (cuda-async/tests/error_handling.rs:174-190).
  if (ordinal < 0 || ordinal >= n) return from_hip(hipErrorInvalidDevice, "cutile_device_get");
  std::lock_guard<std::mutex> lock(g_devices_mutex);
  auto it = g_devices.find(ordinal);
  if (it == g_devices.end()) {
    auto d = std::make_unique<cutile_device>();
    d->ordinal = ordinal;
    it = g_devices.emplace(ordinal, std::move(d)).first;
  }
  *device = it->second.get();
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_device_name(cutile_device_t device, char* buf, size_t buf_len) {
  CUTILE_REQUIRE(device && buf && buf_len, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipDeviceGetName(buf, (int)buf_len, device->ordinal));
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_device_arch(cutile_device_t device, char* buf, size_t buf_len) {
  CUTILE_REQUIRE(device && buf && buf_len, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  CUTILE_API_OR_RETURN(api);
  auto props = std::make_unique<hipDeviceProp_tR0600>();
  CUTILE_HIP_OR_RETURN(api, hipGetDevicePropertiesR0600(props.get(), device->ordinal));
  snprintf(buf, buf_len, "%s", props->gcnArchName);
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_device_bind_to_thread(cutile_device_t device) {
  CUTILE_REQUIRE(device, CUTILE_ERR_INVALID_ARGUMENT, "device is null");
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipSetDevice(device->ordinal));
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_device_synchronize(cutile_device_t device) {
  if (cutile_status_t s = cutile_device_bind_to_thread(device)) return s;
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipDeviceSynchronize());
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_device_l2_cache_size(cutile_device_t device, size_t* bytes) {
  CUTILE_REQUIRE(device && bytes, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  CUTILE_API_OR_RETURN(api);
  int v = 0;
  CUTILE_HIP_OR_RETURN(api, hipDeviceGetAttribute(&v, hipDeviceAttributeL2CacheSize, device->ordinal));
  *bytes = (size_t)v;
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_device_props(cutile_device_t device, cutile_device_props_t* props) {
  CUTILE_REQUIRE(device && props, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  CUTILE_API_OR_RETURN(api);
  memset(props, 0, sizeof(*props));
  struct { hipDeviceAttribute_t attr; int32_t* dst; } q[] = {
      {hipDeviceAttributeMultiprocessorCount, &props->compute_units},
      {hipDeviceAttributeClockRate, &props->clock_khz},
      {hipDeviceAttributeMemoryClockRate, &props->memory_clock_khz},
      {hipDeviceAttributeMemoryBusWidth, &props->memory_bus_bits},
      {hipDeviceAttributeL2CacheSize, &props->l2_bytes},
      {hipDeviceAttributeMaxSharedMemoryPerBlock, &props->lds_bytes_per_block},
      {hipDeviceAttributeWarpSize, &props->wavefront_size},
  };
  for (auto& e : q) {
    int v = 0;
    CUTILE_HIP_OR_RETURN(api, hipDeviceGetAttribute(&v, e.attr, device->ordinal));
    *e.dst = v;
  }
  size_t total = 0;
  CUTILE_HIP_OR_RETURN(api, hipDeviceTotalMem(&total, device->ordinal));
  props->total_memory_bytes = total;
  return CUTILE_SUCCESS;
}

// ---- streams -------------------------------------------------------------------------------
cutile_status_t cutile_stream_create(cutile_device_t device, cutile_stream_t* stream) {
  CUTILE_REQUIRE(device && stream, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  {
    std::lock_guard<std::mutex> lock(device->mutex);
    if (!device->idle_streams.empty()) {
      *stream = device->idle_streams.back();
      device->idle_streams.pop_back();
      return CUTILE_SUCCESS;
    }
  }
  if (cutile_status_t s = cutile_device_bind_to_thread(device)) return s;
  CUTILE_API_OR_RETURN(api);
  hipStream_t st = nullptr;
  CUTILE_HIP_OR_RETURN(api, hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
  {
    std::lock_guard<std::mutex> lock(device->mutex);
    device->streams_created++;
  }
  *stream = st;
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_stream_release(cutile_device_t device, cutile_stream_t stream) {
  CUTILE_REQUIRE(device && stream, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  std::lock_guard<std::mutex> lock(device->mutex);
  device->idle_streams.push_back((hipStream_t)stream);
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_stream_synchronize(cutile_stream_t stream) {
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipStreamSynchronize((hipStream_t)stream));
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_stream_query(cutile_stream_t stream, int32_t* done) {
  CUTILE_REQUIRE(done, CUTILE_ERR_INVALID_ARGUMENT, "done is null");
  CUTILE_API_OR_RETURN(api);
  hipError_t e = api->hipStreamQuery((hipStream_t)stream);
  if (e == hipSuccess) {
    *done = 1;
    return CUTILE_SUCCESS;
  }
  if (e == hipErrorNotReady) {
    *done = 0;
    return CUTILE_SUCCESS;
  }
  return from_hip(e, "hipStreamQuery");
}

cutile_status_t cutile_stream_launch_host_func(cutile_stream_t stream, cutile_host_fn_t fn, void* user) {
  CUTILE_REQUIRE(fn, CUTILE_ERR_INVALID_ARGUMENT, "fn is null");
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipLaunchHostFunc((hipStream_t)stream, (hipHostFn_t)fn, user));
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_stream_begin_capture(cutile_stream_t stream) {
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeRelaxed));
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_stream_end_capture(cutile_stream_t stream, cutile_graph_t* graph) {
  CUTILE_REQUIRE(graph, CUTILE_ERR_INVALID_ARGUMENT, "graph is null");
  CUTILE_API_OR_RETURN(api);
  hipGraph_t g = nullptr;
  CUTILE_HIP_OR_RETURN(api, hipStreamEndCapture((hipStream_t)stream, &g));
  *graph = g;
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_stream_write_value32(cutile_stream_t stream, void* device_ptr, uint32_t value) {
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipStreamWriteValue32((hipStream_t)stream, device_ptr, value, 0));
  return CUTILE_SUCCESS;
}

// ---- events --------------------------------------------------------------------------------
cutile_status_t cutile_event_create(cutile_event_t* event) {
  CUTILE_REQUIRE(event, CUTILE_ERR_INVALID_ARGUMENT, "event is null");
  CUTILE_API_OR_RETURN(api);
  hipEvent_t e = nullptr;
  CUTILE_HIP_OR_RETURN(api, hipEventCreateWithFlags(&e, hipEventDefault));
  *event = e;
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_event_record(cutile_event_t event, cutile_stream_t stream) {
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipEventRecord((hipEvent_t)event, (hipStream_t)stream));
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_event_synchronize(cutile_event_t event) {
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipEventSynchronize((hipEvent_t)event));
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_event_elapsed_ms(cutile_event_t start, cutile_event_t end, float* ms) {
  CUTILE_REQUIRE(ms, CUTILE_ERR_INVALID_ARGUMENT, "ms is null");
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)end));
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_event_destroy(cutile_event_t event) {
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipEventDestroy((hipEvent_t)event));
  return CUTILE_SUCCESS;
}

// ---- modules -------------------------------------------------------------------------------
cutile_status_t cutile_module_load_data(cutile_device_t device, const void* image, size_t size,
                                        cutile_module_t* module) {
  CUTILE_REQUIRE(device && image && module, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  // Reject anything that is not an ELF image before the driver sees it
  // (cuda-core/src/runtime.rs:309-328 does the same for cubins).
  static const unsigned char kElf[4] = {0x7f, 'E', 'L', 'F'};
  CUTILE_REQUIRE(size >= 4 && memcmp(image, kElf, 4) == 0, CUTILE_ERR_INVALID_ARGUMENT,
                 "module image is not an ELF code object");
  if (cutile_status_t s = cutile_device_bind_to_thread(device)) return s;
  CUTILE_API_OR_RETURN(api);
  hipModule_t m = nullptr;
  CUTILE_HIP_OR_RETURN(api, hipModuleLoadData(&m, image));
  auto* out = new cutile_module();
  out->device = device;
  out->handle = m;
  count_module_load();
  *module = out;
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_module_unload(cutile_module_t module) {
  CUTILE_REQUIRE(module, CUTILE_ERR_INVALID_ARGUMENT, "module is null");
  CUTILE_API_OR_RETURN(api);
  hipError_t e = api->hipModuleUnload(module->handle);
  delete module;
  return from_hip(e, "hipModuleUnload");
}

cutile_status_t cutile_module_get_function(cutile_module_t module, const char* name,
                                           cutile_function_t* function) {
  CUTILE_REQUIRE(module && name && function, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  CUTILE_API_OR_RETURN(api);
  hipFunction_t f = nullptr;
  CUTILE_HIP_OR_RETURN(api, hipModuleGetFunction(&f, module->handle, name));
  *function = f;
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_launch_kernel(cutile_function_t function, const uint32_t grid[3],
                                     const uint32_t block[3], uint32_t shared_mem_bytes,
                                     cutile_stream_t stream, void** kernel_params) {
  CUTILE_REQUIRE(function && grid && block, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipModuleLaunchKernel((hipFunction_t)function, grid[0], grid[1], grid[2],
                                                  block[0], block[1], block[2], shared_mem_bytes,
                                                  (hipStream_t)stream, kernel_params, nullptr));
  return CUTILE_SUCCESS;
}

// ---- memory --------------------------------------------------------------------------------
cutile_status_t cutile_malloc_async(size_t bytes, cutile_stream_t stream, void** device_ptr) {
  CUTILE_REQUIRE(device_ptr, CUTILE_ERR_INVALID_ARGUMENT, "device_ptr is null");
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipMallocAsync(device_ptr, bytes, (hipStream_t)stream));
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_malloc_from_pool_async(size_t bytes, cutile_mempool_t pool, cutile_stream_t stream,
                                              void** device_ptr) {
  CUTILE_REQUIRE(device_ptr && pool, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipMallocFromPoolAsync(device_ptr, bytes, (hipMemPool_t)pool, (hipStream_t)stream));
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_free_async(void* device_ptr, cutile_stream_t stream) {
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipFreeAsync(device_ptr, (hipStream_t)stream));
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_memset_d8_async(void* device_ptr, uint8_t value, size_t bytes, cutile_stream_t stream) {
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipMemsetD8Async((hipDeviceptr_t)device_ptr, value, bytes, (hipStream_t)stream));
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_memcpy_htod_async(void* dst, const void* src, size_t bytes, cutile_stream_t stream) {
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipMemcpyHtoDAsync((hipDeviceptr_t)dst, src, bytes, (hipStream_t)stream));
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_memcpy_dtoh_async(void* dst, const void* src, size_t bytes, cutile_stream_t stream) {
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipMemcpyDtoHAsync(dst, (hipDeviceptr_t)src, bytes, (hipStream_t)stream));
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_memcpy_dtod_async(void* dst, const void* src, size_t bytes, cutile_stream_t stream) {
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipMemcpyDtoDAsync((hipDeviceptr_t)dst, (hipDeviceptr_t)src, bytes, (hipStream_t)stream));
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_host_alloc_mapped(size_t bytes, void** host_ptr, void** device_ptr) {
  CUTILE_REQUIRE(host_ptr, CUTILE_ERR_INVALID_ARGUMENT, "host_ptr is null");
  CUTILE_API_OR_RETURN(api);
  void* h = nullptr;
  CUTILE_HIP_OR_RETURN(api, hipHostMalloc(&h, bytes, hipHostMallocPortable | hipHostMallocMapped));
  if (device_ptr) {
    hipError_t e = api->hipHostGetDevicePointer(device_ptr, h, 0);
    if (e != hipSuccess) {
      api->hipHostFree(h);
      return from_hip(e, "hipHostGetDevicePointer");
    }
  }
  *host_ptr = h;
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_host_free(void* host_ptr) {
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipHostFree(host_ptr));
  return CUTILE_SUCCESS;
}

// ---- memory pools --------------------------------------------------------------------------
cutile_status_t cutile_mempool_create(cutile_device_t device, cutile_mempool_t* pool) {
  CUTILE_REQUIRE(device && pool, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  CUTILE_API_OR_RETURN(api);
  hipMemPoolProps props;
  memset(&props, 0, sizeof(props));
  props.allocType = hipMemAllocationTypePinned;
  props.handleTypes = hipMemHandleTypeNone;
  props.location.type = hipMemLocationTypeDevice;
  props.location.id = device->ordinal;
  hipMemPool_t p = nullptr;
  CUTILE_HIP_OR_RETURN(api, hipMemPoolCreate(&p, &props));
  *pool = p;
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_mempool_default(cutile_device_t device, cutile_mempool_t* pool) {
  CUTILE_REQUIRE(device && pool, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  CUTILE_API_OR_RETURN(api);
  hipMemPool_t p = nullptr;
  CUTILE_HIP_OR_RETURN(api, hipDeviceGetDefaultMemPool(&p, device->ordinal));
  *pool = p;
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_mempool_destroy(cutile_mempool_t pool) {
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipMemPoolDestroy((hipMemPool_t)pool));
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_mempool_set_release_threshold(cutile_mempool_t pool, uint64_t bytes) {
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipMemPoolSetAttribute((hipMemPool_t)pool, hipMemPoolAttrReleaseThreshold, &bytes));
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_mempool_stats(cutile_mempool_t pool, cutile_pool_mem_stats_t* stats) {
  CUTILE_REQUIRE(stats, CUTILE_ERR_INVALID_ARGUMENT, "stats is null");
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipMemPoolGetAttribute((hipMemPool_t)pool, hipMemPoolAttrReservedMemCurrent, &stats->reserved_current));
  CUTILE_HIP_OR_RETURN(api, hipMemPoolGetAttribute((hipMemPool_t)pool, hipMemPoolAttrReservedMemHigh, &stats->reserved_high));
  CUTILE_HIP_OR_RETURN(api, hipMemPoolGetAttribute((hipMemPool_t)pool, hipMemPoolAttrUsedMemCurrent, &stats->used_current));
  CUTILE_HIP_OR_RETURN(api, hipMemPoolGetAttribute((hipMemPool_t)pool, hipMemPoolAttrUsedMemHigh, &stats->used_high));
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_mempool_reset_used_high(cutile_mempool_t pool) {
  CUTILE_API_OR_RETURN(api);
  uint64_t zero = 0;
  CUTILE_HIP_OR_RETURN(api, hipMemPoolSetAttribute((hipMemPool_t)pool, hipMemPoolAttrUsedMemHigh, &zero));
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_mempool_reset_reserved_high(cutile_mempool_t pool) {
  CUTILE_API_OR_RETURN(api);
  uint64_t zero = 0;
  CUTILE_HIP_OR_RETURN(api, hipMemPoolSetAttribute((hipMemPool_t)pool, hipMemPoolAttrReservedMemHigh, &zero));
  return CUTILE_SUCCESS;
}

// ---- graphs --------------------------------------------------------------------------------
cutile_status_t cutile_graph_instantiate(cutile_graph_t graph, cutile_graph_exec_t* exec) {
  CUTILE_REQUIRE(graph && exec, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  CUTILE_API_OR_RETURN(api);
  hipGraphExec_t e = nullptr;
  CUTILE_HIP_OR_RETURN(api, hipGraphInstantiateWithFlags(&e, (hipGraph_t)graph, 0));
  *exec = e;
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_graph_upload(cutile_graph_exec_t exec, cutile_stream_t stream) {
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipGraphUpload((hipGraphExec_t)exec, (hipStream_t)stream));
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_graph_launch(cutile_graph_exec_t exec, cutile_stream_t stream) {
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipGraphLaunch((hipGraphExec_t)exec, (hipStream_t)stream));
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_graph_exec_destroy(cutile_graph_exec_t exec) {
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipGraphExecDestroy((hipGraphExec_t)exec));
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_graph_destroy(cutile_graph_t graph) {
  CUTILE_API_OR_RETURN(api);
  CUTILE_HIP_OR_RETURN(api, hipGraphDestroy((hipGraph_t)graph));
  return CUTILE_SUCCESS;
}

}  // extern "C"
