// A recording stand-in for the HIP runtime (declared in cutile_hip_testing.h).
// It runs no kernels; see that header for what it is for.
#include <atomic>
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "../../../include/cutile_hip_testing.h"
#include "common.h"
#include "runtime_state.h"

namespace cutile {
namespace {

struct FakeFunction {
  std::string symbol;
};
struct FakeModule {
  std::map<std::string, FakeFunction*> functions;
};
struct LaunchRecord {
  std::string symbol;
  uint32_t grid[3], block[3], smem;
  void* stream;
  std::vector<unsigned char> args;
  bool in_capture, from_replay;
};
struct HostFuncRecord {
  hipHostFn_t fn;
  void* user;
};
struct GraphNodeRec {
  int kind;  // 0 launch, 1 host func, 2 memcpy, 3 write32
  LaunchRecord launch;
  HostFuncRecord host;
  void* dst = nullptr;
  std::vector<unsigned char> payload;  // memcpy source snapshot is NOT taken: pointer semantics
  const void* src = nullptr;
  size_t bytes = 0;
  uint32_t value = 0;
};
struct FakeGraph {
  std::vector<GraphNodeRec> nodes;
};
struct FakeStream {
  bool capturing = false;
  FakeGraph* graph = nullptr;
};
struct FakeEvent {
  double t_ms = 0.0;
};

std::mutex g_mu;
int g_n_devices = 1;
thread_local int t_device = 0;
std::deque<LaunchRecord> g_log;
std::map<std::string, std::pair<int, int>> g_failures;  // name -> (error, remaining)
std::atomic<uint64_t> g_streams_created{0};
std::atomic<uint64_t> g_bytes{0};
std::map<void*, size_t> g_allocs;

hipError_t injected(const char* name) {
  std::lock_guard<std::mutex> lock(g_mu);
  auto it = g_failures.find(name);
  if (it == g_failures.end() || it->second.second <= 0) return hipSuccess;
  it->second.second--;
  return (hipError_t)it->second.first;
}
#define FAKE_FAIL(name)                 \
  do {                                  \
    hipError_t _e = injected(name);     \
    if (_e != hipSuccess) return _e;    \
  } while (0)

double now_ms() {
  using namespace std::chrono;
  return duration<double, std::milli>(steady_clock::now().time_since_epoch()).count();
}

hipError_t f_hipInit(unsigned int) { FAKE_FAIL("hipInit"); return hipSuccess; }
hipError_t f_hipGetDeviceCount(int* n) { FAKE_FAIL("hipGetDeviceCount"); *n = g_n_devices; return hipSuccess; }
hipError_t f_hipSetDevice(int d) {
  FAKE_FAIL("hipSetDevice");
  if (d < 0 || d >= g_n_devices) return hipErrorInvalidDevice;
  t_device = d;
  return hipSuccess;
}
hipError_t f_hipGetDevice(int* d) { *d = t_device; return hipSuccess; }
hipError_t f_hipDeviceSynchronize(void) { FAKE_FAIL("hipDeviceSynchronize"); return hipSuccess; }
hipError_t f_hipDeviceGetAttribute(int* v, hipDeviceAttribute_t attr, int) {
  switch (attr) {
    case hipDeviceAttributeMultiprocessorCount: *v = 256; break;
    case hipDeviceAttributeClockRate: *v = 2400000; break;
    case hipDeviceAttributeMemoryClockRate: *v = 2000000; break;
    case hipDeviceAttributeMemoryBusWidth: *v = 8192; break;
    case hipDeviceAttributeL2CacheSize: *v = 4 << 20; break;
    case hipDeviceAttributeMaxSharedMemoryPerBlock: *v = 160 << 10; break;
    case hipDeviceAttributeWarpSize: *v = 64; break;
    default: *v = 0;
  }
  return hipSuccess;
}
hipError_t f_hipDeviceGetName(char* buf, int len, hipDevice_t) { snprintf(buf, len, "Fake gfx950 device"); return hipSuccess; }
hipError_t f_hipDeviceTotalMem(size_t* b, hipDevice_t) { *b = 288ull << 30; return hipSuccess; }
hipError_t f_hipGetDeviceProperties(hipDeviceProp_tR0600* p, int) {
  memset(p, 0, sizeof(*p));
  snprintf(p->name, sizeof(p->name), "Fake gfx950 device");
  snprintf(p->gcnArchName, sizeof(p->gcnArchName), "gfx950:sramecc+:xnack-");
  p->multiProcessorCount = 256;
  p->warpSize = 64;
  return hipSuccess;
}
const char* f_hipGetErrorString(hipError_t e) {
  switch (e) {
    case hipSuccess: return "no error";
    case hipErrorInvalidValue: return "invalid argument";
    case hipErrorOutOfMemory: return "out of memory";
    case hipErrorInvalidDevice: return "invalid device ordinal";
    case hipErrorNotReady: return "device not ready";
    case hipErrorStreamCaptureUnsupported: return "operation not permitted when stream is capturing";
    default: return "fake runtime error";
  }
}
hipError_t f_hipStreamCreateWithFlags(hipStream_t* s, unsigned int) {
  FAKE_FAIL("hipStreamCreateWithFlags");
  *s = reinterpret_cast<hipStream_t>(new FakeStream());
  g_streams_created++;
  return hipSuccess;
}
FakeStream* fs(hipStream_t s) { return reinterpret_cast<FakeStream*>(s); }
hipError_t f_hipStreamSynchronize(hipStream_t s) {
  FAKE_FAIL("hipStreamSynchronize");
  if (s && fs(s)->capturing) return hipErrorStreamCaptureUnsupported;
  return hipSuccess;
}
hipError_t f_hipStreamQuery(hipStream_t s) {
  FAKE_FAIL("hipStreamQuery");
  if (s && fs(s)->capturing) return hipErrorStreamCaptureUnsupported;
  return hipSuccess;
}
hipError_t f_hipLaunchHostFunc(hipStream_t s, hipHostFn_t fn, void* user) {
  FAKE_FAIL("hipLaunchHostFunc");
  if (s && fs(s)->capturing) {
    GraphNodeRec n;
    n.kind = 1;
    n.host = {fn, user};
    fs(s)->graph->nodes.push_back(std::move(n));
    return hipSuccess;
  }
  fn(user);
  return hipSuccess;
}
hipError_t f_hipStreamBeginCapture(hipStream_t s, hipStreamCaptureMode) {
  FAKE_FAIL("hipStreamBeginCapture");
  if (!s || fs(s)->capturing) return hipErrorInvalidValue;
  fs(s)->capturing = true;
  fs(s)->graph = new FakeGraph();
  return hipSuccess;
}
hipError_t f_hipStreamEndCapture(hipStream_t s, hipGraph_t* g) {
  if (!s || !fs(s)->capturing) return hipErrorInvalidValue;
  fs(s)->capturing = false;
  FakeGraph* graph = fs(s)->graph;
  fs(s)->graph = nullptr;
  hipError_t e = injected("hipStreamEndCapture");
  if (e != hipSuccess) {
    delete graph;
    *g = nullptr;
    return e;
  }
  *g = reinterpret_cast<hipGraph_t>(graph);
  return hipSuccess;
}
hipError_t f_hipStreamWriteValue32(hipStream_t s, void* p, uint32_t v, unsigned int) {
  FAKE_FAIL("hipStreamWriteValue32");
  if (s && fs(s)->capturing) {
    GraphNodeRec n;
    n.kind = 3;
    n.dst = p;
    n.value = v;
    fs(s)->graph->nodes.push_back(std::move(n));
    return hipSuccess;
  }
  __atomic_store_n(reinterpret_cast<uint32_t*>(p), v, __ATOMIC_RELEASE);
  return hipSuccess;
}
hipError_t f_hipEventCreateWithFlags(hipEvent_t* e, unsigned int) {
  FAKE_FAIL("hipEventCreateWithFlags");
  *e = reinterpret_cast<hipEvent_t>(new FakeEvent());
  return hipSuccess;
}
hipError_t f_hipEventRecord(hipEvent_t e, hipStream_t) {
  FAKE_FAIL("hipEventRecord");
  reinterpret_cast<FakeEvent*>(e)->t_ms = now_ms();
  return hipSuccess;
}
hipError_t f_hipEventSynchronize(hipEvent_t) { FAKE_FAIL("hipEventSynchronize"); return hipSuccess; }
hipError_t f_hipEventElapsedTime(float* ms, hipEvent_t a, hipEvent_t b) {
  *ms = (float)(reinterpret_cast<FakeEvent*>(b)->t_ms - reinterpret_cast<FakeEvent*>(a)->t_ms);
  return hipSuccess;
}
hipError_t f_hipEventDestroy(hipEvent_t e) { delete reinterpret_cast<FakeEvent*>(e); return hipSuccess; }
hipError_t f_hipModuleLoadData(hipModule_t* m, const void*) {
  FAKE_FAIL("hipModuleLoadData");
  *m = reinterpret_cast<hipModule_t>(new FakeModule());
  return hipSuccess;
}
hipError_t f_hipModuleUnload(hipModule_t m) {
  auto* mod = reinterpret_cast<FakeModule*>(m);
  for (auto& kv : mod->functions) delete kv.second;
  delete mod;
  return hipSuccess;
}
hipError_t f_hipModuleGetFunction(hipFunction_t* f, hipModule_t m, const char* name) {
  FAKE_FAIL("hipModuleGetFunction");
  auto* mod = reinterpret_cast<FakeModule*>(m);
  std::lock_guard<std::mutex> lock(g_mu);
  auto& slot = mod->functions[name];
  if (!slot) slot = new FakeFunction{name};
  *f = reinterpret_cast<hipFunction_t>(slot);
  return hipSuccess;
}
hipError_t f_hipModuleLaunchKernel(hipFunction_t f, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned by,
                                   unsigned bz, unsigned smem, hipStream_t s, void** params, void** extra) {
  FAKE_FAIL("hipModuleLaunchKernel");
  LaunchRecord r;
  r.symbol = reinterpret_cast<FakeFunction*>(f)->symbol;
  r.grid[0] = gx; r.grid[1] = gy; r.grid[2] = gz;
  r.block[0] = bx; r.block[1] = by; r.block[2] = bz;
  r.smem = smem;
  r.stream = s;
  r.in_capture = s && fs(s)->capturing;
  r.from_replay = false;
  if (extra) {
    const void* buf = nullptr;
    size_t size = 0;
    for (int i = 0; extra[i] != HIP_LAUNCH_PARAM_END; i += 2) {
      if (extra[i] == HIP_LAUNCH_PARAM_BUFFER_POINTER) buf = extra[i + 1];
      if (extra[i] == HIP_LAUNCH_PARAM_BUFFER_SIZE) size = *reinterpret_cast<size_t*>(extra[i + 1]);
    }
    if (buf && size) r.args.assign((const unsigned char*)buf, (const unsigned char*)buf + size);
  }
  (void)params;
  if (r.in_capture) {
    GraphNodeRec n;
    n.kind = 0;
    n.launch = r;
    fs(s)->graph->nodes.push_back(std::move(n));
  }
  std::lock_guard<std::mutex> lock(g_mu);
  g_log.push_back(std::move(r));
  return hipSuccess;
}
hipError_t fake_alloc(void** p, size_t bytes) {
  void* q = nullptr;
  if (posix_memalign(&q, 256, bytes ? bytes : 1) != 0) return hipErrorOutOfMemory;
  std::lock_guard<std::mutex> lock(g_mu);
  g_allocs[q] = bytes;
  g_bytes += bytes;
  *p = q;
  return hipSuccess;
}
hipError_t fake_free(void* p) {
  if (!p) return hipSuccess;
  std::lock_guard<std::mutex> lock(g_mu);
  auto it = g_allocs.find(p);
  if (it == g_allocs.end()) return hipErrorInvalidValue;
  g_bytes -= it->second;
  g_allocs.erase(it);
  free(p);
  return hipSuccess;
}
hipError_t f_hipMallocAsync(void** p, size_t bytes, hipStream_t s) {
  FAKE_FAIL("hipMallocAsync");
  if (s && fs(s)->capturing) return hipErrorStreamCaptureUnsupported;
  return fake_alloc(p, bytes);
}
hipError_t f_hipMallocFromPoolAsync(void** p, size_t bytes, hipMemPool_t, hipStream_t s) {
  FAKE_FAIL("hipMallocFromPoolAsync");
  if (s && fs(s)->capturing) return hipErrorStreamCaptureUnsupported;
  return fake_alloc(p, bytes);
}
hipError_t f_hipFreeAsync(void* p, hipStream_t) { FAKE_FAIL("hipFreeAsync"); return fake_free(p); }
hipError_t f_hipMemsetD8Async(hipDeviceptr_t p, unsigned char v, size_t n, hipStream_t) {
  FAKE_FAIL("hipMemsetD8Async");
  memset(p, v, n);
  return hipSuccess;
}
hipError_t copy_or_record(void* dst, const void* src, size_t n, hipStream_t s) {
  if (s && fs(s)->capturing) {
    GraphNodeRec node;
    node.kind = 2;
    node.dst = dst;
    node.src = src;
    node.bytes = n;
    fs(s)->graph->nodes.push_back(std::move(node));
    return hipSuccess;
  }
  memmove(dst, src, n);
  return hipSuccess;
}
hipError_t f_hipMemcpyHtoDAsync(hipDeviceptr_t d, const void* s, size_t n, hipStream_t st) {
  FAKE_FAIL("hipMemcpyHtoDAsync");
  return copy_or_record(d, s, n, st);
}
hipError_t f_hipMemcpyDtoHAsync(void* d, hipDeviceptr_t s, size_t n, hipStream_t st) {
  FAKE_FAIL("hipMemcpyDtoHAsync");
  return copy_or_record(d, s, n, st);
}
hipError_t f_hipMemcpyDtoDAsync(hipDeviceptr_t d, hipDeviceptr_t s, size_t n, hipStream_t st) {
  FAKE_FAIL("hipMemcpyDtoDAsync");
  return copy_or_record(d, s, n, st);
}
hipError_t f_hipHostMalloc(void** p, size_t bytes, unsigned int) { FAKE_FAIL("hipHostMalloc"); return fake_alloc(p, bytes); }
hipError_t f_hipHostGetDevicePointer(void** d, void* h, unsigned int) { *d = h; return hipSuccess; }
hipError_t f_hipHostFree(void* p) { return fake_free(p); }
struct FakePool { uint64_t threshold = 0; };
hipError_t f_hipMemPoolCreate(hipMemPool_t* p, const hipMemPoolProps*) {
  FAKE_FAIL("hipMemPoolCreate");
  *p = reinterpret_cast<hipMemPool_t>(new FakePool());
  return hipSuccess;
}
FakePool g_default_pool;
hipError_t f_hipDeviceGetDefaultMemPool(hipMemPool_t* p, int) { *p = reinterpret_cast<hipMemPool_t>(&g_default_pool); return hipSuccess; }
hipError_t f_hipMemPoolDestroy(hipMemPool_t p) {
  if (reinterpret_cast<FakePool*>(p) != &g_default_pool) delete reinterpret_cast<FakePool*>(p);
  return hipSuccess;
}
hipError_t f_hipMemPoolSetAttribute(hipMemPool_t p, hipMemPoolAttr a, void* v) {
  if (a == hipMemPoolAttrReleaseThreshold) reinterpret_cast<FakePool*>(p)->threshold = *reinterpret_cast<uint64_t*>(v);
  return hipSuccess;
}
hipError_t f_hipMemPoolGetAttribute(hipMemPool_t p, hipMemPoolAttr a, void* v) {
  uint64_t out = 0;
  if (a == hipMemPoolAttrReleaseThreshold) out = reinterpret_cast<FakePool*>(p)->threshold;
  if (a == hipMemPoolAttrUsedMemCurrent || a == hipMemPoolAttrReservedMemCurrent) out = g_bytes.load();
  *reinterpret_cast<uint64_t*>(v) = out;
  return hipSuccess;
}
struct FakeGraphExec { FakeGraph graph; };
hipError_t f_hipGraphInstantiateWithFlags(hipGraphExec_t* e, hipGraph_t g, unsigned long long) {
  FAKE_FAIL("hipGraphInstantiateWithFlags");
  auto* ex = new FakeGraphExec();
  ex->graph = *reinterpret_cast<FakeGraph*>(g);
  *e = reinterpret_cast<hipGraphExec_t>(ex);
  return hipSuccess;
}
hipError_t f_hipGraphUpload(hipGraphExec_t, hipStream_t) { FAKE_FAIL("hipGraphUpload"); return hipSuccess; }
hipError_t f_hipGraphLaunch(hipGraphExec_t e, hipStream_t s) {
  FAKE_FAIL("hipGraphLaunch");
  auto* ex = reinterpret_cast<FakeGraphExec*>(e);
  for (auto& n : ex->graph.nodes) {
    switch (n.kind) {
      case 0: {
        LaunchRecord r = n.launch;
        r.stream = s;
        r.in_capture = false;
        r.from_replay = true;
        std::lock_guard<std::mutex> lock(g_mu);
        g_log.push_back(std::move(r));
        break;
      }
      case 1: n.host.fn(n.host.user); break;
      case 2: memmove(n.dst, n.src, n.bytes); break;
      case 3: __atomic_store_n(reinterpret_cast<uint32_t*>(n.dst), n.value, __ATOMIC_RELEASE); break;
    }
  }
  return hipSuccess;
}
hipError_t f_hipGraphExecDestroy(hipGraphExec_t e) { delete reinterpret_cast<FakeGraphExec*>(e); return hipSuccess; }
hipError_t f_hipGraphDestroy(hipGraph_t g) { delete reinterpret_cast<FakeGraph*>(g); return hipSuccess; }

HipApi make_fake_table() {
  HipApi t;
  t.hipInit = f_hipInit;
  t.hipGetDeviceCount = f_hipGetDeviceCount;
  t.hipSetDevice = f_hipSetDevice;
  t.hipGetDevice = f_hipGetDevice;
  t.hipDeviceSynchronize = f_hipDeviceSynchronize;
  t.hipDeviceGetAttribute = f_hipDeviceGetAttribute;
  t.hipDeviceGetName = f_hipDeviceGetName;
  t.hipDeviceTotalMem = f_hipDeviceTotalMem;
  t.hipGetDevicePropertiesR0600 = f_hipGetDeviceProperties;
  t.hipGetErrorString = f_hipGetErrorString;
  t.hipStreamCreateWithFlags = f_hipStreamCreateWithFlags;
  t.hipStreamSynchronize = f_hipStreamSynchronize;
  t.hipStreamQuery = f_hipStreamQuery;
  t.hipLaunchHostFunc = f_hipLaunchHostFunc;
  t.hipStreamBeginCapture = f_hipStreamBeginCapture;
  t.hipStreamEndCapture = f_hipStreamEndCapture;
  t.hipStreamWriteValue32 = f_hipStreamWriteValue32;
  t.hipEventCreateWithFlags = f_hipEventCreateWithFlags;
  t.hipEventRecord = f_hipEventRecord;
  t.hipEventSynchronize = f_hipEventSynchronize;
  t.hipEventElapsedTime = f_hipEventElapsedTime;
  t.hipEventDestroy = f_hipEventDestroy;
  t.hipModuleLoadData = f_hipModuleLoadData;
  t.hipModuleUnload = f_hipModuleUnload;
  t.hipModuleGetFunction = f_hipModuleGetFunction;
  t.hipModuleLaunchKernel = f_hipModuleLaunchKernel;
  t.hipMallocAsync = f_hipMallocAsync;
  t.hipMallocFromPoolAsync = f_hipMallocFromPoolAsync;
  t.hipFreeAsync = f_hipFreeAsync;
  t.hipMemsetD8Async = f_hipMemsetD8Async;
  t.hipMemcpyHtoDAsync = f_hipMemcpyHtoDAsync;
  t.hipMemcpyDtoHAsync = f_hipMemcpyDtoHAsync;
  t.hipMemcpyDtoDAsync = f_hipMemcpyDtoDAsync;
  t.hipHostMalloc = f_hipHostMalloc;
  t.hipHostGetDevicePointer = f_hipHostGetDevicePointer;
  t.hipHostFree = f_hipHostFree;
  t.hipMemPoolCreate = f_hipMemPoolCreate;
  t.hipDeviceGetDefaultMemPool = f_hipDeviceGetDefaultMemPool;
  t.hipMemPoolDestroy = f_hipMemPoolDestroy;
  t.hipMemPoolSetAttribute = f_hipMemPoolSetAttribute;
  t.hipMemPoolGetAttribute = f_hipMemPoolGetAttribute;
  t.hipGraphInstantiateWithFlags = f_hipGraphInstantiateWithFlags;
  t.hipGraphUpload = f_hipGraphUpload;
  t.hipGraphLaunch = f_hipGraphLaunch;
  t.hipGraphExecDestroy = f_hipGraphExecDestroy;
  t.hipGraphDestroy = f_hipGraphDestroy;
  return t;
}

const HipApi g_fake_table = make_fake_table();

}  // namespace
}  // namespace cutile

using namespace cutile;

extern "C" {

cutile_status_t cutile_testing_use_fake_hip(int32_t n_devices) {
  CUTILE_REQUIRE(n_devices >= 0 && n_devices <= 64, CUTILE_ERR_INVALID_ARGUMENT, "n_devices out of range");
  {
    std::lock_guard<std::mutex> lock(g_mu);
    g_n_devices = n_devices;
    g_failures.clear();
    g_log.clear();
  }
  t_device = 0;
  reset_runtime_for_testing();
  install_hip_api(&g_fake_table);
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_testing_use_real_hip(void) {
  reset_runtime_for_testing();
  install_hip_api(nullptr);
  return CUTILE_SUCCESS;
}

int32_t cutile_testing_launch_count(void) {
  std::lock_guard<std::mutex> lock(g_mu);
  return (int32_t)g_log.size();
}

cutile_status_t cutile_testing_get_launch(int32_t index, cutile_testing_launch_record_t* record) {
  CUTILE_REQUIRE(record, CUTILE_ERR_INVALID_ARGUMENT, "record is null");
  std::lock_guard<std::mutex> lock(g_mu);
  CUTILE_REQUIRE(index >= 0 && index < (int32_t)g_log.size(), CUTILE_ERR_INVALID_ARGUMENT, "launch index out of range");
  const LaunchRecord& r = g_log[index];  // deque: stable until cleared
  record->symbol = r.symbol.c_str();
  memcpy(record->grid, r.grid, sizeof(r.grid));
  memcpy(record->block, r.block, sizeof(r.block));
  record->shared_mem_bytes = r.smem;
  record->stream = r.stream;
  record->args = r.args.data();
  record->args_size = r.args.size();
  record->in_capture = r.in_capture;
  record->from_graph_replay = r.from_replay;
  return CUTILE_SUCCESS;
}

void cutile_testing_clear_log(void) {
  std::lock_guard<std::mutex> lock(g_mu);
  g_log.clear();
}

cutile_status_t cutile_testing_inject_failure(const char* hip_function, int32_t hip_error, int32_t count) {
  CUTILE_REQUIRE(hip_function, CUTILE_ERR_INVALID_ARGUMENT, "hip_function is null");
  std::lock_guard<std::mutex> lock(g_mu);
  g_failures[hip_function] = {hip_error, count};
  return CUTILE_SUCCESS;
}

uint64_t cutile_testing_streams_created(void) { return g_streams_created.load(); }
uint64_t cutile_testing_bytes_allocated(void) { return g_bytes.load(); }

}  // extern "C"
