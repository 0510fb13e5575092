// Part E of the C ABI: the asynchronous runtime — the non-generic half of what
// the reference keeps in its cuda-async crate.
//
//  * the thread-local execution lock (one DeviceOp executing per thread,
//    cuda-async/src/device_operation.rs:27-55);
//  * thread-local device contexts: default device, one scheduling policy per
//    device (round robin over 4 streams by default, or a single stream), a
//    dedicated deallocator stream, an optional memory pool
//    (cuda-async/src/device_context.rs:139-450, scheduling_policies.rs:35-87);
//  * the completion reactor: after the submitted work the stream writes a
//    per-use stamp into a pinned, device-mapped word, and one sweeper thread
//    fires the waker of every slot whose word shows its stamp (slot_table.h;
//    observable behaviour of cuda-async/src/reactor.rs:68-179: 1024 slots, an
//    out-of-slots status); host-callback fallback chain as in
//    cuda-async/src/device_future.rs:103-154.
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

#include "common.h"
#include "runtime_state.h"
#include "slot_table.h"

using namespace cutile;

namespace cutile {
namespace {

// ---- execution lock ------------------------------------------------------------------------
thread_local bool t_executing = false;

// ---- thread-local device contexts ----------------------------------------------------------
struct Policy {
  int kind = CUTILE_POLICY_ROUND_ROBIN;
  std::vector<cutile_stream_t> streams;
  std::atomic<size_t> next{0};
};
struct DeviceContext {
  int ordinal = 0;
  cutile_stream_t deallocator = nullptr;
  std::unique_ptr<Policy> policy;
  cutile_mempool_t pool = nullptr;
};
struct ThreadContexts {
  int default_device = 0;
  bool initialized = false;
  std::map<int, DeviceContext> devices;
  uint64_t epoch = 0;
  ~ThreadContexts();
};
thread_local ThreadContexts t_ctx;
std::atomic<uint64_t> g_epoch{1};  // bumped when a test swaps the runtime: stale contexts are dropped

void drop_if_stale() {
  uint64_t e = g_epoch.load(std::memory_order_acquire);
  if (t_ctx.epoch != e) {
    t_ctx.devices.clear();  // streams belong to the previous runtime; never destroyed
    t_ctx.initialized = false;
    t_ctx.default_device = 0;
    t_ctx.epoch = e;
  }
}

ThreadContexts::~ThreadContexts() {
  // A thread's streams go back to the device pool (streams are never destroyed).
  if (epoch != g_epoch.load(std::memory_order_acquire)) return;
  for (auto& kv : devices) {
    cutile_device_t dev = nullptr;
    if (cutile_device_get(kv.first, &dev) != CUTILE_SUCCESS) continue;
    if (kv.second.deallocator) cutile_stream_release(dev, kv.second.deallocator);
    if (kv.second.policy)
      for (auto s : kv.second.policy->streams) cutile_stream_release(dev, s);
  }
}

constexpr int kDefaultPoolStreams = 4;  // DEFAULT_ROUND_ROBIN_STREAM_POOL_SIZE, device_context.rs:39

cutile_status_t make_context(int ordinal, int kind, int num_streams, DeviceContext* out) {
  cutile_device_t dev = nullptr;
  if (cutile_status_t s = cutile_device_get(ordinal, &dev)) return s;
  CUTILE_REQUIRE(kind == CUTILE_POLICY_ROUND_ROBIN || kind == CUTILE_POLICY_SINGLE_STREAM, CUTILE_ERR_INVALID_ARGUMENT,
                 "unknown scheduling policy %d", kind);
  if (kind == CUTILE_POLICY_SINGLE_STREAM) num_streams = 1;
  CUTILE_REQUIRE(num_streams >= 1 && num_streams <= 64, CUTILE_ERR_INVALID_ARGUMENT, "policy needs 1..64 streams");
  out->ordinal = ordinal;
  out->policy = std::make_unique<Policy>();
  out->policy->kind = kind;
  for (int i = 0; i < num_streams; ++i) {
    cutile_stream_t st = nullptr;
    if (cutile_status_t s = cutile_stream_create(dev, &st)) return s;
    out->policy->streams.push_back(st);
  }
  return cutile_stream_create(dev, &out->deallocator);
}

cutile_status_t context_for(int ordinal, DeviceContext** out) {
  drop_if_stale();
  if (ordinal < 0) ordinal = t_ctx.default_device;
  auto it = t_ctx.devices.find(ordinal);
  if (it == t_ctx.devices.end()) {
    // Lazy initialisation with the default policy (init_with_default_policy).
    DeviceContext ctx;
    if (cutile_status_t s = make_context(ordinal, CUTILE_POLICY_ROUND_ROBIN, kDefaultPoolStreams, &ctx)) return s;
    t_ctx.initialized = true;
    it = t_ctx.devices.emplace(ordinal, std::move(ctx)).first;
  }
  *out = &it->second;
  return CUTILE_SUCCESS;
}

// ---- reactor -------------------------------------------------------------------------------
struct Waker {
  cutile_waker_fn_t fn;
  void* user;
};

struct PinnedWords {
  uint32_t* host = nullptr;
  std::atomic<uint32_t>& word(size_t slot) { return *reinterpret_cast<std::atomic<uint32_t>*>(host + slot); }
};
static_assert(sizeof(std::atomic<uint32_t>) == sizeof(uint32_t), "the pinned slab is viewed as atomics");

constexpr size_t kNumSlots = 1024;     // reactor.rs:29
constexpr uint32_t kSpinPasses = 10000;  // reactor.rs:31

struct Reactor {
  std::unique_ptr<SlotTable<Waker, PinnedWords>> table;
  void* device_flags = nullptr;
  std::thread scanner;
  std::mutex park_mutex;
  std::condition_variable park_cv;
  bool unpark_token = false;
  std::atomic<bool> stop{false};
  std::atomic<uint64_t> registrations{0}, wakes{0};

  void unpark() {
    {
      std::lock_guard<std::mutex> lock(park_mutex);
      unpark_token = true;
    }
    park_cv.notify_one();
  }
  void park() {
    std::unique_lock<std::mutex> lock(park_mutex);
    park_cv.wait(lock, [&] { return unpark_token || stop.load(); });
    unpark_token = false;  // a wake that raced ahead of the park is absorbed by the token
  }
  void scan_loop() {
    std::vector<Waker> woken;
    uint32_t idle_passes = 0;
    while (!stop.load(std::memory_order_acquire)) {
      table->sweep(woken);
      if (!woken.empty()) {
        // Wakers fire outside any lock the scan held.
        for (auto& w : woken) {
          wakes.fetch_add(1, std::memory_order_relaxed);
          w.fn(w.user);
        }
        woken.clear();
        idle_passes = 0;
        continue;
      }
      // Sleep only when the pending count reads 0: a slot armed after this pass looked at it is counted already.
      if (table->nothing_pending()) {
        park();
        idle_passes = 0;
        continue;
      }
      if (++idle_passes < kSpinPasses)
        __builtin_ia32_pause();
      else
        std::this_thread::yield();
    }
  }
};

std::mutex g_reactor_mutex;
Reactor* g_reactor = nullptr;      // leaked on purpose: the scanner may outlive static destructors
std::string g_reactor_error;
uint64_t g_reactor_epoch = 0;

cutile_status_t reactor(Reactor** out) {
  std::lock_guard<std::mutex> lock(g_reactor_mutex);
  uint64_t e = g_epoch.load(std::memory_order_acquire);
  if (g_reactor && g_reactor_epoch != e) {
    // The runtime was swapped under a test: retire the old scanner.
    g_reactor->stop.store(true);
    g_reactor->unpark();
    if (g_reactor->scanner.joinable()) g_reactor->scanner.join();
    g_reactor = nullptr;
    g_reactor_error.clear();
  }
  if (!g_reactor && g_reactor_error.empty()) {
    void *host = nullptr, *dev = nullptr;
    cutile_status_t s = cutile_host_alloc_mapped(kNumSlots * sizeof(uint32_t), &host, &dev);
    if (s != CUTILE_SUCCESS) {
      g_reactor_error = std::string("reactor: pinned flag slab allocation failed: ") + cutile_last_error_message();
    } else {
      memset(host, 0, kNumSlots * sizeof(uint32_t));
      auto* r = new Reactor();
      r->table = std::make_unique<SlotTable<Waker, PinnedWords>>(kNumSlots, PinnedWords{(uint32_t*)host});
      r->device_flags = dev;
      r->scanner = std::thread([r] { r->scan_loop(); });
      g_reactor = r;
      g_reactor_epoch = e;
    }
  }
  if (!g_reactor) return fail(CUTILE_ERR_STATE, "%s", g_reactor_error.c_str());
  *out = g_reactor;
  return CUTILE_SUCCESS;
}

struct HostFnPayload {
  Waker w;
};
void host_fn_trampoline(void* p) {
  auto* payload = static_cast<HostFnPayload*>(p);
  payload->w.fn(payload->w.user);
  delete payload;
}

}  // namespace

// Called when a test swaps the HIP runtime under the library.
void reset_async_runtime_for_testing() { g_epoch.fetch_add(1, std::memory_order_acq_rel); }

}  // namespace cutile

extern "C" {

// ---- execution lock ------------------------------------------------------------------------
cutile_status_t cutile_execution_lock_acquire(void) {
  if (t_executing)
    return fail(CUTILE_ERR_STATE,
                "DeviceOp execution is non-reentrant: another DeviceOp is already executing on this thread. If this "
                "is intentional and you have verified there are no cross-stream data races, use `then_unchecked`.");
  t_executing = true;
  return CUTILE_SUCCESS;
}
void cutile_execution_lock_release(void) { t_executing = false; }
int32_t cutile_execution_lock_held(void) { return t_executing ? 1 : 0; }

// ---- device contexts -----------------------------------------------------------------------
int32_t cutile_get_default_device(void) {
  drop_if_stale();
  return t_ctx.default_device;
}
void cutile_set_default_device(int32_t ordinal) {
  drop_if_stale();
  t_ctx.default_device = ordinal;
}

cutile_status_t cutile_init_device_contexts(int32_t default_device, int32_t num_devices) {
  drop_if_stale();
  (void)num_devices;
  CUTILE_REQUIRE(!t_ctx.initialized, CUTILE_ERR_STATE, "Context { device_id: %d, message: \"Context already initialized.\" }",
                 default_device);
  t_ctx.initialized = true;
  t_ctx.default_device = default_device;
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_init_device(int32_t ordinal, cutile_policy_kind_t kind, int32_t num_streams) {
  drop_if_stale();
  CUTILE_REQUIRE(t_ctx.devices.find(ordinal) == t_ctx.devices.end(), CUTILE_ERR_STATE,
                 "Context { device_id: %d, message: \"Device is already initialized.\" }", ordinal);
  DeviceContext ctx;
  if (cutile_status_t s = make_context(ordinal, kind, num_streams > 0 ? num_streams : kDefaultPoolStreams, &ctx)) return s;
  t_ctx.initialized = true;
  t_ctx.devices.emplace(ordinal, std::move(ctx));
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_policy_next_stream(int32_t ordinal, cutile_stream_t* stream) {
  CUTILE_REQUIRE(stream, CUTILE_ERR_INVALID_ARGUMENT, "stream is null");
  DeviceContext* ctx = nullptr;
  if (cutile_status_t s = context_for(ordinal, &ctx)) return s;
  Policy& p = *ctx->policy;
  CUTILE_REQUIRE(!p.streams.empty(), CUTILE_ERR_STATE, "Scheduling: policy has no streams");
  size_t idx = p.next.fetch_add(1, std::memory_order_relaxed) % p.streams.size();
  *stream = p.streams[idx];
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_deallocator_stream(int32_t ordinal, cutile_stream_t* stream) {
  CUTILE_REQUIRE(stream, CUTILE_ERR_INVALID_ARGUMENT, "stream is null");
  DeviceContext* ctx = nullptr;
  if (cutile_status_t s = context_for(ordinal, &ctx)) return s;
  *stream = ctx->deallocator;
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_set_device_pool(int32_t ordinal, cutile_mempool_t pool) {
  DeviceContext* ctx = nullptr;
  if (cutile_status_t s = context_for(ordinal, &ctx)) return s;
  ctx->pool = pool;
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_get_device_pool(int32_t ordinal, cutile_mempool_t* pool) {
  CUTILE_REQUIRE(pool, CUTILE_ERR_INVALID_ARGUMENT, "pool is null");
  DeviceContext* ctx = nullptr;
  if (cutile_status_t s = context_for(ordinal, &ctx)) return s;
  *pool = ctx->pool;
  return CUTILE_SUCCESS;
}

// ---- completion notification ---------------------------------------------------------------
cutile_status_t cutile_reactor_register(cutile_stream_t stream, cutile_waker_fn_t waker, void* user) {
  CUTILE_REQUIRE(waker, CUTILE_ERR_INVALID_ARGUMENT, "waker is null");
  Reactor* r = nullptr;
  if (cutile_status_t s = reactor(&r)) return s;
  auto ticket = r->table->acquire();
  if (!ticket) return fail(CUTILE_ERR_OUT_OF_SLOTS, "reactor slot pool exhausted");
  // The stream stores this use's stamp; whatever an earlier use left in the word is a different value.
  void* addr = static_cast<char*>(r->device_flags) + ticket->slot * sizeof(uint32_t);
  cutile_status_t s = cutile_stream_write_value32(stream, addr, ticket->stamp);
  if (s != CUTILE_SUCCESS) {
    r->table->abandon(*ticket);
    return s;
  }
  r->registrations.fetch_add(1, std::memory_order_relaxed);
  if (r->table->arm(*ticket, Waker{waker, user})) r->unpark();
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_completion_register(cutile_stream_t stream, cutile_waker_fn_t waker, void* user) {
  CUTILE_REQUIRE(waker, CUTILE_ERR_INVALID_ARGUMENT, "waker is null");
  // CUTILE_ASYNC_HOST_SYNC=callback forces the host-function path (the reference's
  // CUDA_ASYNC_HOST_SYNC switch); otherwise reactor first, host function as fallback.
  static const bool force_callback = [] {
    const char* v = getenv("CUTILE_ASYNC_HOST_SYNC");
    return v && (!strcmp(v, "callback") || !strcmp(v, "spin") || !strcmp(v, "block"));
  }();
  if (!force_callback && cutile_reactor_register(stream, waker, user) == CUTILE_SUCCESS) return CUTILE_SUCCESS;
  auto* payload = new HostFnPayload{Waker{waker, user}};
  cutile_status_t s = cutile_stream_launch_host_func(stream, host_fn_trampoline, payload);
  if (s != CUTILE_SUCCESS) delete payload;
  return s;
}

uint64_t cutile_reactor_registrations(void) {
  std::lock_guard<std::mutex> lock(g_reactor_mutex);
  return g_reactor ? g_reactor->registrations.load() : 0;
}
uint64_t cutile_reactor_wakes(void) {
  std::lock_guard<std::mutex> lock(g_reactor_mutex);
  return g_reactor ? g_reactor->wakes.load() : 0;
}
int32_t cutile_reactor_armed(void) {
  std::lock_guard<std::mutex> lock(g_reactor_mutex);
  return g_reactor ? (int32_t)g_reactor->table->pending() : 0;
}

}  // extern "C"
