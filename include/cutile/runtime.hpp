// RAII wrappers over Part A of the C ABI: Device, Stream, Event, MemPool,
// and the ExecutionContext a DeviceOp executes in.
//
// Mirrors cuda-core/src/runtime.rs (Device :82-139, Stream :489-780, Event
// :534-594, MemPool :374-465) and cuda-async/src/device_operation.rs:59-113
// (ExecutionContext).  Handles are shared_ptr where the reference uses Arc.
#pragma once
#include <memory>
#include <string>
#include <vector>

#include "error.hpp"

namespace cutile {

class Stream;
class MemPool;

class Device : public std::enable_shared_from_this<Device> {
 public:
  // Device::new(ordinal) — runtime.rs:126-139
  static Result<std::shared_ptr<Device>> create(int ordinal) {
    cutile_device_t h = nullptr;
    CUTILE_TRY_STATUS(cutile_device_get(ordinal, &h));
    return std::shared_ptr<Device>(new Device(ordinal, h));
  }
  static Result<int> device_count() {  // runtime.rs:196
    int32_t n = 0;
    CUTILE_TRY_STATUS(cutile_device_count(&n));
    return (int)n;
  }
  int ordinal() const { return ordinal_; }
  cutile_device_t handle() const { return handle_; }
  Result<std::string> name() const {  // runtime.rs:214
    char buf[256];
    CUTILE_TRY_STATUS(cutile_device_name(handle_, buf, sizeof(buf)));
    return std::string(buf);
  }
  Result<std::string> arch() const {
    char buf[256];
    CUTILE_TRY_STATUS(cutile_device_arch(handle_, buf, sizeof(buf)));
    return std::string(buf);
  }
  Result<Unit> bind_to_thread() const { return check(cutile_device_bind_to_thread(handle_)); }  // runtime.rs:229
  Result<Unit> synchronize() const { return check(cutile_device_synchronize(handle_)); }        // runtime.rs:244
  Result<size_t> l2_cache_size_bytes() const {                                                   // runtime.rs:597
    size_t b = 0;
    CUTILE_TRY_STATUS(cutile_device_l2_cache_size(handle_, &b));
    return b;
  }
  Result<cutile_device_props_t> props() const {
    cutile_device_props_t p;
    CUTILE_TRY_STATUS(cutile_device_props(handle_, &p));
    return p;
  }
  inline Result<std::shared_ptr<Stream>> new_stream();        // runtime.rs:249
  inline Result<std::shared_ptr<MemPool>> new_mem_pool();     // runtime.rs:335
  inline Result<std::shared_ptr<MemPool>> default_mem_pool(); // runtime.rs:354

 private:
  Device(int ordinal, cutile_device_t h) : ordinal_(ordinal), handle_(h) {}
  int ordinal_;
  cutile_device_t handle_;
};

class Stream {
 public:
  // Owned streams go back to the device's pool on drop; they are never destroyed
  // (runtime.rs:504-520,613-631).
  ~Stream() {
    if (owned_ && raw_) cutile_stream_release(device_->handle(), raw_);
  }
  Stream(const Stream&) = delete;
  Stream& operator=(const Stream&) = delete;
  // Stream::borrow_raw — runtime.rs:646: wraps a stream owned by someone else.
  static std::shared_ptr<Stream> borrow_raw(cutile_stream_t raw, std::shared_ptr<Device> device) {
    return std::shared_ptr<Stream>(new Stream(std::move(device), raw, false));
  }
  cutile_stream_t raw() const { return raw_; }
  const std::shared_ptr<Device>& device() const { return device_; }
  Result<Unit> synchronize() const { return check(cutile_stream_synchronize(raw_)); }  // runtime.rs:696
  Result<bool> query() const {                                                          // runtime.rs:706
    int32_t done = 0;
    CUTILE_TRY_STATUS(cutile_stream_query(raw_, &done));
    return done != 0;
  }

 private:
  friend class Device;
  Stream(std::shared_ptr<Device> d, cutile_stream_t raw, bool owned) : device_(std::move(d)), raw_(raw), owned_(owned) {}
  std::shared_ptr<Device> device_;
  cutile_stream_t raw_;
  bool owned_;
};

inline Result<std::shared_ptr<Stream>> Device::new_stream() {
  cutile_stream_t s = nullptr;
  CUTILE_TRY_STATUS(cutile_stream_create(handle_, &s));
  return std::shared_ptr<Stream>(new Stream(shared_from_this(), s, true));
}

class Event {  // runtime.rs:534-594
 public:
  static Result<std::unique_ptr<Event>> create() {
    cutile_event_t e = nullptr;
    CUTILE_TRY_STATUS(cutile_event_create(&e));
    return std::unique_ptr<Event>(new Event(e));
  }
  ~Event() { cutile_event_destroy(raw_); }
  Result<Unit> record(const Stream& s) { return check(cutile_event_record(raw_, s.raw())); }
  Result<Unit> synchronize() { return check(cutile_event_synchronize(raw_)); }
  Result<float> elapsed_ms(const Event& end) const {
    float ms = 0;
    CUTILE_TRY_STATUS(cutile_event_elapsed_ms(raw_, end.raw_, &ms));
    return ms;
  }

 private:
  explicit Event(cutile_event_t e) : raw_(e) {}
  cutile_event_t raw_;
};

class MemPool {  // runtime.rs:374-465
 public:
  ~MemPool() {
    if (owned_) cutile_mempool_destroy(raw_);
  }
  cutile_mempool_t raw() const { return raw_; }
  Result<Unit> set_release_threshold(uint64_t bytes) { return check(cutile_mempool_set_release_threshold(raw_, bytes)); }
  Result<cutile_pool_mem_stats_t> mem_stats() const {
    cutile_pool_mem_stats_t st;
    CUTILE_TRY_STATUS(cutile_mempool_stats(raw_, &st));
    return st;
  }
  Result<Unit> reset_used_high() { return check(cutile_mempool_reset_used_high(raw_)); }
  Result<Unit> reset_reserved_high() { return check(cutile_mempool_reset_reserved_high(raw_)); }

 private:
  friend class Device;
  MemPool(cutile_mempool_t p, bool owned) : raw_(p), owned_(owned) {}
  cutile_mempool_t raw_;
  bool owned_;
};

inline Result<std::shared_ptr<MemPool>> Device::new_mem_pool() {
  cutile_mempool_t p = nullptr;
  CUTILE_TRY_STATUS(cutile_mempool_create(handle_, &p));
  return std::shared_ptr<MemPool>(new MemPool(p, true));
}
inline Result<std::shared_ptr<MemPool>> Device::default_mem_pool() {
  cutile_mempool_t p = nullptr;
  CUTILE_TRY_STATUS(cutile_mempool_default(handle_, &p));
  return std::shared_ptr<MemPool>(new MemPool(p, false));
}

// What a DeviceOp executes in: the stream (hence the device) plus the thread's
// memory pool for that device, if one was set (device_operation.rs:59-113).
class ExecutionContext {
 public:
  explicit ExecutionContext(std::shared_ptr<Stream> stream) : stream_(std::move(stream)) {
    cutile_mempool_t p = nullptr;
    if (cutile_get_device_pool(stream_->device()->ordinal(), &p) == CUTILE_SUCCESS) pool_ = p;
  }
  const std::shared_ptr<Stream>& stream() const { return stream_; }
  const std::shared_ptr<Device>& device() const { return stream_->device(); }
  int device_id() const { return stream_->device()->ordinal(); }
  cutile_mempool_t pool() const { return pool_; }
  // alloc_async — device_operation.rs:95-100: from the thread's pool if set.
  Result<void*> alloc_async(size_t bytes) const {
    void* p = nullptr;
    if (pool_)
      CUTILE_TRY_STATUS(cutile_malloc_from_pool_async(bytes, pool_, stream_->raw(), &p));
    else
      CUTILE_TRY_STATUS(cutile_malloc_async(bytes, stream_->raw(), &p));
    return p;
  }

 private:
  std::shared_ptr<Stream> stream_;
  cutile_mempool_t pool_ = nullptr;
};

// ---- thread-local device contexts and scheduling policies (device_context.rs, scheduling_policies.rs) ----
inline int get_default_device() { return cutile_get_default_device(); }
inline void set_default_device(int ordinal) { cutile_set_default_device(ordinal); }
enum class PolicyKind { StreamPoolRoundRobin = CUTILE_POLICY_ROUND_ROBIN, SingleStream = CUTILE_POLICY_SINGLE_STREAM };
inline Result<Unit> init_device_contexts(int default_device, int num_devices) {
  return check(cutile_init_device_contexts(default_device, num_devices));
}
inline Result<Unit> init_device(int ordinal, PolicyKind kind, int num_streams = 0) {
  return check(cutile_init_device(ordinal, (cutile_policy_kind_t)kind, num_streams));
}
// with_default_device_policy(|p| p.next_stream()) — device_context.rs:444-450.  The
// stream belongs to the thread's policy; the returned handle only borrows it.
inline Result<std::shared_ptr<Stream>> next_stream(int ordinal = -1) {
  if (ordinal < 0) ordinal = cutile_get_default_device();
  auto dev = Device::create(ordinal);
  if (dev.is_err()) return dev.error();
  cutile_stream_t s = nullptr;
  CUTILE_TRY_STATUS(cutile_policy_next_stream(ordinal, &s));
  return Stream::borrow_raw(s, std::move(dev).unwrap());
}

}  // namespace cutile
