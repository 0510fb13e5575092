// Completion slot table of the reactor: a fixed pool of slots, each with a
// host-visible completion flag that the GPU sets to 1 (a stream write into
// pinned, device-mapped memory) and a waker payload that one scanner thread
// fires when it sees the flag.
//
// Protocol (follows cuda-async/src/slot_table.rs:39-166):
//   registrant:  claim() -> reset_flag() -> [enqueue the device write] ->
//                publish(slot, payload)           (or release(slot) on failure)
//   scanner:     scan_once(): for every armed slot whose flag reads 1: clear
//                its bit, take the payload, recycle the index.
// Ordering: the payload is written, then n_armed is incremented, then the active
// bit is set with release; the scanner loads the bit with acquire before it
// touches the payload, and decrements n_armed only after recycling, so the count
// never underflows and the scanner may park exactly when n_armed == 0.  publish()
// reports the 0 -> 1 transition so the registrant wakes the scanner only when it
// may be parked.
//
// The flag array is a template parameter so the protocol can be exercised on the
// CPU with plain atomics standing in for pinned memory (the reference does the
// same with its MockFlags, slot_table.rs:182-190).
#pragma once
#include <atomic>
#include <cstddef>
#include <cstdint>
#include <mutex>
#include <optional>
#include <vector>

namespace cutile {

template <typename Payload, typename Flags>
class SlotTable {
 public:
  SlotTable(size_t num_slots, Flags flags)
      : flags_(std::move(flags)), active_((num_slots + 63) / 64), payload_(num_slots), num_slots_(num_slots) {
    for (auto& w : active_) w.store(0, std::memory_order_relaxed);
    free_.reserve(num_slots);
    for (size_t i = num_slots; i-- > 0;) free_.push_back(i);
  }

  bool is_idle() const { return n_armed_.load(std::memory_order_acquire) == 0; }
  size_t armed() const { return n_armed_.load(std::memory_order_acquire); }

  // Reserves an idle slot; empty when the pool is exhausted.
  std::optional<size_t> claim() {
    std::lock_guard<std::mutex> lock(free_mutex_);
    if (free_.empty()) return std::nullopt;
    size_t s = free_.back();
    free_.pop_back();
    return s;
  }
  // Returns a claimed slot that was never published (the device write failed).
  void release(size_t slot) {
    std::lock_guard<std::mutex> lock(free_mutex_);
    free_.push_back(slot);
  }
  // Must run before the device write is enqueued, so a stale 0 cannot clobber the 1.
  void reset_flag(size_t slot) { flags_.flag(slot).store(0, std::memory_order_release); }

  // Publishes a claimed, armed slot.  Returns true on the idle -> active transition.
  bool publish(size_t slot, Payload payload) {
    payload_[slot] = std::move(payload);
    bool was_idle = n_armed_.fetch_add(1, std::memory_order_acq_rel) == 0;
    active_[slot / 64].fetch_or(uint64_t(1) << (slot % 64), std::memory_order_release);
    return was_idle;
  }

  // One scan pass; retired payloads are appended to `woken`.  Returns whether any
  // slot was still armed when the pass looked at it.
  bool scan_once(std::vector<Payload>& woken) {
    bool any_active = false;
    retired_.clear();
    for (size_t word = 0; word < active_.size(); ++word) {
      uint64_t bits = active_[word].load(std::memory_order_acquire);
      if (!bits) continue;
      any_active = true;
      while (bits) {
        int bit = __builtin_ctzll(bits);
        bits &= bits - 1;
        size_t slot = word * 64 + bit;
        if (slot >= num_slots_) break;
        if (flags_.flag(slot).load(std::memory_order_acquire) == 1) {
          active_[word].fetch_and(~(uint64_t(1) << bit), std::memory_order_acq_rel);
          // Sole consumer: the bit was observed set, and the slot cannot be
          // claimed again until it is recycled below.
          if (payload_[slot]) {
            woken.push_back(std::move(*payload_[slot]));
            payload_[slot].reset();
          }
          retired_.push_back(slot);
        }
      }
    }
    if (!retired_.empty()) {
      size_t n = retired_.size();
      {
        std::lock_guard<std::mutex> lock(free_mutex_);
        free_.insert(free_.end(), retired_.begin(), retired_.end());
      }
      n_armed_.fetch_sub(n, std::memory_order_acq_rel);
    }
    return any_active;
  }

  Flags& flags() { return flags_; }
  size_t num_slots() const { return num_slots_; }

 private:
  Flags flags_;
  std::vector<std::atomic<uint64_t>> active_;
  std::vector<std::optional<Payload>> payload_;
  std::mutex free_mutex_;
  std::vector<size_t> free_;
  std::vector<size_t> retired_;  // scanner-private scratch
  std::atomic<size_t> n_armed_{0};
  size_t num_slots_;
};

}  // namespace cutile
