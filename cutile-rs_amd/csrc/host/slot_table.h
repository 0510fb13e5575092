// Completion slots of the reactor: a fixed pool of host-visible 32-bit words in pinned, device-mapped memory, one per
// pending notification.  A stream write (hipStreamWriteValue32) stores a slot's current STAMP into its word when
// the stream reaches that point; one sweeper thread compares words with stamps and hands out the payloads (wakers)
// of the slots whose write has landed.
//
// What the HIP side needs, and how this table gives it (observable contract: cuda-async/src/reactor.rs:68-179 —
// a bounded number of slots, an out-of-slots result the caller turns into the host-function fallback, every payload
// handed out exactly once, a sweeper that can sleep when nothing is pending):
//
//   * A stream write can carry any 32-bit value, so a slot is never "reset".  Each use of a slot has a generation;
//     the value written is that generation's stamp (never 0, the word's initial value).  The word left behind by
//     the previous use holds the previous stamp, which cannot equal the new one, so a stale word cannot complete a
//     reused slot and no host store has to be ordered against the device's write.
//   * One 64-bit control word per slot holds {generation, phase}; every transition is a single atomic operation on
//     it: FREE -(acquire(): compare-exchange, generation + 1)-> HELD -(arm(): store)-> ARMED -(sweep(): store)-> FREE,
//     or HELD -(abandon())-> FREE when the stream write could not be enqueued.  No lock, no free list, no bitmap.
//   * acquire() probes from a low-water hint, so live slots stay packed at the bottom and sweep() only looks at the
//     control words below the highest index ever handed out.
//   * pending() counts armed slots; arm() raises it BEFORE the slot becomes visible as ARMED and sweep() lowers it
//     AFTER the slots are free again, so it never under-reports and the sweeper may sleep exactly when it reads 0.
//     arm() returns whether it raised the count from 0: the one case in which the sweeper can be asleep.
//
// The word array is a template parameter, so the protocol runs on the CPU with plain atomics standing in for the
// pinned memory and a thread standing in for the device.
#pragma once
#include <atomic>
#include <cstddef>
#include <cstdint>
#include <memory>
#include <optional>
#include <vector>

namespace cutile {

struct SlotTicket {
  size_t slot;
  uint32_t stamp;  // the value the stream write must store into the slot's word
};

template <typename Payload, typename Words>
class SlotTable {
  enum Phase : uint64_t { kFree = 0, kHeld = 1, kArmed = 2, kPhaseMask = 3 };
  static uint64_t generation(uint64_t control) { return control >> 2; }
  static uint64_t control(uint64_t gen, Phase p) { return (gen << 2) | p; }

 public:
  // generation g -> 1 + (g mod (2^32 - 1)): consecutive generations never share a stamp, and no stamp is 0
  static uint32_t stamp_of(uint64_t gen) { return uint32_t(gen % 0xffffffffull) + 1u; }

  SlotTable(size_t num_slots, Words words)
      : words_(std::move(words)), control_(new std::atomic<uint64_t>[num_slots]), payload_(num_slots), num_slots_(num_slots) {
    for (size_t i = 0; i < num_slots; ++i) control_[i].store(control(0, kFree), std::memory_order_relaxed);
  }

  size_t num_slots() const { return num_slots_; }
  size_t pending() const { return pending_.load(std::memory_order_acquire); }
  bool nothing_pending() const { return pending() == 0; }
  Words& words() { return words_; }

  // Takes a free slot for one notification; empty when all are in use.
  std::optional<SlotTicket> acquire() {
    size_t start = hint_.load(std::memory_order_relaxed);
    if (start >= num_slots_) start = 0;
    for (size_t probe = 0; probe < num_slots_; ++probe) {
      size_t s = start + probe;
      if (s >= num_slots_) s -= num_slots_;
      uint64_t c = control_[s].load(std::memory_order_relaxed);
      if ((c & kPhaseMask) != kFree) continue;
      uint64_t gen = generation(c) + 1;
      if (!control_[s].compare_exchange_strong(c, control(gen, kHeld), std::memory_order_acquire, std::memory_order_relaxed)) continue;
      hint_.store(s + 1, std::memory_order_relaxed);
      raise_top(s + 1);
      return SlotTicket{s, stamp_of(gen)};
    }
    return std::nullopt;
  }

  // Gives back a ticket whose stream write was never enqueued.
  void abandon(const SlotTicket& t) {
    uint64_t c = control_[t.slot].load(std::memory_order_relaxed);
    control_[t.slot].store(control(generation(c), kFree), std::memory_order_release);
    lower_hint(t.slot);
  }

  // Attaches the payload to a ticket whose stream write is enqueued (the write may already have landed).
  // Returns true when nothing was pending before: the sweeper may be asleep and must be woken.
  bool arm(const SlotTicket& t, Payload payload) {
    payload_[t.slot] = std::move(payload);
    bool first = pending_.fetch_add(1, std::memory_order_acq_rel) == 0;
    uint64_t c = control_[t.slot].load(std::memory_order_relaxed);
    control_[t.slot].store(control(generation(c), kArmed), std::memory_order_release);
    return first;
  }

  // One pass of the sweeper (a single thread): moves the payload of every armed slot whose word holds its stamp into
  // `ready`, frees those slots, and returns how many it completed.
  size_t sweep(std::vector<Payload>& ready) {
    size_t top = top_.load(std::memory_order_acquire);
    size_t done = 0, lowest = num_slots_;
    for (size_t s = 0; s < top; ++s) {
      uint64_t c = control_[s].load(std::memory_order_acquire);
      if ((c & kPhaseMask) != kArmed) continue;
      if (words_.word(s).load(std::memory_order_acquire) != stamp_of(generation(c))) continue;
      ready.push_back(std::move(*payload_[s]));
      payload_[s].reset();
      control_[s].store(control(generation(c), kFree), std::memory_order_release);
      if (s < lowest) lowest = s;
      ++done;
    }
    if (done) {
      lower_hint(lowest);
      pending_.fetch_sub(done, std::memory_order_acq_rel);
    }
    return done;
  }

 private:
  void raise_top(size_t v) {
    size_t cur = top_.load(std::memory_order_relaxed);
    while (cur < v && !top_.compare_exchange_weak(cur, v, std::memory_order_release, std::memory_order_relaxed)) {
    }
  }
  void lower_hint(size_t v) {
    size_t cur = hint_.load(std::memory_order_relaxed);
    while (cur > v && !hint_.compare_exchange_weak(cur, v, std::memory_order_relaxed, std::memory_order_relaxed)) {
    }
  }

  Words words_;
  std::unique_ptr<std::atomic<uint64_t>[]> control_;
  std::vector<std::optional<Payload>> payload_;
  size_t num_slots_;
  std::atomic<size_t> pending_{0};
  std::atomic<size_t> hint_{0};  // where acquire() starts probing: a guess, never relied on
  std::atomic<size_t> top_{0};   // 1 + the highest slot index ever handed out: sweep()'s bound
};

}  // namespace cutile
