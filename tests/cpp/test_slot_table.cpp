// The reactor's completion-slot protocol under plain atomics standing in for pinned memory,
// with a modelled "GPU" thread that stores the stamps — the properties the reference checks of its own
// table (cuda-async/src/slot_table.rs:169-330: exactly-once wake, no stale completion, exhaustion, an
// 8 x 500 thread stress), asked of this one.
// Built with -fsanitize=thread as well, so the ordering claims are checked by
// the race detector and not only by the outcome.
#include <atomic>
#include <deque>
#include <memory>
#include <mutex>
#include <thread>

#include "../../cutile-rs_amd/csrc/host/slot_table.h"
#include "check.hpp"

using cutile::SlotTable;

struct HostWords {
  std::shared_ptr<std::vector<std::atomic<uint32_t>>> cells;
  explicit HostWords(size_t n) : cells(std::make_shared<std::vector<std::atomic<uint32_t>>>(n)) {
    for (auto& c : *cells) c.store(0);
  }
  std::atomic<uint32_t>& word(size_t slot) { return (*cells)[slot]; }
};
using Table = SlotTable<int, HostWords>;

TEST(acquire_arm_sweep_reuse) {
  Table t(4, HostWords(4));
  CHECK(t.nothing_pending());
  auto a = t.acquire();
  CHECK(a && a->slot == 0 && a->stamp != 0);  // lowest index first; a stamp is never the word's initial value
  CHECK(t.arm(*a, 42));                       // nothing was pending: the sweeper has to be woken
  auto b = t.acquire();
  CHECK(b && b->slot == 1);
  CHECK(!t.arm(*b, 43));                      // something already pending
  std::vector<int> ready;
  CHECK(t.sweep(ready) == 0 && ready.empty() && t.pending() == 2);  // armed, write not landed: nothing completes
  t.words().word(b->slot).store(b->stamp);
  CHECK(t.sweep(ready) == 1 && ready == std::vector<int>({43}) && t.pending() == 1);
  t.words().word(a->slot).store(a->stamp);
  ready.clear();
  CHECK(t.sweep(ready) == 1 && ready == std::vector<int>({42}) && t.nothing_pending());
  CHECK(t.sweep(ready) == 0);
  // freed slots are handed out again, lowest first, with a new stamp
  auto a2 = t.acquire();
  CHECK(a2 && a2->slot == 0 && a2->stamp != a->stamp);
  t.abandon(*a2);
  // exhaustion, and abandon() gives a ticket back
  std::vector<cutile::SlotTicket> held;
  while (auto c = t.acquire()) held.push_back(*c);
  CHECK(held.size() == 4 && !t.acquire());
  t.abandon(held.back());
  CHECK(t.acquire().has_value());
}

TEST(a_word_left_by_an_earlier_use_cannot_complete_the_slot) {
  Table t(1, HostWords(1));
  std::vector<int> ready;
  auto a = *t.acquire();
  t.arm(a, 1);
  t.words().word(0).store(a.stamp);
  CHECK(t.sweep(ready) == 1);
  // nobody clears the word: it still holds the first use's stamp when the slot is armed again
  auto b = *t.acquire();
  CHECK(b.slot == 0 && b.stamp != a.stamp);
  t.arm(b, 2);
  ready.clear();
  CHECK(t.sweep(ready) == 0 && ready.empty() && t.pending() == 1);
  t.words().word(0).store(b.stamp);
  CHECK(t.sweep(ready) == 1 && ready == std::vector<int>({2}));
}

TEST(write_that_lands_before_arm_is_found_by_the_next_sweep) {
  Table t(2, HostWords(2));
  std::vector<int> ready;
  auto a = *t.acquire();
  t.words().word(a.slot).store(a.stamp);   // the stream got there first
  CHECK(t.sweep(ready) == 0);              // held, not armed: no payload to hand out yet
  CHECK(t.arm(a, 7));
  CHECK(t.sweep(ready) == 1 && ready == std::vector<int>({7}) && t.nothing_pending());
}

TEST(stamps_never_zero_and_never_repeat_back_to_back) {
  for (uint64_t g : {uint64_t(0), uint64_t(1), uint64_t(0xfffffffeull), uint64_t(0xffffffffull), uint64_t(0x100000000ull), uint64_t(0x1fffffffeull)}) {
    CHECK(Table::stamp_of(g) != 0);
    CHECK(Table::stamp_of(g) != Table::stamp_of(g + 1));
  }
}

TEST(stress_eight_registrants_one_scanner_one_device) {
  constexpr int kThreads = 8, kPerThread = 500, kSlots = 64;
  Table t(kSlots, HostWords(kSlots));
  std::mutex q_mu;
  std::deque<cutile::SlotTicket> device_queue;  // stream writes in flight
  std::atomic<bool> stop{false};
  std::atomic<int> woken_total{0};
  std::vector<std::atomic<int>> per_payload(kThreads * kPerThread);
  for (auto& p : per_payload) p.store(0);
  std::thread device([&] {
    while (!stop.load() || !device_queue.empty()) {
      cutile::SlotTicket w{SIZE_MAX, 0};
      {
        std::lock_guard<std::mutex> lock(q_mu);
        if (!device_queue.empty()) { w = device_queue.front(); device_queue.pop_front(); }
      }
      if (w.slot == SIZE_MAX) { std::this_thread::yield(); continue; }
      t.words().word(w.slot).store(w.stamp, std::memory_order_release);
    }
  });
  std::thread scanner([&] {
    std::vector<int> woken;
    while (woken_total.load() < kThreads * kPerThread) {
      t.sweep(woken);
      for (int w : woken) { per_payload[w].fetch_add(1); woken_total.fetch_add(1); }
      woken.clear();
      std::this_thread::yield();
    }
  });
  std::vector<std::thread> regs;
  for (int th = 0; th < kThreads; ++th)
    regs.emplace_back([&, th] {
      for (int i = 0; i < kPerThread; ++i) {
        std::optional<cutile::SlotTicket> s;
        while (!(s = t.acquire())) std::this_thread::yield();  // all slots in use: wait for completions
        {
          std::lock_guard<std::mutex> lock(q_mu);
          device_queue.push_back(*s);  // the device may store the stamp before arm(): the protocol allows that
        }
        t.arm(*s, th * kPerThread + i);
      }
    });
  for (auto& r : regs) r.join();
  scanner.join();
  stop.store(true);
  device.join();
  for (auto& p : per_payload) CHECK(p.load() == 1);  // every waker fired exactly once
  CHECK(t.nothing_pending());
  size_t free_slots = 0;
  while (t.acquire()) ++free_slots;
  CHECK(free_slots == kSlots);  // nothing leaked
}

int main(int argc, char** argv) { return run_all_tests(argc, argv); }
