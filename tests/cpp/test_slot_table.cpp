// The reactor's slot protocol under plain atomics standing in for pinned memory,
// with a modelled "GPU" thread that completes slots — the CPU-side counterpart of
// cuda-async/src/slot_table.rs:169-330 (MockFlags, std-thread stress 8 x 500).
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

struct MockFlags {
  std::shared_ptr<std::vector<std::atomic<uint32_t>>> cells;
  explicit MockFlags(size_t n) : cells(std::make_shared<std::vector<std::atomic<uint32_t>>>(n)) {}
  std::atomic<uint32_t>& flag(size_t slot) { return (*cells)[slot]; }
};

TEST(claim_publish_scan_recycle) {
  SlotTable<int, MockFlags> t(4, MockFlags(4));
  CHECK(t.is_idle());
  auto s = t.claim();
  CHECK(s && *s == 0);  // lowest index first
  t.reset_flag(*s);
  CHECK(t.publish(*s, 42));        // idle -> active transition reported
  auto s2 = t.claim();
  t.reset_flag(*s2);
  CHECK(!t.publish(*s2, 43));      // already active
  std::vector<int> woken;
  CHECK(t.scan_once(woken) && woken.empty() && t.armed() == 2);  // armed, not complete: nothing retires
  t.flags().flag(*s2).store(1);
  CHECK(t.scan_once(woken) && woken == std::vector<int>({43}) && t.armed() == 1);
  t.flags().flag(*s).store(1);
  woken.clear();
  t.scan_once(woken);
  CHECK(woken == std::vector<int>({42}) && t.is_idle());
  CHECK(!t.scan_once(woken));       // nothing armed any more
  // exhaustion and release
  std::vector<size_t> held;
  while (auto c = t.claim()) held.push_back(*c);
  CHECK(held.size() == 4 && !t.claim());
  t.release(held.back());
  CHECK(t.claim().has_value());
}

TEST(stale_flag_cannot_complete_a_reused_slot) {
  SlotTable<int, MockFlags> t(1, MockFlags(1));
  std::vector<int> woken;
  auto s = *t.claim();
  t.reset_flag(s);
  t.publish(s, 1);
  t.flags().flag(s).store(1);
  t.scan_once(woken);
  CHECK(woken.size() == 1);
  // the flag still reads 1 from the first use; reset_flag runs before the slot is armed again
  s = *t.claim();
  t.reset_flag(s);
  t.publish(s, 2);
  woken.clear();
  t.scan_once(woken);
  CHECK(woken.empty() && t.armed() == 1);
}

TEST(stress_eight_registrants_one_scanner_one_device) {
  constexpr int kThreads = 8, kPerThread = 500, kSlots = 64;
  SlotTable<int, MockFlags> t(kSlots, MockFlags(kSlots));
  std::mutex q_mu;
  std::deque<size_t> device_queue;  // slots whose "stream write" is in flight
  std::atomic<bool> stop{false};
  std::atomic<int> woken_total{0};
  std::vector<std::atomic<int>> per_payload(kThreads * kPerThread);
  for (auto& p : per_payload) p.store(0);
  std::thread device([&] {
    while (!stop.load() || !device_queue.empty()) {
      size_t slot = SIZE_MAX;
      {
        std::lock_guard<std::mutex> lock(q_mu);
        if (!device_queue.empty()) { slot = device_queue.front(); device_queue.pop_front(); }
      }
      if (slot == SIZE_MAX) { std::this_thread::yield(); continue; }
      t.flags().flag(slot).store(1, std::memory_order_release);
    }
  });
  std::thread scanner([&] {
    std::vector<int> woken;
    while (woken_total.load() < kThreads * kPerThread) {
      t.scan_once(woken);
      for (int w : woken) { per_payload[w].fetch_add(1); woken_total.fetch_add(1); }
      woken.clear();
      std::this_thread::yield();
    }
  });
  std::vector<std::thread> regs;
  for (int th = 0; th < kThreads; ++th)
    regs.emplace_back([&, th] {
      for (int i = 0; i < kPerThread; ++i) {
        std::optional<size_t> s;
        while (!(s = t.claim())) std::this_thread::yield();  // pool exhausted: wait for retirements
        t.reset_flag(*s);
        {
          std::lock_guard<std::mutex> lock(q_mu);
          device_queue.push_back(*s);  // the device may complete it before publish: the protocol allows that
        }
        t.publish(*s, th * kPerThread + i);
      }
    });
  for (auto& r : regs) r.join();
  scanner.join();
  stop.store(true);
  device.join();
  for (auto& p : per_payload) CHECK(p.load() == 1);  // every waker fired exactly once
  CHECK(t.is_idle());
  size_t free_slots = 0;
  while (t.claim()) ++free_slots;
  CHECK(free_slots == kSlots);  // nothing leaked
}

int main(int argc, char** argv) { return run_all_tests(argc, argv); }
