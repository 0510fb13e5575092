// Device-event benchmarking: do_bench / do_bench_paired.
//
// Mirrors cutile/src/bench.rs: BenchOptions :32-50, Measurement + quantiles
// :52-101, the cache-clearing buffer (2 x L2, clamped to 64..512 MiB) :124-160,
// time_one / do_bench / do_bench_paired :162-254.  The closure must enqueue its
// work on the stream it is given; work on other streams is not timed.
#pragma once
#include <algorithm>
#include <chrono>
#include <cmath>
#include <functional>

#include "runtime.hpp"

namespace cutile {
namespace bench {

struct BenchOptions {
  std::chrono::milliseconds warmup{25};
  std::chrono::milliseconds rep{100};
  size_t min_reps = 5;
  size_t max_reps = 1000;
  bool clear_l2 = true;
  // MI355X has a 256 MiB memory-side cache behind the per-XCD L2s; to take it out
  // of a measurement, raise the clear buffer above it (the default follows the
  // reference's 2 x L2 rule).
  size_t clear_bytes_override = 0;
};

class Measurement {
 public:
  explicit Measurement(std::vector<float> t) : times_ms_(std::move(t)) {}
  size_t reps() const { return times_ms_.size(); }
  const std::vector<float>& times_ms() const { return times_ms_; }
  float min_ms() const { return *std::min_element(times_ms_.begin(), times_ms_.end()); }
  float mean_ms() const {
    double s = 0;
    for (float t : times_ms_) s += t;
    return (float)(s / (double)times_ms_.size());
  }
  float median_ms() const { return quantile_ms(0.5f); }
  // Linear interpolation between order statistics; q is clamped to [0, 1].
  float quantile_ms(float q) const {
    std::vector<float> s = times_ms_;
    std::sort(s.begin(), s.end());
    q = std::min(1.0f, std::max(0.0f, q));
    float pos = q * (float)(s.size() - 1);
    size_t lo = (size_t)std::floor(pos), hi = (size_t)std::ceil(pos);
    if (lo == hi) return s[lo];
    float frac = pos - (float)lo;
    return s[lo] * (1.0f - frac) + s[hi] * frac;
  }

 private:
  std::vector<float> times_ms_;
};

class CacheClear {
 public:
  CacheClear(const std::shared_ptr<Stream>& stream, size_t override_bytes) : stream_(stream) {
    size_t l2 = stream->device()->l2_cache_size_bytes().is_ok() ? stream->device()->l2_cache_size_bytes().value() : 0;
    bytes_ = override_bytes ? override_bytes : std::min<size_t>(std::max<size_t>(l2 * 2, 64u << 20), 512u << 20);
    if (cutile_malloc_async(bytes_, stream->raw(), &ptr_) != CUTILE_SUCCESS) ptr_ = nullptr;
  }
  ~CacheClear() {
    if (ptr_) cutile_free_async(ptr_, stream_->raw());
  }
  Result<Unit> clear() { return ptr_ ? check(cutile_memset_d8_async(ptr_, 0, bytes_, stream_->raw())) : ok(); }
  size_t bytes() const { return bytes_; }

 private:
  std::shared_ptr<Stream> stream_;
  void* ptr_ = nullptr;
  size_t bytes_ = 0;
};

using BenchFn = std::function<Result<Unit>(const std::shared_ptr<Stream>&)>;

inline Result<float> time_one(const std::shared_ptr<Stream>& stream, const BenchFn& f) {
  auto start = Event::create();
  auto end = Event::create();
  if (start.is_err()) return start.error();
  if (end.is_err()) return end.error();
  CUTILE_TRY(start.value()->record(*stream));
  CUTILE_TRY(f(stream));
  CUTILE_TRY(end.value()->record(*stream));
  CUTILE_TRY(end.value()->synchronize());
  return start.value()->elapsed_ms(*end.value());
}

inline Result<Measurement> do_bench(const std::shared_ptr<Stream>& stream, const BenchOptions& opts, const BenchFn& f) {
  auto t0 = std::chrono::steady_clock::now();
  CUTILE_TRY(f(stream));  // at least one warm-up: absorbs the first-launch code-object load
  while (std::chrono::steady_clock::now() - t0 < opts.warmup) CUTILE_TRY(f(stream));
  auto est = time_one(stream, f);
  if (est.is_err()) return est.error();
  double est_ms = std::max<double>(est.value(), 1e-4);
  size_t reps = (size_t)std::llround((double)opts.rep.count() / est_ms);
  reps = std::min(opts.max_reps, std::max(opts.min_reps, reps));
  std::unique_ptr<CacheClear> clr;
  if (opts.clear_l2) clr = std::make_unique<CacheClear>(stream, opts.clear_bytes_override);
  std::vector<float> times;
  for (size_t i = 0; i < reps; ++i) {
    if (clr) CUTILE_TRY(clr->clear());
    auto t = time_one(stream, f);
    if (t.is_err()) return t.error();
    times.push_back(t.value());
  }
  return Measurement(std::move(times));
}

// Interleaved A/B measurement: drift hits both arms alike (bench.rs:213-254).
inline Result<std::pair<Measurement, Measurement>> do_bench_paired(const std::shared_ptr<Stream>& stream, const BenchOptions& opts,
                                                                   const BenchFn& a, const BenchFn& b) {
  auto t0 = std::chrono::steady_clock::now();
  CUTILE_TRY(a(stream));
  CUTILE_TRY(b(stream));
  while (std::chrono::steady_clock::now() - t0 < opts.warmup) {
    CUTILE_TRY(a(stream));
    CUTILE_TRY(b(stream));
  }
  auto est = time_one(stream, a);
  if (est.is_err()) return est.error();
  double est_ms = std::max<double>(est.value(), 1e-4);
  size_t reps = (size_t)std::llround((double)opts.rep.count() / est_ms / 2.0);
  reps = std::min(opts.max_reps, std::max(opts.min_reps, reps));
  std::unique_ptr<CacheClear> clr;
  if (opts.clear_l2) clr = std::make_unique<CacheClear>(stream, opts.clear_bytes_override);
  std::vector<float> ta, tb;
  for (size_t i = 0; i < reps; ++i) {
    if (clr) CUTILE_TRY(clr->clear());
    auto x = time_one(stream, a);
    if (x.is_err()) return x.error();
    ta.push_back(x.value());
    if (clr) CUTILE_TRY(clr->clear());
    auto y = time_one(stream, b);
    if (y.is_err()) return y.error();
    tb.push_back(y.value());
  }
  return std::make_pair(Measurement(std::move(ta)), Measurement(std::move(tb)));
}

}  // namespace bench
}  // namespace cutile
