// Host-visible latency of an N-kernel pipeline under the four execution modes of the host surface, the measurement of
// cutile-benchmarks/paper/sec5_exp2_execution_mode_overhead/launch_overhead_rust/src/main.rs:
//   sync-individual   N separate .sync_on(): the host blocks between kernels
//   sync-chained      .sync_on() of one dependent chain of N launches (a boxed op per launch, built outside the timer)
//   async             the same chain as a DeviceFuture, waited for through the reactor (the reference's .await)
//   graph             the chain captured once, replayed with graph.launch().sync_on()
// The pipeline is N dependent launches of one small kernel on a single buffer of d = 2048 f16 values (the reference's
// k_scale, y = x * g; here the library's f16 saxpy, y = a x + y, which rewrites its buffer the same way).  Per
// configuration: fixed warm-up, then samples of `iters` pipelines each; the median per-pipeline wall time is reported.
//     launch_overhead [--n-list 1,1000] [--samples 50]      -> one JSON object on stdout
#include <cutile/cutile.hpp>

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

using namespace cutile;
using Part = Partition<Tensor<f16>>;
using Input = std::shared_ptr<Tensor<f16>>;
using Clock = std::chrono::steady_clock;

namespace {
constexpr int kD = 2048;

double seconds(Clock::time_point a, Clock::time_point b) { return std::chrono::duration<double>(b - a).count(); }

BoxedDeviceOp<Part> build_chain(Part part, int n, const Input& x) {
  BoxedDeviceOp<Part> chain = saxpy(std::move(part), 1.0f, x).first().boxed();
  for (int i = 1; i < n; ++i) chain = saxpy(std::move(chain), 1.0f, x).first().boxed();
  return chain;
}

struct Summary { double median, min, p25, p75, max; };
Summary summarize(std::vector<double> s) {
  std::sort(s.begin(), s.end());
  auto q = [&](double f) { return s[(size_t)std::llround((s.size() - 1) * f)]; };
  return {s[s.size() / 2], s.front(), q(0.25), q(0.75), s.back()};
}
}  // namespace

int main(int argc, char** argv) {
  std::vector<int> n_list = {1, 1000};
  int n_samples = 50;
  for (int i = 1; i + 1 < argc; ++i) {
    if (!strcmp(argv[i], "--samples")) n_samples = atoi(argv[i + 1]);
    if (!strcmp(argv[i], "--n-list")) {
      n_list.clear();
      for (char* tok = strtok(argv[i + 1], ","); tok; tok = strtok(nullptr, ",")) n_list.push_back(atoi(tok));
    }
  }
  auto stream = Device::create(0).unwrap()->new_stream().unwrap();
  Input x = std::make_shared<Tensor<f16>>(api::ones<f16>({kD}).sync_on(stream).unwrap());
  auto fresh = [&] { return api::zeros<f16>({kD}).sync_on(stream).unwrap().partition({kD}); };
  std::string json = "{\"kernel\": \"saxpy f16, d = 2048, one tile\", \"unit\": \"us per pipeline (median of samples)\", \"samples\": " + std::to_string(n_samples) + ", \"modes\": {";
  bool first_mode = true;
  auto emit = [&](const char* mode, int n, const Summary& s) {
    char buf[256];
    snprintf(buf, sizeof(buf), "%s\"%s/n=%d\": {\"median_us\": %.3f, \"min_us\": %.3f, \"p25_us\": %.3f, \"p75_us\": %.3f, \"max_us\": %.3f}", first_mode ? "" : ", ", mode, n,
             s.median * 1e6, s.min * 1e6, s.p25 * 1e6, s.p75 * 1e6, s.max * 1e6);
    json += buf;
    first_mode = false;
  };
  for (int n : n_list) {
    const int warmup = n >= 100 ? 5 : 200, iters = n >= 100 ? 3 : 200;
    {   // sync-individual
      Part part = fresh();
      auto run = [&](Part p) {
        for (int i = 0; i < n; ++i) p = std::move(std::get<0>(saxpy(std::move(p), 1.0f, x).sync_on(stream).unwrap()));
        return p;
      };
      for (int i = 0; i < warmup; ++i) part = run(std::move(part));
      std::vector<double> samples;
      for (int s = 0; s < n_samples; ++s) {
        stream->synchronize().unwrap();
        auto t0 = Clock::now();
        for (int i = 0; i < iters; ++i) part = run(std::move(part));
        samples.push_back(seconds(t0, Clock::now()) / iters);
      }
      emit("sync-individual", n, summarize(samples));
    }
    {   // sync-chained: chain construction outside the timer, its execute walk (one launcher per kernel) inside
      Part part = fresh();
      for (int i = 0; i < warmup; ++i) part = build_chain(std::move(part), n, x).sync_on(stream).unwrap();
      std::vector<double> samples;
      for (int s = 0; s < n_samples; ++s) {
        stream->synchronize().unwrap();
        double elapsed = 0;
        for (int i = 0; i < iters; ++i) {
          auto chain = build_chain(std::move(part), n, x);
          auto t0 = Clock::now();
          part = std::move(chain).sync_on(stream).unwrap();
          elapsed += seconds(t0, Clock::now());
        }
        samples.push_back(elapsed / iters);
      }
      emit("sync-chained", n, summarize(samples));
    }
    {   // async: the chain as a future, completion through the reactor
      Part part = fresh();
      for (int i = 0; i < warmup; ++i) part = build_chain(std::move(part), n, x).schedule_on(stream).block_on().unwrap();
      std::vector<double> samples;
      for (int s = 0; s < n_samples; ++s) {
        stream->synchronize().unwrap();
        double elapsed = 0;
        for (int i = 0; i < iters; ++i) {
          auto chain = build_chain(std::move(part), n, x);
          auto t0 = Clock::now();
          part = std::move(chain).schedule_on(stream).block_on().unwrap();
          elapsed += seconds(t0, Clock::now());
        }
        samples.push_back(elapsed / iters);
      }
      emit("async", n, summarize(samples));
    }
    {   // graph: captured once, replayed
      auto graph = HipGraph<Part>::capture(stream, build_chain(fresh(), n, x)).unwrap();
      for (int i = 0; i < warmup; ++i) graph.launch().sync_on(stream).unwrap();
      std::vector<double> samples;
      for (int s = 0; s < n_samples; ++s) {
        stream->synchronize().unwrap();
        auto t0 = Clock::now();
        for (int i = 0; i < iters; ++i) graph.launch().sync_on(stream).unwrap();
        samples.push_back(seconds(t0, Clock::now()) / iters);
      }
      emit("graph", n, summarize(samples));
    }
  }
  json += "}}";
  puts(json.c_str());
  return 0;
}
