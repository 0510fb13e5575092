// Tunes the variant choice of the benchmark configurations on the GPU this runs on and writes one provenance-checked
// record per kernel (cutile/src/tune.rs:293-420 Autotuner, :762-906 Record):
//
//     cutile-rs_amd/bin/tune_baseline <output directory>      (normally cutile-rs_amd/tuned)
//
// For every configuration: the candidates are all precompiled variants of the kernel; a candidate that does not fit
// the arguments is recorded as invalid by the tuner; the rest are timed with the do_bench protocol (cache flushed
// before every repetition, median); the winner is filed under the shape class the launcher reports for the launch
// (cutile_last_resolved_bucket) with the variant's fingerprint as its key.  The library applies the records it can
// verify on start-up (csrc/host/tuning.cpp).
#include <cutile/cutile.hpp>

#include <cmath>
#include <cstdio>
#include <map>

using namespace cutile;

namespace {

std::shared_ptr<Stream> g_stream;
std::map<std::string, tune::Record> g_records;

template <class T>
std::shared_ptr<Tensor<T>> converted(Tensor<float> t, std::vector<int32_t> shape) {
  auto arc = std::make_shared<Tensor<float>>(std::move(t));
  return std::make_shared<Tensor<T>>(std::move(api::convert<T>(arc).sync_on(g_stream).unwrap()).reshape(std::move(shape)).unwrap());
}

// `launch(variant, stream)` enqueues one launch with the named variant ("" = the library's own choice).
bool tune_one(const std::string& kernel, const std::string& what, const std::function<Result<Unit>(const std::string&, const std::shared_ptr<Stream>&)>& launch) {
  // every precompiled variant except the any-layout fallbacks (never the answer for a shape a tiled variant fits)
  std::vector<tune::Config> configs;
  for (auto& c : tune::variant_configs(kernel))
    if (c.str("variant")->find("generic") == std::string::npos) configs.push_back(c);
  printf("tuning %s  %s: %zu candidates\n", kernel.c_str(), what.c_str(), configs.size());
  bench::BenchOptions bo;
  bo.warmup = std::chrono::milliseconds(20);
  bo.rep = std::chrono::milliseconds(150);
  bo.min_reps = 10;
  bo.clear_bytes_override = 512u << 20;
  auto tuned = tune::Autotuner(kernel + ":" + what).configs(configs).bench_options(bo).run(
      g_stream, [&](const std::shared_ptr<Stream>& s, const tune::Config& c) -> Result<bench::BenchFn> {
        const std::string v = *c.str("variant");
        auto probe = launch(v, s);                       // a variant that does not fit these arguments is an invalid candidate
        if (probe.is_err()) return probe.error();
        if (auto e = s->synchronize(); e.is_err()) return e.error();
        return bench::BenchFn([&launch, v](const std::shared_ptr<Stream>& st) -> Result<Unit> { return launch(v, st); });
      });
  if (tuned.is_err() || !tuned.value().best) {
    fprintf(stderr, "tune %s (%s): no winner: %s\n", kernel.c_str(), what.c_str(), tuned.is_err() ? tuned.error().message.c_str() : "every candidate invalid");
    return false;
  }
  const tune::Output& out = tuned.value();
  const std::string best = *out.best->str("variant");
  // the class this launch belongs to, as the launcher files it
  if (launch("", g_stream).is_err() || g_stream->synchronize().is_err()) return false;
  const std::string bucket = cutile_last_resolved_bucket();
  if (bucket.empty()) { fprintf(stderr, "tune %s: launcher reports no shape class\n", kernel.c_str()); return false; }
  float best_ms = INFINITY;
  size_t reps = 0;
  printf("%s  %s  [%s]\n", kernel.c_str(), what.c_str(), bucket.c_str());
  for (auto& t : out.trials) {
    std::string name;
    for (auto& c : configs) if (c.id == t.config_id) name = *c.str("variant");
    if (t.measured) printf("    %-40s median %8.4f ms  min %8.4f ms  (%zu reps)%s\n", name.c_str(), t.median_ms, t.min_ms, t.reps, name == best ? "   <- winner" : "");
    if (t.measured && t.config_id == out.best->id && t.median_ms < best_ms) { best_ms = t.median_ms; reps = t.reps; }
  }
  auto it = g_records.find(kernel);
  if (it == g_records.end()) {
    auto ws = tune::Workspace::of_kernel(kernel, tune::space_hash(configs)).unwrap();
    it = g_records.emplace(kernel, tune::Record(ws)).first;
    it->second.gate = "do_bench median, 512 MiB flush, N(0,1) operands";
  }
  it->second.insert({bucket, *out.best, best_ms, reps, tune::variant_key(kernel, best).unwrap()});
  return true;
}

// Tile shape AND variant for one GEMM problem: the candidates are all (tile, variant) pairs of the precompiled tiled
// kernels (the reference's benchmark picks its tile by problem size, cutile-benchmarks/benches/gemm.rs:104-111).  The
// tile of a launch is the caller's partition, so this winner is a record for callers: it is filed in the kernel's
// record under the bucket "problem|<what>" with the parameters (variant, bm, bn); bench.py partitions z accordingly.
bool tune_tiles(const std::string& kernel, const std::string& what, const std::string& dtype,
                const std::function<Result<Unit>(int, int, const std::string&, const std::shared_ptr<Stream>&)>& launch) {
  std::vector<tune::Config> configs;
  for (auto& c : tune::variant_configs(kernel)) {
    const std::string v = *c.str("variant");
    int bm = 0, bn = 0, bk = 0;
    char kind[16] = {0};
    if (v.rfind(dtype + "_", 0) != 0 || sscanf(v.c_str() + dtype.size() + 1, "%dx%dx%d_%15s", &bm, &bn, &bk, kind) != 4) continue;
    configs.push_back(tune::Config::make({{"variant", tune::ParamValue(v)}, {"bm", tune::ParamValue(bm)}, {"bn", tune::ParamValue(bn)}}));
  }
  printf("tuning %s  %s: %zu (tile, variant) candidates\n", kernel.c_str(), what.c_str(), configs.size());
  bench::BenchOptions bo;
  bo.warmup = std::chrono::milliseconds(20);
  bo.rep = std::chrono::milliseconds(100);
  bo.min_reps = 10;
  bo.clear_bytes_override = 512u << 20;
  auto tuned = tune::Autotuner(kernel + ":tiles:" + what).configs(configs).bench_options(bo).run(
      g_stream, [&](const std::shared_ptr<Stream>& s, const tune::Config& c) -> Result<bench::BenchFn> {
        const std::string v = *c.str("variant");
        const int bm = (int)*c.integer("bm"), bn = (int)*c.integer("bn");
        auto probe = launch(bm, bn, v, s);
        if (probe.is_err()) return probe.error();
        if (auto e = s->synchronize(); e.is_err()) return e.error();
        return bench::BenchFn([&launch, v, bm, bn](const std::shared_ptr<Stream>& st) -> Result<Unit> { return launch(bm, bn, v, st); });
      });
  if (tuned.is_err() || !tuned.value().best) {
    fprintf(stderr, "tune %s tiles (%s): no winner\n", kernel.c_str(), what.c_str());
    return false;
  }
  const tune::Output& out = tuned.value();
  const std::string best = *out.best->str("variant");
  float best_ms = INFINITY;
  size_t reps = 0;
  for (auto& t : out.trials) {
    std::string name;
    for (auto& c : configs) if (c.id == t.config_id) name = *c.str("variant");
    if (t.measured) printf("    %-40s median %8.4f ms  min %8.4f ms  (%zu reps)%s\n", name.c_str(), t.median_ms, t.min_ms, t.reps, name == best ? "   <- winner" : "");
    if (t.measured && t.config_id == out.best->id && t.median_ms < best_ms) { best_ms = t.median_ms; reps = t.reps; }
  }
  auto it = g_records.find(kernel);
  if (it == g_records.end()) {
    auto ws = tune::Workspace::of_kernel(kernel, tune::space_hash(configs)).unwrap();
    it = g_records.emplace(kernel, tune::Record(ws)).first;
    it->second.gate = "do_bench median, 512 MiB flush, N(0,1) operands";
  }
  it->second.insert({"problem|" + what, *out.best, best_ms, reps, tune::variant_key(kernel, best).unwrap()});
  return true;
}

template <class L>
Result<Unit> enqueue(L launcher, const std::string& variant, const std::shared_ptr<Stream>& s) {
  auto r = variant.empty() ? std::move(launcher).async_on(s) : std::move(launcher).variant(variant).async_on(s);
  return r.is_err() ? Result<Unit>(r.error()) : ok();
}

}  // namespace

int main(int argc, char** argv) {
  if (argc < 2) { fprintf(stderr, "usage: %s <output directory>\n", argv[0]); return 2; }
  setvbuf(stdout, nullptr, _IOLBF, 0);
  const std::string out_dir = argv[1];
  cutile_tuning_reload("");                              // tune against the table's own order, not against older records
  g_stream = Device::create(0).unwrap()->new_stream().unwrap();
  bool all = true;

  for (int s : {4096, 8192}) {   // GEMM bf16, z += x y, 256 x 256 tiles
    auto x = converted<bf16>(api::randn(0.0f, 1.0f / std::sqrt((float)s), {s * s}, 5).sync_on(g_stream).unwrap(), {s, s});
    auto y = converted<bf16>(api::randn(0.0f, 1.0f / std::sqrt((float)s), {s * s}, 6).sync_on(g_stream).unwrap(), {s, s});
    auto z = api::zeros<bf16>({s, s}).sync_on(g_stream).unwrap();
    all &= tune_one("gemm", "bf16 M=N=K=" + std::to_string(s), [&](const std::string& v, const std::shared_ptr<Stream>& st) {
      return enqueue(gemm(z.partition_mut({256, 256}), x, y, s), v, st);
    });
    all &= tune_tiles("gemm", "bf16|" + std::to_string(s) + "x" + std::to_string(s) + "x" + std::to_string(s), "bf16",
                      [&](int bm, int bn, const std::string& v, const std::shared_ptr<Stream>& st) {
                        return enqueue(gemm(z.partition_mut({bm, bn}), x, y, s), v, st);
                      });
  }
  {   // GEMM f16 at 8192^3 (the operand type of the reference's own published GEMM figure)
    const int s = 8192;
    auto x = converted<f16>(api::randn(0.0f, 1.0f / std::sqrt((float)s), {s * s}, 5).sync_on(g_stream).unwrap(), {s, s});
    auto y = converted<f16>(api::randn(0.0f, 1.0f / std::sqrt((float)s), {s * s}, 6).sync_on(g_stream).unwrap(), {s, s});
    auto z = api::zeros<f16>({s, s}).sync_on(g_stream).unwrap();
    all &= tune_one("gemm", "f16 M=N=K=8192", [&](const std::string& v, const std::shared_ptr<Stream>& st) {
      return enqueue(gemm(z.partition_mut({256, 256}), x, y, s), v, st);
    });
  }
  {   // FMHA bf16 b4 h32 s4096 d128
    const int b = 4, h = 32, s = 4096, d = 128;
    auto mk = [&](uint64_t seed) { return converted<bf16>(api::randn(0.0f, 1.0f, {b * h * s * d}, seed).sync_on(g_stream).unwrap(), {b, h, s, d}); };
    auto q = mk(8), k = mk(9), v = mk(10);
    auto o = api::zeros<bf16>({b * h, s, d}).sync_on(g_stream).unwrap();
    all &= tune_one("fmha", "bf16 b4 h32 s4096 d128 non-causal", [&](const std::string& var, const std::shared_ptr<Stream>& st) {
      return enqueue(fmha(o.partition_mut({1, 256, d}), q, k, v, 1.0f / std::sqrt((float)d), 0, 1), var, st);
    });
    all &= tune_one("fmha", "bf16 b4 h32 s4096 d128 causal", [&](const std::string& var, const std::shared_ptr<Stream>& st) {
      return enqueue(fmha_causal(o.partition_mut({1, 256, d}), q, k, v, 1.0f / std::sqrt((float)d), 0, 1), var, st);
    });
  }
  {   // RMSNorm and row softmax f16 [16384, 8192]
    const int rows = 16384, n = 8192;
    auto x = converted<f16>(api::randn(0.0f, 1.0f, {rows * n}, 3).sync_on(g_stream).unwrap(), {rows, n});
    auto w = converted<f16>(api::rand<float>({n}, 4).sync_on(g_stream).unwrap(), {n});
    auto o = api::zeros<f16>({rows, n}).sync_on(g_stream).unwrap();
    all &= tune_one("rms_norm_f16", "f16 [16384, 8192]", [&](const std::string& v, const std::shared_ptr<Stream>& st) {
      return enqueue(rms_norm_f16(x, w, o.partition_mut({1, n}), 1e-6f), v, st);
    });
    all &= tune_one("softmax", "f16 [16384, 8192] rows", [&](const std::string& v, const std::shared_ptr<Stream>& st) {
      return enqueue(softmax(x, o.partition_mut({1, n})), v, st);
    });
  }
  {   // axpy f32, n = 2^24, tiles of 1024
    const int n = 1 << 24;
    auto x = std::make_shared<Tensor<float>>(api::rand<float>({n}, 1).sync_on(g_stream).unwrap());
    auto y = std::make_shared<Tensor<float>>(api::rand<float>({n}, 2).sync_on(g_stream).unwrap());
    auto z = api::zeros<float>({n}).sync_on(g_stream).unwrap();
    all &= tune_one("axpy", "f32 n=16777216", [&](const std::string& v, const std::shared_ptr<Stream>& st) {
      return enqueue(axpy(z.partition_mut({1024}), 2.0f, x, y), v, st);
    });
  }
  {   // MX fp8 GEMM 8192^3, bf16 out, 256 x 256 tiles: operand bytes with exponents near 1 and unit scales
    const int s = 8192;
    auto bytes = [&](uint8_t lo, uint8_t span, int n, std::vector<int32_t> shape, uint64_t seed) {
      auto host = std::make_shared<std::vector<uint8_t>>(n);
      uint64_t st = seed;
      for (auto& b : *host) { st = st * 6364136223846793005ull + 1442695040888963407ull; b = (uint8_t)(lo + (st >> 33) % span) | (uint8_t)(((st >> 20) & 1) << 7); }
      return std::make_shared<Tensor<uint8_t>>(std::move(api::copy_host_vec_to_device(host).sync_on(g_stream).unwrap()).reshape(std::move(shape)).unwrap());
    };
    auto x = Tensor<uint8_t>::reinterpret<f8e4m3fn>(bytes(0x28, 0x20, s * s, {s, s}, 12), {s, s}).unwrap();
    auto y = Tensor<uint8_t>::reinterpret<f8e4m3fn>(bytes(0x28, 0x20, s * s, {s, s}, 13), {s, s}).unwrap();
    auto xs = Tensor<uint8_t>::reinterpret<f8e8m0fnu>(bytes(0x7c, 6, s * s / 32, {s, s / 32}, 14), {s, s / 32}).unwrap();
    auto ys = Tensor<uint8_t>::reinterpret<f8e8m0fnu>(bytes(0x7c, 6, s * s / 32, {s, s / 32}, 15), {s, s / 32}).unwrap();
    for (auto* t : {&xs, &ys}) (void)t;
    auto z = api::zeros<bf16>({s, s}).sync_on(g_stream).unwrap();
    all &= tune_one("linear_tile", "mxfp8 8192^3 -> bf16", [&](const std::string& v, const std::shared_ptr<Stream>& st) {
      return enqueue(linear_tile(z.partition_mut({256, 256}), x, y, xs, ys, 1.0f), v, st);
    });
  }
  for (auto& [kernel, record] : g_records) {
    const std::string path = out_dir + "/" + kernel + ".json";
    if (record.save(path).is_err()) { fprintf(stderr, "cannot write %s\n", path.c_str()); all = false; }
    else printf("wrote %s (%zu buckets)\n", path.c_str(), record.entries.size());
  }
  return all ? 0 : 1;
}
