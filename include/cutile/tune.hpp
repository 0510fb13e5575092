// A small autotuner over kernel variants and tile shapes.
//
// Mirrors the core of cutile/src/tune.rs: Config :53-123, space_hash :126-140,
// Trial / TrialState :145-177 (an invalid candidate is data, not an error),
// Oracle / Searcher / GridSearch with resume :180-253, best_config :255-290,
// Autotuner with prune / budget / JSONL trial log and a paired runoff between the
// two best candidates :293-470.  The winner is applied with
// cutile_kernel_set_preferred_variant, which the launchers consult.
#pragma once
#include <cstdio>
#include <fstream>
#include <map>
#include <set>
#include <sstream>

#include "bench.hpp"

namespace cutile {
namespace tune {

struct Config {
  std::string id;                                // stable identity, e.g. "variant=bf16_256x256x64_d2x4"
  std::map<std::string, std::string> params;     // ordered: the id is derived from it
  static Config make(std::map<std::string, std::string> params) {
    Config c;
    c.params = std::move(params);
    for (auto& kv : c.params) c.id += (c.id.empty() ? "" : ",") + kv.first + "=" + kv.second;
    return c;
  }
  std::optional<int64_t> integer(const std::string& k) const {
    auto it = params.find(k);
    if (it == params.end()) return std::nullopt;
    try { return std::stoll(it->second); } catch (...) { return std::nullopt; }
  }
  std::optional<std::string> str(const std::string& k) const {
    auto it = params.find(k);
    if (it == params.end()) return std::nullopt;
    return it->second;
  }
};

// Order-independent hash of the candidate set: a resumed log is only trusted for
// the space it was written for.
inline std::string space_hash(const std::vector<Config>& configs) {
  std::set<std::string> ids;
  for (auto& c : configs) ids.insert(c.id);
  uint64_t h = 1469598103934665603ull;  // FNV-1a
  for (auto& id : ids) {
    for (unsigned char ch : id) { h ^= ch; h *= 1099511628211ull; }
    h ^= 0xff; h *= 1099511628211ull;
  }
  char buf[17];
  snprintf(buf, sizeof(buf), "%016llx", (unsigned long long)h);
  return buf;
}

struct Trial {
  std::string config_id;
  bool measured = false;
  float median_ms = 0, min_ms = 0;
  size_t reps = 0;
  std::string invalid_reason;
  static Trial ok(std::string id, float median, float mn, size_t reps) { Trial t; t.config_id = std::move(id); t.measured = true; t.median_ms = median; t.min_ms = mn; t.reps = reps; return t; }
  static Trial invalid(std::string id, std::string why) { Trial t; t.config_id = std::move(id); t.invalid_reason = std::move(why); return t; }
  std::optional<float> median() const { return measured ? std::optional<float>(median_ms) : std::nullopt; }
};

struct Oracle {
  virtual ~Oracle() = default;
  virtual const std::vector<Config>& configs() const = 0;
  virtual Trial measure(size_t index) = 0;
  virtual bool budget_exhausted() const = 0;
};

struct GridSearch {
  std::vector<Trial> known;
  GridSearch resume(std::vector<Trial> k) && { known = std::move(k); return std::move(*this); }
  // Resumed trials count only if their config is still in the space and they
  // measured; invalid ones are retried (they may have been transient).
  std::vector<Trial> search(Oracle& oracle) {
    std::set<std::string> current;
    for (auto& c : oracle.configs()) current.insert(c.id);
    std::vector<Trial> trials;
    std::set<std::string> visited;
    for (auto& t : known)
      if (current.count(t.config_id) && t.measured) { trials.push_back(t); visited.insert(t.config_id); }
    known.clear();
    for (size_t i = 0; i < oracle.configs().size(); ++i) {
      if (visited.count(oracle.configs()[i].id)) continue;
      if (oracle.budget_exhausted()) break;
      trials.push_back(oracle.measure(i));
    }
    return trials;
  }
};

inline const Config* best_config(const std::vector<Config>& configs, const std::vector<Trial>& trials) {
  const Config* best = nullptr;
  float best_ms = 0;
  for (auto& t : trials) {
    if (!t.measured || !std::isfinite(t.median_ms)) continue;
    const Config* c = nullptr;
    for (auto& cand : configs)
      if (cand.id == t.config_id) { c = &cand; break; }
    if (!c) continue;  // stale record: neither wins nor shadows
    if (!best || t.median_ms < best_ms) { best = c; best_ms = t.median_ms; }
  }
  return best;
}

struct Output {
  std::vector<Trial> trials;
  std::optional<Config> best;
};

// Append-only JSONL trial log, guarded by tuner name + space hash.
class TrialLog {
 public:
  TrialLog(std::string path, const std::string& name, const std::string& hash) : path_(std::move(path)) {
    if (path_.empty()) return;
    header_ = "{\"tuner\":\"" + name + "\",\"space\":\"" + hash + "\"}";
    std::ifstream in(path_);
    std::string line;
    bool match = false, first = true;
    while (std::getline(in, line)) {
      if (first) { match = line == header_; first = false; continue; }
      if (!match) break;
      Trial t;
      if (parse(line, &t)) existing_.push_back(t);
    }
    if (!match) {  // other tuner or other space: start over
      existing_.clear();
      std::ofstream out(path_, std::ios::trunc);
      out << header_ << "\n";
    }
  }
  const std::vector<Trial>& existing_trials() const { return existing_; }
  void append(const Trial& t) {
    if (path_.empty()) return;
    std::ofstream out(path_, std::ios::app);
    if (t.measured)
      out << "{\"config\":\"" << t.config_id << "\",\"median_ms\":" << t.median_ms << ",\"min_ms\":" << t.min_ms << ",\"reps\":" << t.reps << "}\n";
    else
      out << "{\"config\":\"" << t.config_id << "\",\"invalid\":\"" << t.invalid_reason << "\"}\n";
  }

 private:
  static bool field(const std::string& line, const std::string& key, std::string* out) {
    auto p = line.find("\"" + key + "\":");
    if (p == std::string::npos) return false;
    p += key.size() + 3;
    if (line[p] == '"') { auto e = line.find('"', p + 1); *out = line.substr(p + 1, e - p - 1); }
    else { auto e = line.find_first_of(",}", p); *out = line.substr(p, e - p); }
    return true;
  }
  static bool parse(const std::string& line, Trial* t) {
    std::string v;
    if (!field(line, "config", &t->config_id)) return false;
    if (field(line, "invalid", &v)) { t->invalid_reason = v; return true; }
    if (!field(line, "median_ms", &v)) return false;
    t->measured = true; t->median_ms = std::stof(v);
    if (field(line, "min_ms", &v)) t->min_ms = std::stof(v);
    if (field(line, "reps", &v)) t->reps = (size_t)std::stoul(v);
    return true;
  }
  std::string path_, header_;
  std::vector<Trial> existing_;
};

class Autotuner {
 public:
  using Setup = std::function<Result<bench::BenchFn>(const std::shared_ptr<Stream>&, const Config&)>;
  explicit Autotuner(std::string name) : name_(std::move(name)) {}
  Autotuner configs(std::vector<Config> c) && { configs_ = std::move(c); return std::move(*this); }
  Autotuner prune(std::function<bool(const Config&)> keep) && { prune_.push_back(std::move(keep)); return std::move(*this); }
  Autotuner budget(std::chrono::milliseconds b) && { budget_ = b; return std::move(*this); }
  Autotuner bench_options(bench::BenchOptions b) && { bench_ = b; return std::move(*this); }
  Autotuner log(std::string path) && { log_path_ = std::move(path); return std::move(*this); }

  // setup(stream, config) returns the closure to time, or an error: the candidate
  // is then recorded as invalid and the search goes on.
  Result<Output> run(const std::shared_ptr<Stream>& stream, Setup setup) && {
    std::vector<Config> kept;
    for (auto& c : configs_) {
      bool keep = true;
      for (auto& p : prune_) keep = keep && p(c);
      if (keep) kept.push_back(c);
    }
    TrialLog log(log_path_, name_, space_hash(kept));
    BenchOracle oracle{kept, stream, setup, bench_, budget_, std::chrono::steady_clock::now(), &log};
    std::vector<Trial> trials = GridSearch{}.resume(log.existing_trials()).search(oracle);
    // Paired runoff between the two best: sequential medians can be skewed by drift.
    std::vector<std::pair<float, const Config*>> ranked;
    for (auto& c : kept) {
      float best = INFINITY;
      for (auto& t : trials)
        if (t.config_id == c.id && t.measured && std::isfinite(t.median_ms)) best = std::min(best, t.median_ms);
      if (std::isfinite(best)) ranked.emplace_back(best, &c);
    }
    std::sort(ranked.begin(), ranked.end(), [](auto& a, auto& b) { return a.first < b.first; });
    Output out;
    if (ranked.empty()) { out.trials = std::move(trials); return out; }
    const Config* winner = ranked[0].second;
    if (ranked.size() > 1 && !oracle.budget_exhausted()) {
      const Config* a = ranked[0].second;
      const Config* b = ranked[1].second;
      auto fa = setup(stream, *a);
      auto fb = setup(stream, *b);
      if (fa.is_ok() && fb.is_ok()) {
        auto pair = bench::do_bench_paired(stream, bench_, fa.value(), fb.value());
        if (pair.is_ok()) {
          Trial ta = Trial::ok(a->id, pair.value().first.median_ms(), pair.value().first.min_ms(), pair.value().first.reps());
          Trial tb = Trial::ok(b->id, pair.value().second.median_ms(), pair.value().second.min_ms(), pair.value().second.reps());
          log.append(ta); log.append(tb);
          winner = tb.median_ms < ta.median_ms ? b : a;
          trials.push_back(ta); trials.push_back(tb);
        }
      }
    }
    out.best = *winner;
    out.trials = std::move(trials);
    return out;
  }

 private:
  struct BenchOracle : Oracle {
    std::vector<Config> cfgs;
    std::shared_ptr<Stream> stream;
    Setup setup;
    bench::BenchOptions bench;
    std::optional<std::chrono::milliseconds> budget;
    std::chrono::steady_clock::time_point start;
    TrialLog* log;
    BenchOracle(std::vector<Config> c, std::shared_ptr<Stream> s, Setup su, bench::BenchOptions b,
                std::optional<std::chrono::milliseconds> bu, std::chrono::steady_clock::time_point st, TrialLog* l)
        : cfgs(std::move(c)), stream(std::move(s)), setup(std::move(su)), bench(b), budget(bu), start(st), log(l) {}
    const std::vector<Config>& configs() const override { return cfgs; }
    bool budget_exhausted() const override { return budget && std::chrono::steady_clock::now() - start >= *budget; }
    Trial measure(size_t i) override {
      Trial t;
      auto f = setup(stream, cfgs[i]);
      if (f.is_err()) {
        t = Trial::invalid(cfgs[i].id, f.error().to_string());
      } else {
        auto m = bench::do_bench(stream, bench, f.value());
        t = m.is_err() ? Trial::invalid(cfgs[i].id, m.error().to_string())
                       : Trial::ok(cfgs[i].id, m.value().median_ms(), m.value().min_ms(), m.value().reps());
      }
      log->append(t);
      return t;
    }
  };
  std::string name_;
  std::vector<Config> configs_;
  std::vector<std::function<bool(const Config&)>> prune_;
  std::optional<std::chrono::milliseconds> budget_;
  bench::BenchOptions bench_;
  std::string log_path_;
};

// All precompiled variants of `function` as tuning candidates.
inline std::vector<Config> variant_configs(const std::string& function, const std::string& must_contain = "") {
  int n = cutile_kernel_list(nullptr, 0);
  std::vector<const char*> names(n);
  cutile_kernel_list(names.data(), n);
  std::vector<Config> out;
  for (const char* s : names) {
    std::string e = s;
    auto colon = e.find(':');
    if (e.substr(0, colon) != function) continue;
    std::string v = e.substr(colon + 1);
    if (!must_contain.empty() && v.find(must_contain) == std::string::npos) continue;
    out.push_back(Config::make({{"variant", v}}));
  }
  return out;
}

}  // namespace tune
}  // namespace cutile
