// Autotuner over kernel variants and tile shapes, with resumable trial logs and
// provenance-checked records of winners.
//
// Mirrors cutile/src/tune.rs: Config / ParamValue :53-123, space_hash :126-140,
// Trial / TrialState :145-177 (an invalid candidate is data, not an error), Oracle /
// Searcher / GridSearch with resume :180-253, best_config :255-290, Autotuner with
// prune / budget / log and the paired runoff between the two best candidates
// :293-620, the JSONL trial log headed by (schema, tuner, space) :622-760, and Record /
// RecordEntry / Workspace with load_verified :762-1016.  File formats follow the
// reference's serde layout, so logs and records are interchangeable in both directions.
// What the reference takes from its JIT as provenance comes here from the ahead-of-time
// kernel table: source_hash = fingerprint of the code object that holds the kernel,
// l2 key = fingerprint of (code object, variant symbol), toolchain fingerprint = the
// device compiler's version text at build time, arch = gfx950.
// A winner reaches the launchers per shape class (cutile_kernel_set_preferred_variant_for, which is also how verified
// records are applied) or function-wide (cutile_kernel_set_preferred_variant, which takes precedence over records).
#pragma once
#include <cstdio>
#include <ctime>
#include <fstream>
#include <map>
#include <set>
#include <sstream>
#include <variant>

#include "bench.hpp"
#include "json.hpp"

namespace cutile {
namespace tune {

// ---- Config ------------------------------------------------------------------------------------
struct ParamValue {
  std::variant<int64_t, std::string> v;
  ParamValue(int64_t i) : v(i) {}
  ParamValue(int i) : v((int64_t)i) {}
  ParamValue(std::string s) : v(std::move(s)) {}
  ParamValue(const char* s) : v(std::string(s)) {}
  bool is_int() const { return v.index() == 0; }
  bool operator==(const ParamValue& o) const { return v == o.v; }
};

struct Config {
  std::string id;                             // derived from the parameters; logs and records key on it
  std::map<std::string, ParamValue> params;   // ordered: keys sorted

  // id = "k1=v1,k2=v2" over the sorted keys.  String values are JSON-quoted so that the int 1 and
  // the string "1" differ and a value holding ',' or '=' cannot pass for further parameters; keys
  // holding a separator or a quote are quoted the same way (tune.rs:73-104).
  static Config make(std::map<std::string, ParamValue> params) {
    Config c;
    c.params = std::move(params);
    for (auto& kv : c.params) {
      const std::string key = kv.first.find_first_of("=,\"") != std::string::npos ? json::quote(kv.first) : kv.first;
      c.id += (c.id.empty() ? "" : ",") + key + "=" +
              (kv.second.is_int() ? std::to_string(std::get<int64_t>(kv.second.v)) : json::quote(std::get<std::string>(kv.second.v)));
    }
    return c;
  }
  std::optional<int64_t> integer(const std::string& k) const {
    auto it = params.find(k);
    if (it == params.end() || !it->second.is_int()) return std::nullopt;
    return std::get<int64_t>(it->second.v);
  }
  std::optional<std::string> str(const std::string& k) const {
    auto it = params.find(k);
    if (it == params.end() || it->second.is_int()) return std::nullopt;
    return std::get<std::string>(it->second.v);
  }
  json::Value to_json() const {
    json::Value p = json::Value::object();
    for (auto& kv : params)
      p.set(kv.first, kv.second.is_int() ? json::Value::integer(std::get<int64_t>(kv.second.v)) : json::Value::string(std::get<std::string>(kv.second.v)));
    return json::Value::object().set("id", json::Value::string(id)).set("params", std::move(p));
  }
  static std::optional<Config> from_json(const json::Value& v) {
    const json::Value* id = v.get("id");
    const json::Value* params = v.get("params");
    if (!id || !id->is_string() || !params || !params->is_object()) return std::nullopt;
    Config c;
    c.id = id->s;   // kept as stored: load_verified compares it with the id the parameters derive
    for (auto& kv : params->fields) {
      if (kv.second.kind == json::Value::Kind::Int) c.params.emplace(kv.first, ParamValue(kv.second.i));
      else if (kv.second.is_string()) c.params.emplace(kv.first, ParamValue(kv.second.s));
      else return std::nullopt;
    }
    return c;
  }
};

// Order-independent fingerprint of a candidate set: FNV-1a over the sorted ids, each closed by
// a zero byte (tune.rs:126-140).  Logs and records carry it, so resuming or applying against
// another search space is detected instead of trusted.
inline std::string space_hash(const std::vector<Config>& configs) {
  std::vector<std::string> ids;
  for (auto& c : configs) ids.push_back(c.id);
  std::sort(ids.begin(), ids.end());
  uint64_t h = 0xcbf29ce484222325ull;
  for (auto& id : ids) {
    for (unsigned char ch : id) { h ^= ch; h *= 0x100000001b3ull; }
    h *= 0x100000001b3ull;   // the closing zero byte: h ^= 0 changes nothing
  }
  char buf[17];
  snprintf(buf, sizeof(buf), "%016llx", (unsigned long long)h);
  return buf;
}

// ---- Trial -------------------------------------------------------------------------------------
struct Trial {
  std::string config_id;
  bool measured = false;
  float median_ms = 0, min_ms = 0;
  size_t reps = 0;
  std::string invalid_reason;
  static Trial ok(std::string id, float median, float mn, size_t reps) { Trial t; t.config_id = std::move(id); t.measured = true; t.median_ms = median; t.min_ms = mn; t.reps = reps; return t; }
  static Trial invalid(std::string id, std::string why) { Trial t; t.config_id = std::move(id); t.invalid_reason = std::move(why); return t; }
  // no timed reps (BenchOptions with min_reps 0 and no budget) is an invalid trial, never a crash (tune.rs:618-631)
  static Trial from_measurement(std::string id, const bench::Measurement& m) {
    if (m.reps() == 0) return invalid(std::move(id), "no timed reps (check BenchOptions)");
    return ok(std::move(id), m.median_ms(), m.min_ms(), m.reps());
  }
  std::optional<float> median() const { return measured ? std::optional<float>(median_ms) : std::nullopt; }

  // {"config_id": .., "state": {"Measured": {"median_ms": .., "min_ms": .., "reps": ..}}}  or  {"Invalid": {"reason": ..}}
  json::Value to_json() const {
    json::Value state = json::Value::object();
    if (measured)
      state.set("Measured", json::Value::object().set("median_ms", json::Value::number(median_ms)).set("min_ms", json::Value::number(min_ms))
                                .set("reps", json::Value::integer((int64_t)reps)));
    else
      state.set("Invalid", json::Value::object().set("reason", json::Value::string(invalid_reason)));
    return json::Value::object().set("config_id", json::Value::string(config_id)).set("state", std::move(state));
  }
  static std::optional<Trial> from_json(const json::Value& v) {
    const json::Value* id = v.get("config_id");
    const json::Value* state = v.get("state");
    if (!id || !id->is_string() || !state || !state->is_object()) return std::nullopt;
    auto number = [](const json::Value* x) { return !x || x->is_null() ? NAN : (float)x->as_double(); };   // NaN is written as null
    if (const json::Value* m = state->get("Measured")) {
      const json::Value* reps = m->get("reps");
      if (!m->get("median_ms") || !m->get("min_ms") || !reps || !reps->is_number()) return std::nullopt;
      return ok(id->s, number(m->get("median_ms")), number(m->get("min_ms")), (size_t)reps->as_double());
    }
    if (const json::Value* bad = state->get("Invalid")) {
      const json::Value* reason = bad->get("reason");
      if (!reason || !reason->is_string()) return std::nullopt;
      return invalid(id->s, reason->s);
    }
    return std::nullopt;
  }
};

// ---- Oracle / Searcher ---------------------------------------------------------------------------
struct Oracle {
  virtual ~Oracle() = default;
  virtual const std::vector<Config>& configs() const = 0;          // pruned, in declaration order
  virtual Trial measure(size_t index) = 0;                        // never throws for a bad candidate
  virtual std::optional<std::chrono::nanoseconds> budget_remaining() const = 0;
  bool budget_exhausted() const { auto b = budget_remaining(); return b && b->count() <= 0; }
};

struct Searcher {
  virtual ~Searcher() = default;
  virtual std::vector<Trial> search(Oracle& oracle) = 0;          // every trial visited, in visit order
};

struct GridSearch : Searcher {
  std::vector<Trial> known;
  GridSearch resume(std::vector<Trial> k) && { known = std::move(k); return std::move(*this); }
  // Resumed trials count only if their config is still in the space and they measured;
  // invalid ones are retried: they may have been transient (tune.rs:226-251).
  std::vector<Trial> search(Oracle& oracle) override {
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

// The measured candidate with the lowest finite median; trials of configs that left the space
// neither win nor shadow a valid winner (tune.rs:255-290).
inline const Config* best_config(const std::vector<Config>& configs, const std::vector<Trial>& trials) {
  const Config* best = nullptr;
  float best_ms = 0;
  for (auto& t : trials) {
    if (!t.measured || !std::isfinite(t.median_ms)) continue;
    const Config* c = nullptr;
    for (auto& cand : configs)
      if (cand.id == t.config_id) { c = &cand; break; }
    if (!c) continue;
    if (!best || t.median_ms < best_ms) { best = c; best_ms = t.median_ms; }
  }
  return best;
}

// The two best measured candidates by their best median (runoff entries may repeat a config), tune.rs:459-487.
inline std::pair<const Config*, const Config*> top_two(const std::vector<Config>& configs, const std::vector<Trial>& trials) {
  std::vector<std::pair<const Config*, float>> ranked;
  for (auto& t : trials) {
    if (!t.measured || !std::isfinite(t.median_ms)) continue;
    for (auto& c : configs)
      if (c.id == t.config_id) {
        auto it = std::find_if(ranked.begin(), ranked.end(), [&](auto& r) { return r.first == &c; });
        if (it == ranked.end()) ranked.emplace_back(&c, t.median_ms);
        else it->second = std::min(it->second, t.median_ms);
        break;
      }
  }
  std::stable_sort(ranked.begin(), ranked.end(), [](auto& a, auto& b) { return a.second < b.second; });
  return {ranked.empty() ? nullptr : ranked[0].first, ranked.size() > 1 ? ranked[1].first : nullptr};
}

struct Output {
  std::vector<Trial> trials;
  std::optional<Config> best;
};

// ---- trial log -----------------------------------------------------------------------------------
// Append-only JSONL, first line {"log_schema":1,"tuner":..,"space":..}.  A log written by another
// tuner or for another space is REFUSED, not adopted and not overwritten; a missing, empty or
// whitespace-only file is fresh; a torn last line (crash mid-write) is dropped and the next record
// starts on a line of its own (tune.rs:648-760).
class TrialLog {
 public:
  static Result<TrialLog> open(const std::optional<std::string>& path, const std::string& tuner, const std::string& space) {
    TrialLog log;
    if (!path) return log;
    const std::string header = json::dump(json::Value::object().set("log_schema", json::Value::integer(1))
                                              .set("tuner", json::Value::string(tuner)).set("space", json::Value::string(space)));
    bool fresh = true, needs_newline = false;
    std::ifstream in(*path, std::ios::binary);
    if (in) {
      std::stringstream ss;
      ss << in.rdbuf();
      const std::string contents = ss.str();
      if (contents.find_first_not_of(" \t\r\n") != std::string::npos) {
        std::istringstream lines(contents);
        std::string line;
        std::getline(lines, line);
        auto head = json::parse(line);
        const json::Value* schema = head ? head->get("log_schema") : nullptr;
        const json::Value* t = head ? head->get("tuner") : nullptr;
        const json::Value* s = head ? head->get("space") : nullptr;
        if (!schema || !t || !s || !t->is_string() || !s->is_string())
          return DeviceError::tensor("trial log " + *path + " has no valid header; delete it or point .log() elsewhere");
        if (schema->kind != json::Value::Kind::Int || schema->i != 1 || t->s != tuner || s->s != space)
          return DeviceError::tensor("trial log " + *path + " belongs to tuner " + json::quote(t->s) + " (space " + s->s + "), not " +
                                     json::quote(tuner) + " (space " + space + "); delete it or point .log() elsewhere");
        while (std::getline(lines, line)) {
          auto v = json::parse(line);
          if (!v) continue;
          if (auto trial = Trial::from_json(*v)) log.existing_.push_back(*trial);
        }
        needs_newline = contents.back() != '\n';
        fresh = false;
      }
    }
    log.path_ = *path;
    std::ofstream out(*path, fresh ? std::ios::trunc : std::ios::app);
    if (!out) return DeviceError::tensor("trial log " + *path + " cannot be opened for append");
    if (needs_newline) out << "\n";
    if (fresh) out << header << "\n";
    return log;
  }
  const std::vector<Trial>& existing_trials() const { return existing_; }
  void append(const Trial& t) {   // best effort after a successful open
    if (path_.empty()) return;
    std::ofstream out(path_, std::ios::app);
    out << json::dump(t.to_json()) << "\n";
  }

 private:
  std::string path_;
  std::vector<Trial> existing_;
};

// ---- runoff ----------------------------------------------------------------------------------------
// Why a runoff gave no verdict: one finalist failed its own setup (it forfeits and is recorded
// invalid), or the paired measurement failed after both set up (nobody is blamed, the sequential
// leader stays) — tune.rs:553-616.
struct RunoffError {
  enum class Kind { SetupA, SetupB, Bench } kind;
  DeviceError error;
};
using RunoffResult = std::variant<std::pair<bench::Measurement, bench::Measurement>, RunoffError>;

// `a` is the sequential leader: it wins ties and unattributable failures; a non-finite median never wins.
inline Config runoff_verdict(const Config& a, const Config& b, const RunoffResult& result, std::vector<Trial>* trials, TrialLog* log) {
  if (auto* err = std::get_if<RunoffError>(&result)) {
    if (err->kind == RunoffError::Kind::Bench) return a;
    const bool b_failed = err->kind == RunoffError::Kind::SetupB;
    Trial t = Trial::invalid(b_failed ? b.id : a.id, "runoff setup failed: " + err->error.to_string());
    log->append(t);
    trials->push_back(t);
    return b_failed ? a : b;
  }
  auto& pair = std::get<0>(result);
  Trial ta = Trial::from_measurement(a.id, pair.first), tb = Trial::from_measurement(b.id, pair.second);
  for (Trial* t : {&ta, &tb}) { log->append(*t); trials->push_back(*t); }
  auto key = [](const Trial& t) { return t.measured && std::isfinite(t.median_ms) ? t.median_ms : INFINITY; };
  return key(ta) <= key(tb) ? a : b;
}

// ---- Autotuner -------------------------------------------------------------------------------------
class Autotuner {
 public:
  using Setup = std::function<Result<bench::BenchFn>(const std::shared_ptr<Stream>&, const Config&)>;
  explicit Autotuner(std::string name) : name_(std::move(name)) {}
  const std::string& name() const { return name_; }
  Autotuner configs(std::vector<Config> c) && { configs_ = std::move(c); return std::move(*this); }
  // predicates run at search time, so prune() and configs() compose in either order
  Autotuner prune(std::function<bool(const Config&)> keep) && { prune_.push_back(std::move(keep)); return std::move(*this); }
  Autotuner budget(std::chrono::milliseconds b) && { budget_ = b; return std::move(*this); }
  Autotuner bench_options(bench::BenchOptions b) && { bench_ = b; return std::move(*this); }
  Autotuner log(std::string path) && { log_path_ = std::move(path); return std::move(*this); }
  std::vector<Config> pruned_configs() const {
    std::vector<Config> kept;
    for (auto& c : configs_) {
      bool keep = true;
      for (auto& p : prune_) keep = keep && p(c);
      if (keep) kept.push_back(c);
    }
    return kept;
  }

  // setup(stream, config) returns the closure to time, or an error: the candidate is then
  // recorded as invalid and the search goes on.
  Result<Output> run(const std::shared_ptr<Stream>& stream, Setup setup) && {
    std::vector<Config> kept = pruned_configs();
    auto log = TrialLog::open(log_path_, name_, space_hash(kept));
    if (log.is_err()) return log.error();
    GridSearch grid = GridSearch{}.resume(log.value().existing_trials());
    return run_searcher(grid, std::move(kept), stream, std::move(setup), &log.value());
  }
  Result<Output> run_with(Searcher& searcher, const std::shared_ptr<Stream>& stream, Setup setup) && {
    std::vector<Config> kept = pruned_configs();
    auto log = TrialLog::open(log_path_, name_, space_hash(kept));
    if (log.is_err()) return log.error();
    return run_searcher(searcher, std::move(kept), stream, std::move(setup), &log.value());
  }

 private:
  struct BenchOracle : Oracle {
    std::vector<Config> cfgs;
    std::shared_ptr<Stream> stream;
    Setup setup;
    bench::BenchOptions bench;
    std::optional<std::chrono::steady_clock::time_point> deadline;
    TrialLog* log;
    const std::vector<Config>& configs() const override { return cfgs; }
    std::optional<std::chrono::nanoseconds> budget_remaining() const override {
      if (!deadline) return std::nullopt;
      auto left = *deadline - std::chrono::steady_clock::now();
      return std::max(left, std::chrono::steady_clock::duration::zero());
    }
    Trial measure(size_t i) override {
      Trial t;
      auto f = setup(stream, cfgs[i]);
      if (f.is_err()) {
        t = Trial::invalid(cfgs[i].id, f.error().to_string());
      } else {
        auto m = bench::do_bench(stream, bench, f.value());
        t = m.is_err() ? Trial::invalid(cfgs[i].id, m.error().to_string()) : Trial::from_measurement(cfgs[i].id, m.value());
      }
      log->append(t);
      return t;
    }
    // contemporaneous A/B/A/B re-measurement of the two finalists
    RunoffResult runoff(const Config& a, const Config& b) {
      auto fa = setup(stream, a);
      if (fa.is_err()) return RunoffError{RunoffError::Kind::SetupA, fa.error()};
      auto fb = setup(stream, b);
      if (fb.is_err()) return RunoffError{RunoffError::Kind::SetupB, fb.error()};
      auto pair = bench::do_bench_paired(stream, bench, fa.value(), fb.value());
      if (pair.is_err()) return RunoffError{RunoffError::Kind::Bench, pair.error()};
      return pair.value();
    }
  };

  Result<Output> run_searcher(Searcher& searcher, std::vector<Config> kept, const std::shared_ptr<Stream>& stream, Setup setup, TrialLog* log) {
    BenchOracle oracle;
    oracle.cfgs = std::move(kept);
    oracle.stream = stream;
    oracle.setup = std::move(setup);
    oracle.bench = bench_;
    if (budget_) oracle.deadline = std::chrono::steady_clock::now() + *budget_;
    oracle.log = log;
    Output out;
    out.trials = searcher.search(oracle);
    // Sequential medians drift with clocks and temperature: the two best meet again, interleaved.
    // An exhausted budget skips that and lets the sequential medians decide.
    auto [first, second] = top_two(oracle.cfgs, out.trials);
    if (first && !second) out.best = *first;
    else if (first && second) {
      if (oracle.budget_exhausted()) out.best = *first;
      else {
        const Config a = *first, b = *second;
        out.best = runoff_verdict(a, b, oracle.runoff(a, b), &out.trials, log);
      }
    }
    return out;
  }

  std::string name_;
  std::vector<Config> configs_;
  std::vector<std::function<bool(const Config&)>> prune_;
  std::optional<std::chrono::milliseconds> budget_;
  bench::BenchOptions bench_;
  std::optional<std::string> log_path_;
};

// ---- records of winners ------------------------------------------------------------------------------
constexpr uint32_t kRecordSchema = 1;

struct RecordEntry {
  std::string bucket;                    // shape class this winner applies to, e.g. "n<=8192"
  Config config;
  float median_ms = 0;
  size_t samples = 0;
  std::optional<std::string> l2_key;     // the winner's kernel fingerprint at tune time, for the strong staleness check
};

// The provenance a record is checked against.
struct Workspace {
  std::string kernel;                    // kernel / tuner the caller loads FOR
  std::string source_hash;
  std::string arch;
  std::string tileiras_fingerprint;      // field name kept from the reference's format: the device toolchain's fingerprint
  std::optional<std::string> space_hash;

  // The running library's provenance for `function` (one of cutile_kernel_list()'s kernels).
  static Result<Workspace> of_kernel(const std::string& function, std::optional<std::string> space = std::nullopt) {
    char fp[17];
    CUTILE_TRY_STATUS(cutile_kernel_fingerprint(function.c_str(), nullptr, fp));
    return Workspace{function, fp, cutile_target_arch(), cutile_toolchain_fingerprint(), std::move(space)};
  }
};

// Fingerprint of one variant in the running library: what `verify_l2` returns for an entry whose
// config names a variant.
inline Result<std::optional<std::string>> variant_key(const std::string& function, const std::string& variant) {
  char fp[17];
  CUTILE_TRY_STATUS(cutile_kernel_fingerprint(function.c_str(), variant.c_str(), fp));
  return std::optional<std::string>(fp);
}

struct Record {
  uint32_t schema = kRecordSchema;
  std::string kernel, source_hash, cutile_version, tileiras_fingerprint, arch, machine;
  uint64_t created_unix_secs = 0;
  std::optional<std::string> space_hash, gate;
  std::vector<RecordEntry> entries;

  explicit Record(const Workspace& ws)
      : kernel(ws.kernel), source_hash(ws.source_hash), cutile_version(cutile_library_version()),
        tileiras_fingerprint(ws.tileiras_fingerprint), arch(ws.arch), machine(hostname()),
        created_unix_secs((uint64_t)std::time(nullptr)), space_hash(ws.space_hash) {}
  Record() = default;

  // one winner per bucket; replacement keeps the entry's place so that committed records diff cleanly
  void insert(RecordEntry e) {
    for (auto& slot : entries)
      if (slot.bucket == e.bucket) { slot = std::move(e); return; }
    entries.push_back(std::move(e));
  }
  const RecordEntry* get(const std::string& bucket) const {
    for (auto& e : entries)
      if (e.bucket == bucket) return &e;
    return nullptr;
  }

  Result<Unit> save(const std::string& path) const {
    auto opt = [](const std::optional<std::string>& s) { return s ? json::Value::string(*s) : json::Value::null(); };
    json::Value list = json::Value::array();
    for (auto& e : entries)
      list.items.push_back(json::Value::object().set("bucket", json::Value::string(e.bucket)).set("config", e.config.to_json())
                               .set("median_ms", json::Value::number(e.median_ms)).set("samples", json::Value::integer((int64_t)e.samples))
                               .set("l2_key", opt(e.l2_key)));
    json::Value v = json::Value::object();
    v.set("schema", json::Value::integer(schema)).set("kernel", json::Value::string(kernel)).set("source_hash", json::Value::string(source_hash))
        .set("cutile_version", json::Value::string(cutile_version)).set("tileiras_fingerprint", json::Value::string(tileiras_fingerprint))
        .set("arch", json::Value::string(arch)).set("machine", json::Value::string(machine))
        .set("created_unix_secs", json::Value::integer((int64_t)created_unix_secs)).set("space_hash", opt(space_hash)).set("gate", opt(gate))
        .set("entries", std::move(list));
    std::ofstream out(path, std::ios::trunc);
    if (!out) return DeviceError::tensor("record write: cannot open " + path);
    out << json::dump(v, true);
    if (!out.good()) return DeviceError::tensor("record write: " + path);
    return ok();
  }

  // Loads without verification; prefer load_verified wherever the entries will be applied.
  static Result<Record> load(const std::string& path) {
    std::ifstream in(path, std::ios::binary);
    if (!in) return DeviceError::tensor("record read: cannot open " + path);
    std::stringstream ss;
    ss << in.rdbuf();
    auto doc = json::parse(ss.str());
    auto bad = [&](const std::string& what) { return DeviceError::tensor("record parse: " + what + " (" + path + ")"); };
    if (!doc || !doc->is_object()) return bad("not a JSON object");
    Record r;
    auto text = [&](const char* key, std::string* dst) { const json::Value* x = doc->get(key); if (!x || !x->is_string()) return false; *dst = x->s; return true; };
    auto opt_text = [&](const char* key, std::optional<std::string>* dst) { const json::Value* x = doc->get(key); if (x && x->is_string()) *dst = x->s; };
    const json::Value* schema = doc->get("schema");
    if (!schema || schema->kind != json::Value::Kind::Int) return bad("missing field `schema`");
    r.schema = (uint32_t)schema->i;
    for (auto kv : {std::make_pair("kernel", &r.kernel), std::make_pair("source_hash", &r.source_hash), std::make_pair("cutile_version", &r.cutile_version),
                    std::make_pair("tileiras_fingerprint", &r.tileiras_fingerprint), std::make_pair("arch", &r.arch), std::make_pair("machine", &r.machine)})
      if (!text(kv.first, kv.second)) return bad(std::string("missing field `") + kv.first + "`");
    if (const json::Value* c = doc->get("created_unix_secs")) r.created_unix_secs = (uint64_t)c->as_double();
    opt_text("space_hash", &r.space_hash);
    opt_text("gate", &r.gate);
    const json::Value* list = doc->get("entries");
    if (!list || !list->is_array()) return bad("missing field `entries`");
    for (auto& item : list->items) {
      RecordEntry e;
      const json::Value* bucket = item.get("bucket");
      const json::Value* config = item.get("config");
      const json::Value* median = item.get("median_ms");
      const json::Value* samples = item.get("samples");
      auto cfg = config ? Config::from_json(*config) : std::nullopt;
      if (!bucket || !bucket->is_string() || !cfg || !median || !samples || !samples->is_number()) return bad("malformed entry");
      e.bucket = bucket->s;
      e.config = *cfg;
      e.median_ms = median->is_null() ? NAN : (float)median->as_double();
      e.samples = (size_t)samples->as_double();
      if (const json::Value* k = item.get("l2_key"); k && k->is_string()) e.l2_key = k->s;
      r.entries.push_back(std::move(e));
    }
    return r;
  }

  // Loads and verifies against the running workspace (tune.rs:906-1016).
  // REFUSES on a schema, kernel, arch or source_hash mismatch; a space_hash mismatch when both sides
  // carry one; duplicate buckets; an entry whose id disagrees with its parameters; and, when the
  // toolchain fingerprints match, a stored key that differs from the one `verify_l2` recomputes.
  // WARNS (returned, never silent) on toolchain drift (the key check is then skipped: keys made by
  // another toolchain cannot match), a record without space_hash where the workspace has one,
  // entries without a key, entries whose key the verifier declined to recompute, and library version drift.
  using VerifyKey = std::function<Result<std::optional<std::string>>(const RecordEntry&)>;
  static Result<std::pair<Record, std::vector<std::string>>> load_verified(const std::string& path, const Workspace& ws, const VerifyKey& verify_l2) {
    auto loaded = load(path);
    if (loaded.is_err()) return loaded.error();
    Record record = std::move(loaded).unwrap();
    auto refuse = [&](const std::string& what, const std::string& stored, const std::string& current) {
      return DeviceError::tensor("stale tuning record at " + path + ": " + what + " mismatch (record: " + stored + ", workspace: " + current +
                                 "); re-tune or delete it");
    };
    if (record.schema != kRecordSchema) return refuse("schema", std::to_string(record.schema), std::to_string(kRecordSchema));
    if (record.kernel != ws.kernel) return refuse("kernel", record.kernel, ws.kernel);
    if (record.arch != ws.arch) return refuse("arch", record.arch, ws.arch);
    if (record.source_hash != ws.source_hash) return refuse("source_hash", record.source_hash, ws.source_hash);
    if (record.space_hash && ws.space_hash && *record.space_hash != *ws.space_hash) return refuse("space_hash", *record.space_hash, *ws.space_hash);
    std::set<std::string> seen;
    for (auto& e : record.entries) {
      if (!seen.insert(e.bucket).second)
        return DeviceError::tensor("tuning record at " + path + " has duplicate entries for bucket " + json::quote(e.bucket) + "; fix or re-tune it");
      const std::string derived = Config::make(e.config.params).id;
      if (e.config.id != derived) return refuse("config id for bucket " + json::quote(e.bucket), e.config.id, derived);
    }
    std::vector<std::string> warnings;
    if (!record.space_hash && ws.space_hash)
      warnings.push_back("tuning record carries no space_hash; the search-space match was not checked");
    if (record.tileiras_fingerprint != ws.tileiras_fingerprint) {
      warnings.push_back("tuning record was produced by a different tileiras (" + record.tileiras_fingerprint + " vs " + ws.tileiras_fingerprint +
                         "); configs remain valid but timings may have shifted and per-entry key verification was skipped — consider re-tuning");
    } else {
      for (auto& e : record.entries) {
        if (!e.l2_key) {
          warnings.push_back("bucket " + json::quote(e.bucket) + " carries no l2 key; only source-level staleness checks applied");
          continue;
        }
        auto current = verify_l2(e);
        if (current.is_err()) return current.error();
        if (!current.value()) warnings.push_back("bucket " + json::quote(e.bucket) + ": verifier declined to recompute the l2 key; stored key not checked");
        else if (*current.value() != *e.l2_key) return refuse("l2 key for bucket " + json::quote(e.bucket), *e.l2_key, *current.value());
      }
    }
    if (record.cutile_version != cutile_library_version())
      warnings.push_back("tuning record was produced by cutile " + record.cutile_version + " (running " + cutile_library_version() + ")");
    return std::make_pair(std::move(record), std::move(warnings));
  }

 private:
  static std::string hostname() {
    std::ifstream in("/etc/hostname");
    std::string h;
    if (in && std::getline(in, h)) {
      h.erase(0, h.find_first_not_of(" \t\r\n"));
      h.erase(h.find_last_not_of(" \t\r\n") + 1);
      if (!h.empty()) return h;
    }
    const char* env = getenv("HOSTNAME");
    return env && *env ? env : "unknown";
  }
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
    if (v.find('+') != std::string::npos) continue;      // a member of a kernel family: chosen by the launcher, not a variant of its own
    if (!must_contain.empty() && v.find(must_contain) == std::string::npos) continue;
    out.push_back(Config::make({{"variant", ParamValue(v)}}));
  }
  return out;
}

}  // namespace tune
}  // namespace cutile
