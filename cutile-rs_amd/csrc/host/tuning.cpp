// Tuning records at library start-up: the winners the autotuner measured for shape classes of the benchmark
// configurations, committed as JSON next to the library (cutile-rs_amd/tuned/<kernel>.json, the format of
// cutile/src/tune.rs:762-832) and applied through the bucket preferences of the kernel table.
//
// A record is applied only after Record::load_verified accepts it against the running library: same schema, kernel,
// architecture and code-object fingerprint (source_hash), and for every entry a variant fingerprint equal to the
// stored one.  A stale or foreign record is refused as a whole and reported (cutile_tuning_report), never half
// applied; without records the table's own order decides, so deleting them changes only where a choice comes from.
#include <dirent.h>
#include <dlfcn.h>

#include <algorithm>
#include <mutex>
#include <string>
#include <vector>

#include "../../../include/cutile/tune.hpp"
#include "kernel_table.h"

namespace cutile {
namespace {
std::once_flag g_once;
std::mutex g_report_mutex;
std::string g_report;
int32_t g_applied = 0;

std::string default_directory() {
  if (const char* env = getenv("CUTILE_TUNING_RECORDS")) return env;   // an empty value switches records off
  Dl_info info;
  if (dladdr((const void*)&cutile_tuning_reload, &info) && info.dli_fname) {
    std::string self = info.dli_fname;
    size_t slash = self.rfind('/');
    if (slash != std::string::npos) return self.substr(0, slash) + "/../tuned";
  }
  return "";
}

void load_directory(const std::string& dir) {
  std::lock_guard<std::mutex> lock(g_report_mutex);
  clear_bucket_preferences();
  g_report.clear();
  g_applied = 0;
  if (dir.empty()) { g_report = "tuning records: switched off\n"; return; }
  std::vector<std::string> files;
  if (DIR* d = opendir(dir.c_str())) {
    while (dirent* e = readdir(d)) {
      std::string name = e->d_name;
      if (name.size() > 5 && name.substr(name.size() - 5) == ".json") files.push_back(dir + "/" + name);
    }
    closedir(d);
  } else {
    g_report = "tuning records: no directory " + dir + "\n";
    return;
  }
  std::sort(files.begin(), files.end());
  for (const std::string& path : files) {
    auto raw = tune::Record::load(path);
    if (raw.is_err()) { g_report += "refused " + path + ": " + raw.error().message + "\n"; continue; }
    auto ws = tune::Workspace::of_kernel(raw.value().kernel);
    if (ws.is_err()) { g_report += "refused " + path + ": " + ws.error().message + "\n"; continue; }
    const std::string kernel = raw.value().kernel;
    auto verified = tune::Record::load_verified(path, ws.value(), [&](const tune::RecordEntry& e) -> Result<std::optional<std::string>> {
      auto v = e.config.str("variant");
      if (!v) return std::optional<std::string>();
      return tune::variant_key(kernel, *v);
    });
    if (verified.is_err()) { g_report += "refused " + path + ": " + verified.error().message + "\n"; continue; }
    // a toolchain other than the one that built this library means the stored keys were not compared: do not apply
    bool drift = false;
    for (auto& w : verified.value().second) {
      g_report += "warning " + path + ": " + w + "\n";
      if (w.find("different tileiras") != std::string::npos) drift = true;
    }
    if (drift) { g_report += "refused " + path + ": produced by another device toolchain; re-tune\n"; continue; }
    int n = 0;
    for (auto& e : verified.value().first.entries) {
      auto v = e.config.str("variant");
      if (!v) continue;
      if (cutile_kernel_set_preferred_variant_for(kernel.c_str(), e.bucket.c_str(), v->c_str()) == CUTILE_SUCCESS) ++n;
      else g_report += "warning " + path + ": bucket " + e.bucket + " names an unknown variant " + *v + "\n";
    }
    g_applied += n;
    g_report += "applied " + path + ": " + std::to_string(n) + " bucket(s) of kernel " + kernel + "\n";
  }
}
}  // namespace

void ensure_tuning_records_loaded() {
  std::call_once(g_once, [] { load_directory(default_directory()); });
}
}  // namespace cutile

extern "C" {
cutile_status_t cutile_tuning_reload(const char* directory) {
  cutile::ensure_tuning_records_loaded();                 // so that a later first use does not undo this call
  cutile::load_directory(directory ? std::string(directory) : cutile::default_directory());
  return CUTILE_SUCCESS;
}
const char* cutile_tuning_report(void) {
  cutile::ensure_tuning_records_loaded();
  std::lock_guard<std::mutex> lock(cutile::g_report_mutex);
  static thread_local std::string copy;
  copy = cutile::g_report;
  return copy.c_str();
}
int32_t cutile_tuning_applied_count(void) {
  cutile::ensure_tuning_records_loaded();
  std::lock_guard<std::mutex> lock(cutile::g_report_mutex);
  return cutile::g_applied;
}
}  // extern "C"
