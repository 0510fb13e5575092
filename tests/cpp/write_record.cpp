// Test helper: writes one tuning record through the C++ surface (tune::Record::save), with the running library's
// provenance unless a field is overridden:  write_record <path> <kernel> <bucket> <variant> [field=value ...]
// fields: source_hash, arch, tileiras_fingerprint, schema, l2_key
#include <cutile/cutile.hpp>

#include <cstdio>
#include <cstring>

using namespace cutile;

int main(int argc, char** argv) {
  if (argc < 5) { fprintf(stderr, "usage: %s <path> <kernel> <bucket> <variant> [field=value ...]\n", argv[0]); return 2; }
  const std::string path = argv[1], kernel = argv[2], bucket = argv[3], variant = argv[4];
  auto ws = tune::Workspace::of_kernel(kernel);
  if (ws.is_err()) { fprintf(stderr, "%s\n", ws.error().message.c_str()); return 1; }
  tune::Record record(ws.value());
  auto key = tune::variant_key(kernel, variant);
  if (key.is_err()) { fprintf(stderr, "%s\n", key.error().message.c_str()); return 1; }
  tune::RecordEntry entry{bucket, tune::Config::make({{"variant", tune::ParamValue(variant)}}), 1.0f, 10, key.value()};
  for (int i = 5; i < argc; ++i) {
    const char* eq = strchr(argv[i], '=');
    if (!eq) continue;
    const std::string field(argv[i], eq - argv[i]), value(eq + 1);
    if (field == "source_hash") record.source_hash = value;
    else if (field == "arch") record.arch = value;
    else if (field == "tileiras_fingerprint") record.tileiras_fingerprint = value;
    else if (field == "schema") record.schema = (uint32_t)atoi(value.c_str());
    else if (field == "l2_key") entry.l2_key = value;
  }
  record.insert(std::move(entry));
  return record.save(path).is_ok() ? 0 : 1;
}
