// Parts C and D of the C ABI: the launch builder and the per-kernel launchers.
//
// A launcher here does what the reference's macro-generated launcher does in
// execute() (cutile-macro/src/kernel_launcher_generator.rs:821-987): infer or
// check the generics, validate every tensor against the kernel's signature,
// infer and validate the launch grid from the output partition
// (cutile/src/tile_kernel.rs:782-808,934-967), resolve the kernel (here: pick a
// precompiled variant instead of compiling), push the arguments in signature
// order (cutile/src/tensor.rs:1723-1739,2005-2016) and launch.  Every check runs
// before any GPU work, as in the reference.
#include <dlfcn.h>

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "common.h"
#include "kernel_table.h"
#include "runtime_state.h"
#include "scratch.h"
#include "../kernels/mapped_partition.h"

using cutile::MappedArg;
using cutile::MappedRangeArg;
using cutile::mapped_index;

using namespace cutile;

namespace cutile {

cutile_status_t current_device(cutile_device_t* device) {
  if (cutile_status_t s = ensure_init()) return s;
  CUTILE_API_OR_RETURN(api);
  int ord = 0;
  CUTILE_HIP_OR_RETURN(api, hipGetDevice(&ord));
  return cutile_device_get(ord, device);
}

cutile_status_t compute_units(cutile_device_t device, int* count) {
  CUTILE_REQUIRE(device && count, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  std::lock_guard<std::mutex> lock(device->mutex);
  if (device->compute_units <= 0) {
    CUTILE_API_OR_RETURN(api);
    int v = 0;
    CUTILE_HIP_OR_RETURN(api, hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, device->ordinal));
    device->compute_units = v;
  }
  *count = device->compute_units;
  return CUTILE_SUCCESS;
}

namespace {

struct DTypeInfo {
  const char* name;
  size_t size;
};
const DTypeInfo kDTypes[CUTILE_DTYPE_COUNT] = {
    {"f32", 4}, {"f64", 8}, {"f16", 2}, {"bf16", 2}, {"i8", 1},  {"i16", 2},      {"i32", 4},    {"i64", 8},
    {"u8", 1},  {"u16", 2}, {"u32", 4}, {"u64", 8},  {"bool", 1}, {"f8e4m3fn", 1}, {"f8e5m2", 1}, {"f8e8m0fnu", 1},
    {"f4e2m1fnx2", 1}};

uint16_t f32_to_f16_bits(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u, abs = x & 0x7fffffffu;
  if (abs >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (abs > 0x7f800000u ? 0x0200u : 0));
  if (abs >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);
  if (abs < 0x38800000u) {
    if (abs < 0x33000000u) return (uint16_t)sign;
    int e = (int)(abs >> 23);
    uint32_t man = (abs & 0x7fffffu) | 0x800000u;
    int shift = 126 - e;
    uint32_t q = man >> shift, rem = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint16_t)(sign | q);
  }
  uint32_t h = (((abs >> 23) - 112u) << 10) | ((abs & 0x7fffffu) >> 13);
  uint32_t rem = abs & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
  return (uint16_t)(sign | h);
}
uint16_t f32_to_bf16_bits(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
  x += 0x7fffu + ((x >> 16) & 1u);
  return (uint16_t)(x >> 16);
}

// Encodes a scalar kernel argument of type `dt` from a double (floats) or an
// int64 (integers).  Returns the number of bytes written, 0 if unsupported.
size_t scalar_bits(cutile_dtype_t dt, double v, int64_t iv, unsigned char out[8]) {
  switch (dt) {
    case CUTILE_DTYPE_F32: { float f = (float)v; memcpy(out, &f, 4); return 4; }
    case CUTILE_DTYPE_F64: memcpy(out, &v, 8); return 8;
    case CUTILE_DTYPE_F16: { uint16_t h = f32_to_f16_bits((float)v); memcpy(out, &h, 2); return 2; }
    case CUTILE_DTYPE_BF16: { uint16_t h = f32_to_bf16_bits((float)v); memcpy(out, &h, 2); return 2; }
    case CUTILE_DTYPE_I8: case CUTILE_DTYPE_U8: case CUTILE_DTYPE_BOOL: { int8_t x = (int8_t)iv; memcpy(out, &x, 1); return 1; }
    case CUTILE_DTYPE_I16: case CUTILE_DTYPE_U16: { int16_t x = (int16_t)iv; memcpy(out, &x, 2); return 2; }
    case CUTILE_DTYPE_I32: case CUTILE_DTYPE_U32: { int32_t x = (int32_t)iv; memcpy(out, &x, 4); return 4; }
    case CUTILE_DTYPE_I64: case CUTILE_DTYPE_U64: memcpy(out, &iv, 8); return 8;
    default: return 0;
  }
}

// Kernel-argument buffer laid out like the kernarg segment: every value at its
// natural alignment, in push order.
struct ArgPacker {
  std::vector<unsigned char> buf;
  void push(const void* v, size_t size, size_t align) {
    size_t off = (buf.size() + align - 1) / align * align;
    buf.resize(off + size);
    memcpy(buf.data() + off, v, size);
  }
  template <typename T>
  void push_val(T v) { push(&v, sizeof(T), alignof(T)); }
  void push_tensor(const cutile_tensor_arg_t& t) {
    push_val<void*>(t.ptr);
    for (int i = 0; i < t.rank; ++i) push_val<int32_t>(t.shape[i]);
    for (int i = 0; i < t.rank; ++i) push_val<int32_t>(t.strides[i]);
  }
  void push_partition(const cutile_partition_arg_t& p) {
    push_tensor(p.tensor);
    for (int i = 0; i < p.tensor.rank; ++i) push_val<int32_t>(p.partition_shape[i]);
    for (int i = 0; i < p.tensor.rank; ++i) push_val<int32_t>(p.partition_strides[i]);
  }
  void push_tile_grid(const uint32_t g[3]) {
    uint32_t v[4] = {g[0], g[1], g[2], 0};
    push(v, sizeof(v), 4);
  }
};

// What the calling thread's next launcher calls do once their checks have passed (cutile_set_launch_mode), and the
// table entry the thread's last launcher call resolved (cutile_last_resolved_kernel).
thread_local int g_launch_mode = 0;
// Shape class of the launch being resolved (set by the launchers that tuning records cover) and where the last
// resolved variant came from: "caller" (opts.variant), "record:<bucket>" (a verified tuning record), "pinned"
// (cutile_kernel_set_preferred_variant) or "table" (the table's order).
thread_local std::string g_bucket;
thread_local std::string g_last_source;
thread_local std::string g_last_bucket;
struct BucketScope {
  explicit BucketScope(std::string b) { g_bucket = std::move(b); }
  ~BucketScope() { g_bucket.clear(); }
};
thread_local const KernelEntry* g_last_entry = nullptr;
thread_local hipFunction_t g_last_fn = nullptr;

cutile_status_t launch_packed(hipFunction_t fn, const uint32_t grid[3], const uint32_t block[3],
                              uint32_t dyn_lds, cutile_stream_t stream, ArgPacker& args) {
  if (g_launch_mode != 0) {   // compile-only / specialize-only: every check has run, nothing is enqueued
    CUTILE_REQUIRE(grid[0] > 0 && grid[1] > 0 && grid[2] > 0, CUTILE_ERR_KERNEL_LAUNCH,
                   "launch grid (%u, %u, %u) has a zero axis", grid[0], grid[1], grid[2]);
    return CUTILE_SUCCESS;
  }
  CUTILE_API_OR_RETURN(api);
  CUTILE_REQUIRE(grid[0] > 0 && grid[1] > 0 && grid[2] > 0, CUTILE_ERR_KERNEL_LAUNCH,
                 "launch grid (%u, %u, %u) has a zero axis", grid[0], grid[1], grid[2]);
  // what one dispatch can express: 2^31 - 1 workgroups on x, 65535 on y and z, fewer than 2^32 lanes per axis
  CUTILE_REQUIRE(grid[0] <= 0x7fffffffu && grid[1] <= 65535u && grid[2] <= 65535u &&
                     (uint64_t)grid[0] * block[0] <= 0xffffffffull,
                 CUTILE_ERR_KERNEL_LAUNCH, "launch grid (%u, %u, %u) exceeds what one dispatch can hold", grid[0], grid[1], grid[2]);
  size_t size = args.buf.size();
  void* extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, args.buf.data(), HIP_LAUNCH_PARAM_BUFFER_SIZE, &size,
                   HIP_LAUNCH_PARAM_END};
  CUTILE_HIP_OR_RETURN(api, hipModuleLaunchKernel(fn, grid[0], grid[1], grid[2], block[0], block[1], block[2],
                                                  dyn_lds, (hipStream_t)stream, nullptr, extra));
  return CUTILE_SUCCESS;
}

// ---- validation helpers --------------------------------------------------------------------
cutile_status_t check_tensor(const cutile_tensor_arg_t* t, const char* name, int rank_lo, int rank_hi) {
  CUTILE_REQUIRE(t, CUTILE_ERR_INVALID_ARGUMENT, "%s is null", name);
  CUTILE_REQUIRE(t->rank >= rank_lo && t->rank <= rank_hi, CUTILE_ERR_KERNEL_LAUNCH,
                 "%s: expected rank %d%s, got %d", name, rank_lo, rank_lo == rank_hi ? "" : "+", t->rank);
  CUTILE_REQUIRE((unsigned)t->dtype < CUTILE_DTYPE_COUNT, CUTILE_ERR_INVALID_ARGUMENT, "%s: bad dtype", name);
  for (int i = 0; i < t->rank; ++i)
    CUTILE_REQUIRE(t->shape[i] > 0, CUTILE_ERR_TENSOR, "%s: Shape dimensions must be positive.", name);
  CUTILE_REQUIRE(t->ptr, CUTILE_ERR_INVALID_ARGUMENT, "%s: null device pointer", name);
  return CUTILE_SUCCESS;
}

cutile_status_t check_partition(const cutile_partition_arg_t* p, const char* name, int rank_lo, int rank_hi) {
  CUTILE_REQUIRE(p, CUTILE_ERR_INVALID_ARGUMENT, "%s is null", name);
  if (cutile_status_t s = check_tensor(&p->tensor, name, rank_lo, rank_hi)) return s;
  for (int i = 0; i < p->tensor.rank; ++i)
    CUTILE_REQUIRE(p->partition_shape[i] > 0, CUTILE_ERR_TENSOR, "%s: partition shape must be positive", name);
  return CUTILE_SUCCESS;
}

bool is_contiguous(const cutile_tensor_arg_t& t) {
  int64_t expect = 1;
  for (int i = t.rank - 1; i >= 0; --i) {
    if (t.shape[i] != 1 && t.strides[i] != expect) return false;
    expect *= t.shape[i];
  }
  return true;
}
bool same_shape(const cutile_tensor_arg_t& a, const cutile_tensor_arg_t& b) {
  if (a.rank != b.rank) return false;
  for (int i = 0; i < a.rank; ++i)
    if (a.shape[i] != b.shape[i]) return false;
  return true;
}
bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

// The pipelined matrix kernels address a whole operand through one buffer descriptor with 32-bit byte offsets, and
// offset 0x80000000 stands for "outside": an operand must end below 2 GiB from its first element.  Bytes from the
// first element of row 0 to the end of the last row of a rank-2 tensor (rank-2 view of the two innermost axes).
int64_t extent_bytes_2d(int64_t rows, int64_t cols, int64_t row_stride, int64_t elem_size) {
  return rows > 0 && cols > 0 ? ((rows - 1) * row_stride + cols) * elem_size : 0;
}
int64_t extent_bytes_2d(const cutile_tensor_arg_t& t) {
  return extent_bytes_2d(t.shape[0], t.shape[1], t.strides[0], (int64_t)cutile_dtype_size(t.dtype));
}
constexpr int64_t kDescriptorLimit = 1ll << 31;
int64_t numel(const cutile_tensor_arg_t& t) {
  int64_t n = 1;
  for (int i = 0; i < t.rank; ++i) n *= t.shape[i];
  return n;
}

// Optional .generics() check: entry i of the caller's list must equal `expect`.
cutile_status_t check_generic(const cutile_launch_opts_t* o, int i, const std::string& expect, const char* what) {
  if (!o || !o->generics || i >= o->n_generics) return CUTILE_SUCCESS;
  CUTILE_REQUIRE(o->generics[i] && expect == o->generics[i], CUTILE_ERR_KERNEL_LAUNCH,
                 "generic %s: launcher was given '%s' but the arguments imply '%s'", what,
                 o->generics[i] ? o->generics[i] : "(null)", expect.c_str());
  return CUTILE_SUCCESS;
}
int generic_int(const cutile_launch_opts_t* o, int i, int fallback) {
  if (!o || !o->generics || i >= o->n_generics || !o->generics[i]) return fallback;
  return atoi(o->generics[i]);
}

struct Resolved {
  const KernelEntry* entry = nullptr;
  hipFunction_t fn = nullptr;
  uint32_t tile_grid[3] = {0, 0, 0};
  cutile_device_t device = nullptr;
};

// Infers/validates the tile grid from the output partition and the caller's
// explicit grid.
cutile_status_t resolve_grid(const cutile_partition_arg_t* out, const cutile_launch_opts_t* opts, uint32_t grid[3]) {
  uint32_t explicit_grid[3] = {0, 0, 0};
  if (opts) memcpy(explicit_grid, opts->grid, sizeof(explicit_grid));
  const cutile_partition_arg_t* parts[1] = {out};
  return cutile_infer_launch_grid(explicit_grid, parts, 1, grid);
}

// Picks the variant.  Precedence: the caller's variant, the function-wide pin set at run time
// (cutile_kernel_set_preferred_variant), the shape class's winner (a verified tuning record or
// cutile_kernel_set_preferred_variant_for), then `fallback` (the table's order).  A pin or a winner that does not fit
// these arguments is passed over, not an error.
cutile_status_t resolve_entry(const char* function, const cutile_launch_opts_t* opts, const std::string& fallback,
                              const std::vector<std::string>& acceptable, Resolved* r) {
  std::string want;
  g_last_source = "caller";
  g_last_bucket = g_bucket;
  auto fits = [&](const std::string& v) { return !v.empty() && std::find(acceptable.begin(), acceptable.end(), v) != acceptable.end(); };
  if (opts && opts->variant) want = opts->variant;
  if (want.empty()) {
    std::string pref = preferred_variant(function);
    if (fits(pref)) {
      want = pref;
      g_last_source = "pinned";
    }
  }
  if (want.empty() && !g_bucket.empty()) {
    ensure_tuning_records_loaded();
    std::string pref = preferred_variant_for(function, g_bucket);
    if (fits(pref)) {
      want = pref;
      g_last_source = "record:" + g_bucket;
    }
  }
  if (want.empty()) {
    want = fallback;
    g_last_source = "table";
  }
  if (!acceptable.empty() && std::find(acceptable.begin(), acceptable.end(), want) == acceptable.end()) {
    std::string list;
    for (auto& a : acceptable) list += (list.empty() ? "" : ", ") + a;
    return fail(CUTILE_ERR_KERNEL_NOT_FOUND, "variant '%s' of kernel '%s' does not fit these arguments; fitting: %s",
                want.c_str(), function, list.c_str());
  }
  r->entry = find_entry(function, want);
  CUTILE_REQUIRE(r->entry, CUTILE_ERR_KERNEL_NOT_FOUND, "no variant '%s' of kernel '%s'; available: %s",
                 want.c_str(), function, list_variants(function).c_str());
  g_last_entry = r->entry;
  g_last_fn = nullptr;
  if (g_launch_mode == 2) return CUTILE_SUCCESS;   // specialize-only: the identity is known, nothing is loaded
  if (cutile_status_t s = current_device(&r->device)) return s;
  if (cutile_status_t s = load_entry(r->device, r->entry, &r->fn)) return s;
  g_last_fn = r->fn;
  return CUTILE_SUCCESS;
}

uint32_t div_up(uint64_t a, uint64_t b) { return (uint32_t)((a + b - 1) / b); }

// The streaming GEMM variants ("..._s2x4"): a family of kernels behind one variant name.
bool is_stream_variant(const char* variant) { return strstr(variant, "_s2x4") != nullptr; }
// An output of this size or more is read and stored past the caches (it cannot still be cached when its consumer runs,
// and the caches are left to the operand panels): the rule of the staged epilogue, decided on the host for this family.
constexpr int64_t kStreamedOutputBytes = 64ll << 20;
// Replaces the resolved family entry by the member for (z read as the initial accumulator?, z past the caches?) and
// gives the launch grid: one workgroup per compute unit, or per tile if there are fewer tiles.
cutile_status_t stream_member(Resolved* r, const char* function, bool accumulate, const cutile_tensor_arg_t& zt, uint64_t tiles,
                              uint32_t* grid) {
  const bool past_caches = (int64_t)zt.shape[0] * zt.shape[1] * (int64_t)cutile_dtype_size(zt.dtype) >= kStreamedOutputBytes;
  std::string member = r->entry->variant;
  if (!accumulate) member += "+new";
  if (!past_caches) member += "+cached";
  const KernelEntry* e = find_entry(function, member);
  CUTILE_REQUIRE(e, CUTILE_ERR_KERNEL_NOT_FOUND, "kernel '%s' has no member '%s'", function, member.c_str());
  int cus = 256;
  if (g_launch_mode != 2) {
    if (cutile_status_t s = compute_units(r->device, &cus)) return s;
    if (e != r->entry)
      if (cutile_status_t s = load_entry(r->device, e, &r->fn)) return s;
    g_last_fn = r->fn;
  }
  *grid = (uint32_t)std::min<uint64_t>(tiles, (uint64_t)std::max(cus, 1));
  return CUTILE_SUCCESS;
}

// Shape classes of tuning records: row lengths by the next power of two (at least 256).
std::string pow2_class(int64_t n) {
  int64_t p = 256;
  while (p < n) p *= 2;
  return "<=" + std::to_string(p);
}

const char* float_dtype_name(cutile_dtype_t dt) { return kDTypes[dt].name; }

}  // namespace
}  // namespace cutile

extern "C" {

// ---- dtypes --------------------------------------------------------------------------------
const char* cutile_dtype_name(cutile_dtype_t dtype) {
  return (unsigned)dtype < CUTILE_DTYPE_COUNT ? kDTypes[dtype].name : "?";
}
size_t cutile_dtype_size(cutile_dtype_t dtype) { return (unsigned)dtype < CUTILE_DTYPE_COUNT ? kDTypes[dtype].size : 0; }
cutile_dtype_t cutile_dtype_from_name(const char* name) {
  if (name)
    for (int i = 0; i < CUTILE_DTYPE_COUNT; ++i)
      if (strcmp(kDTypes[i].name, name) == 0) return (cutile_dtype_t)i;
  return CUTILE_DTYPE_COUNT;
}

// ---- grid inference ------------------------------------------------------------------------
cutile_status_t cutile_partition_grid(const cutile_partition_arg_t* p, uint32_t grid[3]) {
  CUTILE_REQUIRE(p && grid, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  const cutile_tensor_arg_t& t = p->tensor;
  CUTILE_REQUIRE(t.rank >= 1 && t.rank <= 3, CUTILE_ERR_TENSOR, "Mutable tensor must be at most rank 3.");
  for (int i = 0; i < t.rank; ++i)
    CUTILE_REQUIRE(t.shape[i] > 0, CUTILE_ERR_TENSOR, "Shape dimensions must be positive.");
  grid[0] = grid[1] = grid[2] = 1;
  for (int i = 0; i < t.rank; ++i) {
    CUTILE_REQUIRE(p->partition_shape[i] > 0, CUTILE_ERR_TENSOR, "partition shape must be positive");
    grid[i] = div_up((uint32_t)t.shape[i], (uint32_t)p->partition_shape[i]);
  }
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_infer_launch_grid(const uint32_t explicit_grid[3], const cutile_partition_arg_t* const* partitions,
                                         int32_t n_partitions, uint32_t grid[3]) {
  CUTILE_REQUIRE(grid && (partitions || n_partitions <= 0), CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  struct Bound { uint32_t g[3]; bool exact; };
  std::vector<Bound> bounds;
  for (int i = 0; i < n_partitions; ++i) {
    Bound b;
    if (cutile_status_t s = cutile_partition_grid(partitions[i], b.g)) return s;
    b.exact = !partitions[i]->prefix_coverage;
    bounds.push_back(b);
  }
  auto validate = [&](const uint32_t g[3]) -> cutile_status_t {
    for (auto& b : bounds)
      if (b.exact && (b.g[0] != g[0] || b.g[1] != g[1] || b.g[2] != g[2]))
        return fail(CUTILE_ERR_KERNEL_LAUNCH,
                    "launch grid (%u, %u, %u) does not match the inferred partition grid (%u, %u, %u)", g[0], g[1],
                    g[2], b.g[0], b.g[1], b.g[2]);
    for (auto& b : bounds)
      if (!b.exact)
        for (int k = 0; k < 3; ++k)
          if (g[k] > b.g[k])
            return fail(CUTILE_ERR_KERNEL_LAUNCH,
                        "launch grid (%u, %u, %u) exceeds the partial-coverage partition grid (%u, %u, %u) on axis %d",
                        g[0], g[1], g[2], b.g[0], b.g[1], b.g[2], k);
    return CUTILE_SUCCESS;
  };
  const uint32_t zero[3] = {0, 0, 0};
  const uint32_t* eg = explicit_grid ? explicit_grid : zero;
  if (eg[0] || eg[1] || eg[2]) {
    if (cutile_status_t s = validate(eg)) return s;
    memcpy(grid, eg, 3 * sizeof(uint32_t));
    return CUTILE_SUCCESS;
  }
  const Bound* first_exact = nullptr;
  for (auto& b : bounds)
    if (b.exact) { first_exact = &b; break; }
  if (!first_exact) {
    if (bounds.empty()) return fail(CUTILE_ERR_KERNEL_LAUNCH, "Launch grid required.");
    return fail(CUTILE_ERR_KERNEL_LAUNCH,
                "Launch grid required: a partial-coverage (partition_prefix) binding only bounds the grid; specify "
                "the grid explicitly or bind with partition().");
  }
  if (cutile_status_t s = validate(first_exact->g)) return s;
  memcpy(grid, first_exact->g, 3 * sizeof(uint32_t));
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_compute_spec(const cutile_tensor_arg_t* t, cutile_spec_bits_t* spec) {
  CUTILE_REQUIRE(t && spec, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  CUTILE_REQUIRE(t->rank >= 0 && t->rank <= CUTILE_MAX_RANK, CUTILE_ERR_INVALID_ARGUMENT, "bad rank");
  auto pow2 = [](int32_t v) -> int32_t {
    if (v == 0) return 16;
    int32_t d = v & (int32_t)(0u - (uint32_t)v);
    return d < 16 && d > 0 ? d : 16;
  };
  memset(spec, 0, sizeof(*spec));
  spec->base_ptr_div = pow2((int32_t)(uint64_t)(uintptr_t)t->ptr);
  std::vector<std::pair<int32_t, int32_t>> sorted;
  for (int i = 0; i < t->rank; ++i) {
    spec->shape_div[i] = pow2(t->shape[i]);
    spec->stride_div[i] = pow2(t->strides[i]);
    spec->stride_one[i] = t->strides[i] == 1;
    sorted.emplace_back(t->strides[i], t->shape[i]);
  }
  std::sort(sorted.begin(), sorted.end());
  spec->elements_disjoint = sorted.empty() ? 1 : sorted[0].first > 0;
  for (size_t i = 0; i + 1 < sorted.size(); ++i)
    if (sorted[i + 1].first <= 0 || (int64_t)sorted[i + 1].first < (int64_t)sorted[i].first * sorted[i].second) {
      spec->elements_disjoint = 0;
      break;
    }
  return CUTILE_SUCCESS;
}

// ---- Part C: launch builder ----------------------------------------------------------------
}  // extern "C"

struct cutile_launch {
  hipFunction_t function = nullptr;
  ArgPacker args;
  uint32_t grid[3] = {1, 1, 1}, block[3] = {1, 1, 1};
  uint32_t smem = 0;
  bool configured = false;
};

extern "C" {

cutile_status_t cutile_launch_create(cutile_function_t function, cutile_launch_t* launch) {
  CUTILE_REQUIRE(function && launch, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  auto* l = new cutile_launch();
  l->function = (hipFunction_t)function;
  *launch = l;
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_launch_destroy(cutile_launch_t launch) {
  delete launch;
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_launch_push_arg(cutile_launch_t launch, const void* value, size_t size, size_t align) {
  CUTILE_REQUIRE(launch && value && size, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  CUTILE_REQUIRE(align && (align & (align - 1)) == 0, CUTILE_ERR_INVALID_ARGUMENT, "alignment must be a power of two");
  launch->args.push(value, size, align);
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_launch_push_device_ptr(cutile_launch_t launch, void* device_ptr) {
  CUTILE_REQUIRE(launch, CUTILE_ERR_INVALID_ARGUMENT, "launch is null");
  launch->args.push_val<void*>(device_ptr);
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_launch_set_config(cutile_launch_t launch, const uint32_t grid[3], const uint32_t block[3],
                                         uint32_t shared_mem_bytes) {
  CUTILE_REQUIRE(launch && grid && block, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  memcpy(launch->grid, grid, sizeof(launch->grid));
  memcpy(launch->block, block, sizeof(launch->block));
  launch->smem = shared_mem_bytes;
  launch->configured = true;
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_launch_execute(cutile_launch_t launch, cutile_stream_t stream) {
  CUTILE_REQUIRE(launch, CUTILE_ERR_INVALID_ARGUMENT, "launch is null");
  CUTILE_REQUIRE(launch->configured, CUTILE_ERR_KERNEL_LAUNCH, "Launch grid required.");
  return launch_packed(launch->function, launch->grid, launch->block, launch->smem, stream, launch->args);
}

// ---- Part B: generic lookup ----------------------------------------------------------------
cutile_status_t cutile_kernel_lookup(cutile_device_t device, const char* function, const char* const* generics,
                                     int32_t n_generics, const char* variant, cutile_kernel_info_t* info) {
  CUTILE_REQUIRE(device && function && info, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  const KernelEntry* found = nullptr;
  std::string want = variant ? variant : preferred_variant(function);
  for (const auto& e : kernel_table()) {
    if (strcmp(e.function, function) != 0) continue;
    if (!want.empty()) {
      if (want == e.variant) { found = &e; break; }
      continue;
    }
    // Match on generics: a dtype string must equal the entry's dtype; integer
    // generics are compared against the entry's tile shape, in order.
    bool ok = true;
    int tile_i = 0;
    for (int i = 0; i < n_generics && ok; ++i) {
      const char* gstr = generics[i];
      if (!gstr) { ok = false; break; }
      if (cutile_dtype_from_name(gstr) != CUTILE_DTYPE_COUNT) {
        ok = strncmp(e.dtype, gstr, strlen(gstr)) == 0;
      } else if (tile_i < 3 && e.tile[tile_i] != 0) {
        ok = atoi(gstr) == e.tile[tile_i];
        ++tile_i;
      }
    }
    if (ok) { found = &e; break; }
  }
  if (!found) {
    std::string key;
    for (int i = 0; i < n_generics; ++i) key += std::string(i ? ", " : "") + (generics[i] ? generics[i] : "?");
    return fail(CUTILE_ERR_KERNEL_NOT_FOUND, "no precompiled variant of %s<%s>%s%s; available: %s", function,
                key.c_str(), want.empty() ? "" : " named ", want.c_str(), list_variants(function).c_str());
  }
  hipFunction_t fn = nullptr;
  if (cutile_status_t s = load_entry(device, found, &fn)) return s;
  info->function = fn;
  info->symbol = found->symbol;
  info->variant = found->variant;
  memcpy(info->block, found->block, sizeof(info->block));
  info->lds_bytes = found->lds_bytes;
  memcpy(info->tile, found->tile, sizeof(info->tile));
  return CUTILE_SUCCESS;
}

// ---- Part D: entry launchers ---------------------------------------------------------------
static cutile_status_t launch_elementwise3(const char* fn_name, cutile_stream_t stream,
                                           const cutile_partition_arg_t* out, const double* a,
                                           const cutile_tensor_arg_t* in0, const cutile_tensor_arg_t* in1,
                                           bool in_place, const cutile_launch_opts_t* opts) {
  // out <- f(in0, in1) (or f(a, in0, in1)).  For the in-place saxpy, in1 is null
  // and the second operand is `out` itself.
  if (cutile_status_t s = check_partition(out, "output", 1, 2)) return s;
  const cutile_tensor_arg_t& ot = out->tensor;
  const int rank = ot.rank;
  if (cutile_status_t s = check_tensor(in0, "x", rank, rank)) return s;
  if (in1)
    if (cutile_status_t s = check_tensor(in1, "y", rank, rank)) return s;
  CUTILE_REQUIRE(in0->dtype == ot.dtype && (!in1 || in1->dtype == ot.dtype), CUTILE_ERR_KERNEL_LAUNCH,
                 "%s: all operands must have element type %s", fn_name, cutile_dtype_name(ot.dtype));
  const std::string dt = cutile_dtype_name(ot.dtype);
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(out, opts, tg)) return s;
  uint32_t full[3];
  cutile_partition_grid(out, full);
  const bool full_cover = tg[0] == full[0] && tg[1] == full[1] && tg[2] == full[2];

  bool flat_ok = is_contiguous(ot) && is_contiguous(*in0) && same_shape(ot, *in0) && aligned16(ot.ptr) &&
                 aligned16(in0->ptr) && (rank == 1 || full_cover);
  if (in1) flat_ok = flat_ok && is_contiguous(*in1) && same_shape(ot, *in1) && aligned16(in1->ptr);
  const std::string r = "_r" + std::to_string(rank);
  std::vector<std::string> acceptable;
  if (flat_ok && find_entry(fn_name, dt + r + "_flat")) acceptable.push_back(dt + r + "_flat");
  if (find_entry(fn_name, dt + r + "_tiled")) acceptable.push_back(dt + r + "_tiled");
  CUTILE_REQUIRE(!acceptable.empty(), CUTILE_ERR_KERNEL_NOT_FOUND, "no precompiled variant of %s<%s> for rank %d; available: %s",
                 fn_name, dt.c_str(), rank, list_variants(fn_name).c_str());
  Resolved res;
  BucketScope bucket(dt + r);
  if (cutile_status_t s = resolve_entry(fn_name, opts, acceptable[0], acceptable, &res)) return s;

  ArgPacker args;
  args.push_partition(*out);
  if (a) {
    unsigned char bits[8];
    size_t n = scalar_bits(ot.dtype, *a, (int64_t)*a, bits);
    args.push(bits, n, n);
  }
  args.push_tensor(*in0);
  if (in1) args.push_tensor(*in1);
  args.push_tile_grid(tg);

  uint32_t grid[3] = {tg[0], tg[1], tg[2]};
  if (strstr(res.entry->variant, "_flat")) {
    uint64_t count = rank == 1 ? std::min<uint64_t>((uint64_t)tg[0] * out->partition_shape[0], ot.shape[0]) : (uint64_t)numel(ot);
    uint64_t per_wg = 256ull * 4ull * (16 / cutile_dtype_size(ot.dtype));
    grid[0] = std::max<uint32_t>(1, div_up(count, per_wg));
    grid[1] = grid[2] = 1;
  }
  (void)in_place;
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

cutile_status_t cutile_launch_saxpy(cutile_stream_t stream, const cutile_partition_arg_t* y, double a,
                                    const cutile_tensor_arg_t* x, const cutile_launch_opts_t* opts) {
  return launch_elementwise3("saxpy", stream, y, &a, x, nullptr, true, opts);
}
cutile_status_t cutile_launch_axpy(cutile_stream_t stream, const cutile_partition_arg_t* z, double a,
                                   const cutile_tensor_arg_t* x, const cutile_tensor_arg_t* y,
                                   const cutile_launch_opts_t* opts) {
  CUTILE_REQUIRE(z && z->tensor.rank == 1, CUTILE_ERR_KERNEL_LAUNCH, "axpy: output must be rank 1");
  return launch_elementwise3("axpy", stream, z, &a, x, y, false, opts);
}
// add_2d_f16 / silu_mul_2d_f16: rank-2 f16, output tiles [1, BLOCK_SIZE].
static cutile_status_t launch_pointwise_2d_f16(const char* name, const char* kernel, cutile_stream_t stream,
                                               const cutile_partition_arg_t* out, const cutile_tensor_arg_t* a,
                                               const cutile_tensor_arg_t* b, const cutile_launch_opts_t* opts) {
  CUTILE_REQUIRE(out && out->tensor.rank == 2 && out->tensor.dtype == CUTILE_DTYPE_F16 && out->partition_shape[0] == 1,
                 CUTILE_ERR_KERNEL_LAUNCH, "%s: out must be a rank-2 f16 tensor partitioned [1, BLOCK_SIZE]", name);
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(out->partition_shape[1]), "BLOCK_SIZE")) return s;
  cutile_launch_opts_t o = opts ? *opts : cutile_launch_opts_t{};
  o.generics = nullptr;   // validated above; the kernels themselves are keyed by the element type
  o.n_generics = 0;
  return launch_elementwise3(kernel, stream, out, nullptr, a, b, false, &o);
}
cutile_status_t cutile_launch_add_2d_f16(cutile_stream_t stream, const cutile_partition_arg_t* out,
                                         const cutile_tensor_arg_t* lhs, const cutile_tensor_arg_t* rhs,
                                         const cutile_launch_opts_t* opts) {
  return launch_pointwise_2d_f16("add_2d_f16", "add", stream, out, lhs, rhs, opts);
}
cutile_status_t cutile_launch_silu_mul_2d_f16(cutile_stream_t stream, const cutile_partition_arg_t* out,
                                              const cutile_tensor_arg_t* gate, const cutile_tensor_arg_t* up,
                                              const cutile_launch_opts_t* opts) {
  return launch_pointwise_2d_f16("silu_mul_2d_f16", "silu_mul_2d_f16", stream, out, gate, up, opts);
}
cutile_status_t cutile_launch_add(cutile_stream_t stream, const cutile_partition_arg_t* z, const cutile_tensor_arg_t* x,
                                  const cutile_tensor_arg_t* y, const cutile_launch_opts_t* opts) {
  CUTILE_REQUIRE(y, CUTILE_ERR_INVALID_ARGUMENT, "y is null");
  return launch_elementwise3("add", stream, z, nullptr, x, y, false, opts);
}

static cutile_status_t launch_creation(const char* fn_name, cutile_stream_t stream, const cutile_partition_arg_t* t,
                                       const unsigned char* scalar, size_t scalar_size, bool scalar_first,
                                       const float* extra_f32, int n_extra, const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_partition(t, "tensor", 1, 1)) return s;
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(t, opts, tg)) return s;
  const std::string dt = cutile_dtype_name(t->tensor.dtype);
  Resolved res;
  if (cutile_status_t s = resolve_entry(fn_name, opts, dt, {dt}, &res)) return s;
  ArgPacker args;
  if (scalar && scalar_first) args.push(scalar, scalar_size, scalar_size);
  args.push_partition(*t);
  for (int i = 0; i < n_extra; ++i) args.push_val<float>(extra_f32[i]);
  args.push_tile_grid(tg);
  uint64_t count = std::min<uint64_t>((uint64_t)tg[0] * t->partition_shape[0], t->tensor.shape[0]);
  uint32_t grid[3] = {std::min<uint32_t>(std::max<uint32_t>(1, div_up(count, 256 * 4)), 16384), 1, 1};
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

cutile_status_t cutile_launch_full(cutile_stream_t stream, double value, int64_t int_value,
                                   const cutile_partition_arg_t* t, const cutile_launch_opts_t* opts) {
  CUTILE_REQUIRE(t, CUTILE_ERR_INVALID_ARGUMENT, "tensor is null");
  unsigned char bits[8];
  size_t n = scalar_bits(t->tensor.dtype, value, int_value, bits);
  CUTILE_REQUIRE(n, CUTILE_ERR_KERNEL_NOT_FOUND, "full: unsupported element type %s", cutile_dtype_name(t->tensor.dtype));
  return launch_creation("full", stream, t, bits, n, true, nullptr, 0, opts);
}
cutile_status_t cutile_launch_arange(cutile_stream_t stream, const cutile_partition_arg_t* t,
                                     const cutile_launch_opts_t* opts) {
  return launch_creation("arange", stream, t, nullptr, 0, false, nullptr, 0, opts);
}
cutile_status_t cutile_launch_eye(cutile_stream_t stream, const cutile_partition_arg_t* t, const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_partition(t, "tensor", 2, 2)) return s;
  CUTILE_REQUIRE(t->tensor.dtype == CUTILE_DTYPE_F32, CUTILE_ERR_KERNEL_LAUNCH, "eye: tensor must be f32");
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(t->partition_shape[0]), "BR")) return s;
  if (cutile_status_t s = check_generic(opts, 1, std::to_string(t->partition_shape[1]), "BC")) return s;
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(t, opts, tg)) return s;
  Resolved res;
  if (cutile_status_t s = resolve_entry("eye", opts, "f32", {"f32"}, &res)) return s;
  ArgPacker args;
  args.push_partition(*t);
  args.push_tile_grid(tg);
  const uint64_t rows = std::min<uint64_t>((uint64_t)tg[0] * t->partition_shape[0], t->tensor.shape[0]);
  const uint64_t cols = std::min<uint64_t>((uint64_t)tg[1] * t->partition_shape[1], t->tensor.shape[1]);
  uint32_t grid[3] = {std::min<uint32_t>(std::max<uint32_t>(1, div_up(rows * cols, 256 * 4)), 16384), 1, 1};
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}
// ---- the example programs' small kernels ---------------------------------------------------
// grid of a flat f32 stream over `count` elements: a workgroup per 1024 vectors of 16 bytes (the kernels loop beyond 2^20 workgroups)
static void flat_f32_grid(uint64_t count, uint32_t grid[3]) {
  grid[0] = std::min<uint32_t>(std::max<uint32_t>(1, div_up(count, 256 * 4 * 4)), 1u << 20);
  grid[1] = grid[2] = 1;
}
cutile_status_t cutile_launch_relu(cutile_stream_t stream, const cutile_partition_arg_t* input_output,
                                   const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_partition(input_output, "input_output", 1, 1)) return s;
  CUTILE_REQUIRE(input_output->tensor.dtype == CUTILE_DTYPE_F32, CUTILE_ERR_KERNEL_LAUNCH, "relu: tensor must be f32");
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(input_output->partition_shape[0]), "D")) return s;
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(input_output, opts, tg)) return s;
  Resolved res;
  if (cutile_status_t s = resolve_entry("relu", opts, "f32", {"f32"}, &res)) return s;
  ArgPacker args;
  args.push_partition(*input_output);
  args.push_tile_grid(tg);
  uint32_t grid[3];
  flat_f32_grid(std::min<uint64_t>((uint64_t)tg[0] * input_output->partition_shape[0], input_output->tensor.shape[0]), grid);
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}
cutile_status_t cutile_launch_dropout(cutile_stream_t stream, float p, const cutile_tensor_arg_t* x,
                                      const cutile_tensor_arg_t* x_keep, const cutile_partition_arg_t* out,
                                      const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_tensor(x, "x", 1, 1)) return s;
  if (cutile_status_t s = check_tensor(x_keep, "x_keep", 1, 1)) return s;
  if (cutile_status_t s = check_partition(out, "out", 1, 1)) return s;
  CUTILE_REQUIRE(x->dtype == CUTILE_DTYPE_F32 && x_keep->dtype == CUTILE_DTYPE_F32 && out->tensor.dtype == CUTILE_DTYPE_F32,
                 CUTILE_ERR_KERNEL_LAUNCH, "dropout: x, x_keep and out must be f32");
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(out->partition_shape[0]), "S")) return s;
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(out, opts, tg)) return s;
  Resolved res;
  if (cutile_status_t s = resolve_entry("dropout", opts, "f32", {"f32"}, &res)) return s;
  ArgPacker args;
  args.push_val<float>(p);
  args.push_tensor(*x);
  args.push_tensor(*x_keep);
  args.push_partition(*out);
  args.push_tile_grid(tg);
  uint32_t grid[3];
  flat_f32_grid(std::min<uint64_t>((uint64_t)tg[0] * out->partition_shape[0], out->tensor.shape[0]), grid);
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}
cutile_status_t cutile_launch_scale_ptr(cutile_stream_t stream, void* out_ptr, const void* in_ptr, float scale, int32_t len,
                                        const cutile_launch_opts_t* opts) {
  CUTILE_REQUIRE(out_ptr && in_ptr, CUTILE_ERR_INVALID_ARGUMENT, "scale_ptr: null device pointer");
  // no partition argument to infer a grid from: the caller names it, as for every launcher of pointer arguments
  CUTILE_REQUIRE(opts && opts->grid[0] > 0 && opts->grid[1] > 0 && opts->grid[2] > 0, CUTILE_ERR_KERNEL_LAUNCH, "Launch grid required.");
  CUTILE_REQUIRE(len >= 0, CUTILE_ERR_KERNEL_LAUNCH, "scale_ptr: len must be non-negative");
  Resolved res;
  if (cutile_status_t s = resolve_entry("scale_ptr", opts, "f32", {"f32"}, &res)) return s;
  ArgPacker args;
  args.push_val<void*>(out_ptr);
  args.push_val<const void*>(in_ptr);
  args.push_val<float>(scale);
  args.push_val<int32_t>(len);
  uint32_t grid[3];
  flat_f32_grid((uint64_t)len, grid);
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}
cutile_status_t cutile_launch_matvec(cutile_stream_t stream, const cutile_partition_arg_t* z, const cutile_tensor_arg_t* x,
                                     const cutile_tensor_arg_t* y, int32_t k, const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_partition(z, "z", 1, 1)) return s;
  if (cutile_status_t s = check_tensor(x, "x", 2, 2)) return s;
  if (cutile_status_t s = check_tensor(y, "y", 1, 1)) return s;
  CUTILE_REQUIRE(z->tensor.dtype == CUTILE_DTYPE_F32 && x->dtype == CUTILE_DTYPE_F32 && y->dtype == CUTILE_DTYPE_F32,
                 CUTILE_ERR_KERNEL_LAUNCH, "matvec: z, x and y must be f32");
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(z->partition_shape[0]), "BM")) return s;
  const int bk = generic_int(opts, 1, 1);
  CUTILE_REQUIRE(bk > 0, CUTILE_ERR_KERNEL_LAUNCH, "matvec: BK must be positive");
  CUTILE_REQUIRE(k >= 0, CUTILE_ERR_KERNEL_LAUNCH, "matvec: k must be non-negative");
  if (cutile_status_t s = check_generic(opts, 2, std::to_string(k), "K")) return s;
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(z, opts, tg)) return s;
  Resolved res;
  if (cutile_status_t s = resolve_entry("matvec", opts, "f32", {"f32"}, &res)) return s;
  ArgPacker args;
  args.push_partition(*z);
  args.push_tensor(*x);
  args.push_tensor(*y);
  args.push_val<int32_t>((k / bk) * bk);   // the tile program runs k / BK whole K tiles
  args.push_tile_grid(tg);
  const uint64_t rows = std::min<uint64_t>((uint64_t)tg[0] * z->partition_shape[0], z->tensor.shape[0]);
  uint32_t grid[3] = {std::min<uint32_t>(std::max<uint32_t>(1, div_up(rows, 4)), 65536), 1, 1};   // one wavefront per row
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}
cutile_status_t cutile_launch_linspace(cutile_stream_t stream, const cutile_partition_arg_t* t, float start, float step,
                                       const cutile_launch_opts_t* opts) {
  CUTILE_REQUIRE(t && t->tensor.dtype == CUTILE_DTYPE_F32, CUTILE_ERR_KERNEL_LAUNCH, "linspace: tensor must be f32");
  float extra[2] = {start, step};
  return launch_creation("linspace", stream, t, nullptr, 0, false, extra, 2, opts);
}

cutile_status_t cutile_launch_convert(cutile_stream_t stream, const cutile_tensor_arg_t* src,
                                      const cutile_partition_arg_t* dst, const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_tensor(src, "src", 1, 1)) return s;
  if (cutile_status_t s = check_partition(dst, "dst", 1, 1)) return s;
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(dst, opts, tg)) return s;
  const std::string v = std::string(cutile_dtype_name(src->dtype)) + "_" + cutile_dtype_name(dst->tensor.dtype);
  Resolved res;
  if (cutile_status_t s = resolve_entry("convert", opts, v, {v}, &res)) return s;
  ArgPacker args;
  args.push_tensor(*src);
  args.push_partition(*dst);
  args.push_tile_grid(tg);
  uint64_t count = std::min<uint64_t>((uint64_t)tg[0] * dst->partition_shape[0], dst->tensor.shape[0]);
  uint32_t grid[3] = {std::min<uint32_t>(std::max<uint32_t>(1, div_up(count, 256 * 4)), 16384), 1, 1};
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

// Row-wise kernels: variants that hold a whole segment in registers, best first.
// Measured on MI355X: up to 4 vectors (64 bytes) per lane stream at full rate, so
// among those the smallest capacity wins and wider segments are split over more
// wavefronts; only segments too long for that take more vectors per lane.
static std::vector<std::string> fitting_row_variants(const char* fn_name, const std::string& prefix, int64_t seg_len) {
  std::vector<const KernelEntry*> fit;
  for (const auto& e : kernel_table())
    if (strcmp(e.function, fn_name) == 0 && e.capacity >= seg_len &&
        strncmp(e.variant, prefix.c_str(), prefix.size()) == 0)
      fit.push_back(&e);
  std::stable_sort(fit.begin(), fit.end(), [](const KernelEntry* a, const KernelEntry* b) {
    const int va = std::max(a->tile[2], 4), vb = std::max(b->tile[2], 4);
    if (va != vb) return va < vb;
    if (a->capacity != b->capacity) return a->capacity < b->capacity;
    return a->tile[3] < b->tile[3];  // fewer wavefronts per segment first
  });
  std::vector<std::string> names;
  for (auto* e : fit) names.push_back(e->variant);
  return names;
}

// Launch grid of a row-wise kernel over `segments` tile rows: register-resident
// variants take 4 / WPR segments per workgroup, the any-layout ones walk the
// segments with a grid stride.
static void row_launch_grid(const KernelEntry* e, uint64_t segments, uint32_t grid[3]) {
  grid[0] = grid[1] = grid[2] = 1;
  if (e->capacity <= 0)
    grid[0] = (uint32_t)std::min<uint64_t>(std::max<uint64_t>(segments, 1), 1u << 20);
  else if (e->tile[1] > 0)   // short-row variants: tile[1] rows per workgroup
    grid[0] = std::max<uint32_t>(1, div_up(segments, e->tile[1]));
  else
    grid[0] = std::max<uint32_t>(1, div_up(segments, 4 / e->tile[3]));
}

// RMSNorm moves every byte exactly once, and with all 8 workgroups a compute unit
// can hold resident far more rows are in flight than HBM needs, which costs
// bandwidth (measured: 3-6 % at N >= 8192).  Unused dynamic LDS caps residency at
// about 96 KiB of rows in flight per compute unit, never below 5 workgroups.
static uint32_t rms_norm_residency_lds(const KernelEntry* e, int32_t n) {
  if (e->capacity <= 0) return 0;
  const uint64_t bytes_per_wg = (uint64_t)(4 / e->tile[3]) * (uint64_t)n * 2;
  const uint64_t wgs = std::min<uint64_t>(8, std::max<uint64_t>(5, (96 * 1024 + bytes_per_wg / 2) / bytes_per_wg));
  if (wgs >= 8) return 0;
  return (uint32_t)(160 * 1024 / wgs - 1024);
}

cutile_status_t cutile_launch_rms_norm_f16(cutile_stream_t stream, const cutile_tensor_arg_t* x,
                                           const cutile_tensor_arg_t* w, const cutile_partition_arg_t* out, float eps,
                                           const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_tensor(x, "x", 2, 2)) return s;
  if (cutile_status_t s = check_tensor(w, "w", 1, 1)) return s;
  if (cutile_status_t s = check_partition(out, "out", 2, 2)) return s;
  const cutile_tensor_arg_t& ot = out->tensor;
  CUTILE_REQUIRE(x->dtype == CUTILE_DTYPE_F16 && w->dtype == CUTILE_DTYPE_F16 && ot.dtype == CUTILE_DTYPE_F16,
                 CUTILE_ERR_KERNEL_LAUNCH, "rms_norm_f16: x, w and out must be f16");
  const int32_t n = x->shape[1];
  // Signature: x [-1, N], w [N], out tiles [1, N].
  CUTILE_REQUIRE(w->shape[0] == n, CUTILE_ERR_KERNEL_LAUNCH, "rms_norm_f16: w has %d elements, expected N = %d", w->shape[0], n);
  CUTILE_REQUIRE(out->partition_shape[0] == 1 && out->partition_shape[1] == n, CUTILE_ERR_KERNEL_LAUNCH,
                 "rms_norm_f16: out must be partitioned [1, %d], got [%d, %d]", n, out->partition_shape[0],
                 out->partition_shape[1]);
  CUTILE_REQUIRE(ot.shape[1] == n && ot.shape[0] <= x->shape[0], CUTILE_ERR_KERNEL_LAUNCH,
                 "rms_norm_f16: out is [%d, %d] but x is [%d, %d]", ot.shape[0], ot.shape[1], x->shape[0], n);
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(n), "N")) return s;
  const int block = generic_int(opts, 1, 0);
  CUTILE_REQUIRE(block >= 0 && (block == 0 || n % block == 0), CUTILE_ERR_KERNEL_LAUNCH,
                 "rms_norm_f16: N = %d is not a multiple of BLOCK_SIZE = %d", n, block);
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(out, opts, tg)) return s;

  const bool vec_ok = n % 8 == 0 && x->strides[1] == 1 && ot.strides[1] == 1 && w->strides[0] == 1 &&
                      x->strides[0] % 8 == 0 && ot.strides[0] % 8 == 0 && aligned16(x->ptr) && aligned16(ot.ptr) &&
                      aligned16(w->ptr);
  std::vector<std::string> acceptable;
  if (vec_ok) acceptable = fitting_row_variants("rms_norm_f16", "", n);
  acceptable.push_back("generic");
  Resolved res;
  BucketScope bucket("n" + pow2_class(n));
  if (cutile_status_t s = resolve_entry("rms_norm_f16", opts, acceptable[0], acceptable, &res)) return s;

  ArgPacker args;
  args.push_tensor(*x);
  args.push_tensor(*w);
  args.push_partition(*out);
  args.push_val<float>(eps);
  args.push_tile_grid(tg);
  const uint64_t rows = std::min<uint64_t>(tg[0], ot.shape[0]);
  uint32_t grid[3];
  row_launch_grid(res.entry, rows, grid);
  return launch_packed(res.fn, grid, res.entry->block, rms_norm_residency_lds(res.entry, n), stream, args);
}

// rms_norm<N, BLOCK_SIZE> of cutile-examples/examples/rms_norm.rs:17-61: f32 throughout, square root rounded down.
cutile_status_t cutile_launch_rms_norm_f32(cutile_stream_t stream, const cutile_tensor_arg_t* x, const cutile_tensor_arg_t* w,
                                           const cutile_partition_arg_t* out, float eps, const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_tensor(x, "x", 2, 2)) return s;
  if (cutile_status_t s = check_tensor(w, "w", 1, 1)) return s;
  if (cutile_status_t s = check_partition(out, "out", 2, 2)) return s;
  const cutile_tensor_arg_t& ot = out->tensor;
  CUTILE_REQUIRE(x->dtype == CUTILE_DTYPE_F32 && w->dtype == CUTILE_DTYPE_F32 && ot.dtype == CUTILE_DTYPE_F32,
                 CUTILE_ERR_KERNEL_LAUNCH, "rms_norm: x, w and out must be f32");
  const int32_t n = x->shape[1];
  CUTILE_REQUIRE(w->shape[0] == n, CUTILE_ERR_KERNEL_LAUNCH, "rms_norm: w has %d elements, expected N = %d", w->shape[0], n);
  CUTILE_REQUIRE(out->partition_shape[0] == 1 && out->partition_shape[1] == n, CUTILE_ERR_KERNEL_LAUNCH,
                 "rms_norm: out must be partitioned [1, %d], got [%d, %d]", n, out->partition_shape[0], out->partition_shape[1]);
  CUTILE_REQUIRE(ot.shape[1] == n && ot.shape[0] <= x->shape[0], CUTILE_ERR_KERNEL_LAUNCH,
                 "rms_norm: out is [%d, %d] but x is [%d, %d]", ot.shape[0], ot.shape[1], x->shape[0], n);
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(n), "N")) return s;
  const int block = generic_int(opts, 1, 0);
  CUTILE_REQUIRE(block >= 0 && (block == 0 || n % block == 0), CUTILE_ERR_KERNEL_LAUNCH,
                 "rms_norm: N = %d is not a multiple of BLOCK_SIZE = %d", n, block);
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(out, opts, tg)) return s;
  cutile_launch_opts_t o = opts ? *opts : cutile_launch_opts_t{};
  o.generics = nullptr;
  o.n_generics = 0;
  Resolved res;
  if (cutile_status_t s = resolve_entry("rms_norm", &o, "f32", {"f32"}, &res)) return s;
  ArgPacker args;
  args.push_tensor(*x);
  args.push_tensor(*w);
  args.push_partition(*out);
  args.push_val<float>(eps);
  args.push_tile_grid(tg);
  const uint64_t rows = std::min<uint64_t>(tg[0], ot.shape[0]);
  uint32_t grid[3] = {(uint32_t)std::min<uint64_t>(std::max<uint64_t>(rows, 1), 1u << 20), 1, 1};
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

// rms_norm<N, BLOCK_SIZE> of cutile-benchmarks/benches/rmsnorm.rs:20-66: every operation in f16.  One wavefront per
// row, BLOCK_SIZE / 64 tile lanes per lane; the tile's reduce_sum is the stride-halving tree over BLOCK_SIZE lanes.
static bool is_pow2(int64_t v) { return v > 0 && (v & (v - 1)) == 0; }
cutile_status_t cutile_launch_rms_norm_all_f16(cutile_stream_t stream, const cutile_tensor_arg_t* x, const cutile_tensor_arg_t* w,
                                               const cutile_partition_arg_t* out, float eps, const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_tensor(x, "x", 2, 2)) return s;
  if (cutile_status_t s = check_tensor(w, "w", 1, 1)) return s;
  if (cutile_status_t s = check_partition(out, "out", 2, 2)) return s;
  const cutile_tensor_arg_t& ot = out->tensor;
  CUTILE_REQUIRE(x->dtype == CUTILE_DTYPE_F16 && w->dtype == CUTILE_DTYPE_F16 && ot.dtype == CUTILE_DTYPE_F16,
                 CUTILE_ERR_KERNEL_LAUNCH, "rms_norm_all_f16: x, w and out must be f16");
  const int32_t n = x->shape[1];
  CUTILE_REQUIRE(w->shape[0] == n, CUTILE_ERR_KERNEL_LAUNCH, "rms_norm_all_f16: w has %d elements, expected N = %d", w->shape[0], n);
  CUTILE_REQUIRE(out->partition_shape[0] == 1 && out->partition_shape[1] == n, CUTILE_ERR_KERNEL_LAUNCH,
                 "rms_norm_all_f16: out must be partitioned [1, %d], got [%d, %d]", n, out->partition_shape[0],
                 out->partition_shape[1]);
  CUTILE_REQUIRE(ot.shape[1] == n && ot.shape[0] <= x->shape[0], CUTILE_ERR_KERNEL_LAUNCH,
                 "rms_norm_all_f16: out is [%d, %d] but x is [%d, %d]", ot.shape[0], ot.shape[1], x->shape[0], n);
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(n), "N")) return s;
  const int block = generic_int(opts, 1, 0);
  CUTILE_REQUIRE(block > 0, CUTILE_ERR_KERNEL_LAUNCH,
                 "rms_norm_all_f16: the generics [N, BLOCK_SIZE] are required (BLOCK_SIZE is the width of the f16 accumulator tile)");
  CUTILE_REQUIRE(is_pow2(block) && block <= 1024 && n >= block && n % block == 0, CUTILE_ERR_KERNEL_NOT_FOUND,
                 "rms_norm_all_f16: BLOCK_SIZE = %d must be a power of two, at most 1024, that divides N = %d", block, n);
  const int v = std::max(1, block / 64);
  CUTILE_REQUIRE(x->strides[1] == 1 && ot.strides[1] == 1 && w->strides[0] == 1 && x->strides[0] % v == 0 && ot.strides[0] % v == 0 &&
                     ((uintptr_t)x->ptr | (uintptr_t)ot.ptr | (uintptr_t)w->ptr) % (2 * (uintptr_t)std::min(v, 8)) == 0,
                 CUTILE_ERR_KERNEL_NOT_FOUND, "rms_norm_all_f16: rows must be contiguous and aligned to %d bytes", 2 * std::min(v, 8));
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(out, opts, tg)) return s;
  cutile_launch_opts_t o = opts ? *opts : cutile_launch_opts_t{};
  o.generics = nullptr;
  o.n_generics = 0;
  const std::string variant = "v" + std::to_string(v);
  Resolved res;
  if (cutile_status_t s = resolve_entry("rms_norm_all_f16", &o, variant, {variant}, &res)) return s;
  ArgPacker args;
  args.push_tensor(*x);
  args.push_tensor(*w);
  args.push_partition(*out);
  args.push_val<float>(eps);
  args.push_val<int32_t>(block);
  args.push_tile_grid(tg);
  const uint64_t rows = std::min<uint64_t>(tg[0], ot.shape[0]);
  uint32_t grid[3] = {(uint32_t)std::min<uint64_t>(std::max<uint64_t>(div_up(rows, 4), 1), 1u << 20), 1, 1};
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

// softmax<BM, BN> of cutile-benchmarks/benches/softmax.rs:19-35: every operation in f16.  One wavefront per tile row.
cutile_status_t cutile_launch_softmax_all_f16(cutile_stream_t stream, const cutile_tensor_arg_t* x, const cutile_partition_arg_t* y,
                                              const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_tensor(x, "x", 2, 2)) return s;
  if (cutile_status_t s = check_partition(y, "y", 2, 2)) return s;
  const cutile_tensor_arg_t& yt = y->tensor;
  CUTILE_REQUIRE(x->dtype == CUTILE_DTYPE_F16 && yt.dtype == CUTILE_DTYPE_F16, CUTILE_ERR_KERNEL_LAUNCH,
                 "softmax_all_f16: x and y must be f16");
  const int32_t bm = y->partition_shape[0], bn = y->partition_shape[1];
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(bm), "BM")) return s;
  if (cutile_status_t s = check_generic(opts, 1, std::to_string(bn), "BN")) return s;
  CUTILE_REQUIRE(is_pow2(bn) && bn <= 16384, CUTILE_ERR_KERNEL_NOT_FOUND,
                 "softmax_all_f16: BN = %d must be a power of two, at most 16384 (the row is held in one wavefront's registers)", bn);
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(y, opts, tg)) return s;
  const uint64_t rows = std::min<uint64_t>((uint64_t)tg[0] * bm, yt.shape[0]);
  const int v = bn >= 512 ? 8 : std::max(1, bn / 64), ch = bn >= 512 ? bn / 512 : 1;
  CUTILE_REQUIRE(x->shape[1] == yt.shape[1] && (uint64_t)x->shape[0] >= rows, CUTILE_ERR_KERNEL_LAUNCH,
                 "softmax_all_f16: x is [%d, %d] but y is [%d, %d]", x->shape[0], x->shape[1], yt.shape[0], yt.shape[1]);
  CUTILE_REQUIRE(x->strides[1] == 1 && yt.strides[1] == 1 && x->strides[0] % v == 0 && yt.strides[0] % v == 0 &&
                     ((uintptr_t)x->ptr | (uintptr_t)yt.ptr) % (2 * (uintptr_t)v) == 0,
                 CUTILE_ERR_KERNEL_NOT_FOUND, "softmax_all_f16: rows must be contiguous and aligned to %d bytes", 2 * v);
  cutile_launch_opts_t o = opts ? *opts : cutile_launch_opts_t{};
  o.generics = nullptr;
  o.n_generics = 0;
  const std::string variant = "c" + std::to_string(ch) + "v" + std::to_string(v);
  Resolved res;
  if (cutile_status_t s = resolve_entry("softmax_all_f16", &o, variant, {variant}, &res)) return s;
  ArgPacker args;
  args.push_tensor(*x);
  args.push_partition(*y);
  args.push_tile_grid(tg);
  const uint64_t segments = rows * tg[1];
  uint32_t grid[3] = {(uint32_t)std::min<uint64_t>(std::max<uint64_t>(div_up(segments, 4), 1), 1u << 20), 1, 1};
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

// The two fused row norms: same shape rules and variant choice as rms_norm_f16.
static cutile_status_t launch_fused_norm(const char* fn, cutile_stream_t stream, const cutile_tensor_arg_t* a,
                                         const cutile_tensor_arg_t* b, const cutile_tensor_arg_t* w,
                                         const cutile_tensor_arg_t* w2, const cutile_partition_arg_t* out,
                                         const cutile_partition_arg_t* out2, float eps, const int32_t* num_q_rows,
                                         const cutile_launch_opts_t* opts) {
  const bool qk = num_q_rows != nullptr;
  if (cutile_status_t s = check_tensor(a, qk ? "q" : "residual", 2, 2)) return s;
  if (cutile_status_t s = check_tensor(b, qk ? "k" : "x", 2, 2)) return s;
  if (cutile_status_t s = check_tensor(w, qk ? "q_weight" : "w", 1, 1)) return s;
  if (w2)
    if (cutile_status_t s = check_tensor(w2, "k_weight", 1, 1)) return s;
  if (cutile_status_t s = check_partition(out, "out", 2, 2)) return s;
  if (out2)
    if (cutile_status_t s = check_partition(out2, "residual_out", 2, 2)) return s;
  const cutile_tensor_arg_t& ot = out->tensor;
  const int32_t n = a->shape[1];
  bool f16 = a->dtype == CUTILE_DTYPE_F16 && b->dtype == CUTILE_DTYPE_F16 && w->dtype == CUTILE_DTYPE_F16 &&
             ot.dtype == CUTILE_DTYPE_F16 && (!w2 || w2->dtype == CUTILE_DTYPE_F16) &&
             (!out2 || out2->tensor.dtype == CUTILE_DTYPE_F16);
  CUTILE_REQUIRE(f16, CUTILE_ERR_KERNEL_LAUNCH, "%s: every tensor must be f16", fn);
  CUTILE_REQUIRE(b->shape[1] == n && w->shape[0] == n && (!w2 || w2->shape[0] == n) && ot.shape[1] == n,
                 CUTILE_ERR_KERNEL_LAUNCH, "%s: row length N = %d must be shared by all tensors", fn, n);
  CUTILE_REQUIRE(out->partition_shape[0] == 1 && out->partition_shape[1] == n &&
                     (!out2 || (out2->partition_shape[0] == 1 && out2->partition_shape[1] == n)),
                 CUTILE_ERR_KERNEL_LAUNCH, "%s: outputs must be partitioned [1, %d]", fn, n);
  if (qk) {
    CUTILE_REQUIRE(*num_q_rows >= 0 && *num_q_rows <= a->shape[0] && ot.shape[0] <= *num_q_rows + b->shape[0],
                   CUTILE_ERR_KERNEL_LAUNCH, "%s: out has %d rows but q supplies %d (num_q_rows) and k %d", fn, ot.shape[0],
                   *num_q_rows, b->shape[0]);
  } else {
    CUTILE_REQUIRE(ot.shape[0] <= a->shape[0] && ot.shape[0] <= b->shape[0] && out2->tensor.shape[0] == ot.shape[0] &&
                       out2->tensor.shape[1] == n,
                   CUTILE_ERR_KERNEL_LAUNCH, "%s: out is [%d, %d] but residual is [%d, %d] and x [%d, %d]", fn, ot.shape[0],
                   ot.shape[1], a->shape[0], n, b->shape[0], n);
  }
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(n), "N")) return s;
  uint32_t tg[3];
  if (out2) {
    uint32_t explicit_grid[3] = {0, 0, 0};
    if (opts) memcpy(explicit_grid, opts->grid, sizeof(explicit_grid));
    const cutile_partition_arg_t* parts[2] = {out, out2};
    if (cutile_status_t s = cutile_infer_launch_grid(explicit_grid, parts, 2, tg)) return s;
  } else if (cutile_status_t s = resolve_grid(out, opts, tg)) {
    return s;
  }
  auto row_ok = [&](const cutile_tensor_arg_t& t) { return t.strides[1] == 1 && t.strides[0] % 8 == 0 && aligned16(t.ptr); };
  const bool vec_ok = n % 8 == 0 && row_ok(*a) && row_ok(*b) && row_ok(ot) && (!out2 || row_ok(out2->tensor)) &&
                      w->strides[0] == 1 && aligned16(w->ptr) && (!w2 || (w2->strides[0] == 1 && aligned16(w2->ptr)));
  std::vector<std::string> acceptable;
  if (vec_ok) acceptable = fitting_row_variants(fn, "", n);
  acceptable.push_back("generic");
  Resolved res;
  if (cutile_status_t s = resolve_entry(fn, opts, acceptable[0], acceptable, &res)) return s;
  ArgPacker args;
  args.push_tensor(*a);
  args.push_tensor(*b);
  args.push_tensor(*w);
  if (w2) args.push_tensor(*w2);
  args.push_partition(*out);
  if (out2) args.push_partition(*out2);
  args.push_val<float>(eps);
  if (qk) args.push_val<int32_t>(*num_q_rows);
  args.push_tile_grid(tg);
  const uint64_t rows = std::min<uint64_t>(tg[0], ot.shape[0]);
  uint32_t grid[3];
  row_launch_grid(res.entry, rows, grid);
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

cutile_status_t cutile_launch_add_rms_norm_f16(cutile_stream_t stream, const cutile_tensor_arg_t* residual,
                                               const cutile_tensor_arg_t* x, const cutile_tensor_arg_t* w,
                                               const cutile_partition_arg_t* out,
                                               const cutile_partition_arg_t* residual_out, float eps,
                                               const cutile_launch_opts_t* opts) {
  CUTILE_REQUIRE(residual_out, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  return launch_fused_norm("add_rms_norm_f16", stream, residual, x, w, nullptr, out, residual_out, eps, nullptr, opts);
}

// add_rms_norm_decode_raw_f16<N, BLOCK_SIZE> (cutile-kernels/src/experimental/norms.rs:22-153): add_rms_norm_f16 on one
// row of N halves given as raw device pointers (the reference assumes them 16-byte aligned).
cutile_status_t cutile_launch_add_rms_norm_decode_raw_f16(cutile_stream_t stream, const void* residual, const void* x,
                                                          const void* w, void* out, void* residual_out, float eps,
                                                          int32_t n, const cutile_launch_opts_t* opts) {
  CUTILE_REQUIRE(residual && x && w && out && residual_out, CUTILE_ERR_INVALID_ARGUMENT, "add_rms_norm_decode_raw_f16: null device pointer");
  CUTILE_REQUIRE(n > 0, CUTILE_ERR_KERNEL_LAUNCH, "add_rms_norm_decode_raw_f16: N must be positive");
  auto row = [&](const void* p) {
    cutile_tensor_arg_t t{};
    t.ptr = const_cast<void*>(p);
    t.dtype = CUTILE_DTYPE_F16;
    t.rank = 2;
    t.shape[0] = 1, t.shape[1] = n;
    t.strides[0] = n, t.strides[1] = 1;
    return t;
  };
  cutile_tensor_arg_t rt = row(residual), xt = row(x), wt{};
  wt.ptr = const_cast<void*>(w);
  wt.dtype = CUTILE_DTYPE_F16;
  wt.rank = 1;
  wt.shape[0] = n;
  wt.strides[0] = 1;
  auto part = [&](void* p) {
    cutile_partition_arg_t pa{};
    pa.tensor = row(p);
    pa.partition_shape[0] = 1, pa.partition_shape[1] = n;
    pa.partition_strides[0] = n, pa.partition_strides[1] = 1;
    return pa;
  };
  cutile_partition_arg_t op = part(out), rp = part(residual_out);
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(n), "N")) return s;
  cutile_launch_opts_t o = opts ? *opts : cutile_launch_opts_t{};
  o.generics = nullptr;
  o.n_generics = 0;
  return cutile_launch_add_rms_norm_f16(stream, &rt, &xt, &wt, &op, &rp, eps, &o);
}

cutile_status_t cutile_launch_qk_norm_f16(cutile_stream_t stream, const cutile_tensor_arg_t* q,
                                          const cutile_tensor_arg_t* k, const cutile_tensor_arg_t* q_weight,
                                          const cutile_tensor_arg_t* k_weight, const cutile_partition_arg_t* out,
                                          float eps, int32_t num_q_rows, const cutile_launch_opts_t* opts) {
  CUTILE_REQUIRE(k_weight, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  return launch_fused_norm("qk_norm_f16", stream, q, k, q_weight, k_weight, out, nullptr, eps, &num_q_rows, opts);
}

// Rotary embedding, all three reference forms: `k` may be null (rope_seq*), and
// the start position comes either by value or from one u32 in device memory.
cutile_status_t cutile_launch_rope_f16(cutile_stream_t stream, const cutile_tensor_arg_t* q,
                                       const cutile_tensor_arg_t* k, const cutile_tensor_arg_t* inv_freq,
                                       const cutile_tensor_arg_t* position_start_dev, int32_t position_start,
                                       const cutile_partition_arg_t* out, int32_t num_q_heads,
                                       const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_tensor(q, k ? "q" : "x", 3, 3)) return s;
  if (k)
    if (cutile_status_t s = check_tensor(k, "k", 3, 3)) return s;
  if (cutile_status_t s = check_tensor(inv_freq, "inv_freq", 1, 1)) return s;
  if (cutile_status_t s = check_partition(out, "out", 3, 3)) return s;
  const cutile_tensor_arg_t& ot = out->tensor;
  const int32_t d = q->shape[2], half = d / 2;
  CUTILE_REQUIRE(q->dtype == CUTILE_DTYPE_F16 && ot.dtype == CUTILE_DTYPE_F16 && (!k || k->dtype == CUTILE_DTYPE_F16) &&
                     inv_freq->dtype == CUTILE_DTYPE_F32,
                 CUTILE_ERR_KERNEL_LAUNCH, "rope: x / q / k / out must be f16 and inv_freq f32");
  CUTILE_REQUIRE(d % 2 == 0 && inv_freq->shape[0] == half && ot.shape[2] == d && (!k || k->shape[2] == d),
                 CUTILE_ERR_KERNEL_LAUNCH, "rope: head dimension D = %d needs inv_freq of D/2 = %d entries and matching tensors", d, half);
  CUTILE_REQUIRE(out->partition_shape[0] == 1 && out->partition_shape[1] == 1 && out->partition_shape[2] == half,
                 CUTILE_ERR_KERNEL_LAUNCH, "rope: out must be partitioned [1, 1, %d] (HALF_D), got [%d, %d, %d]", half,
                 out->partition_shape[0], out->partition_shape[1], out->partition_shape[2]);
  if (!k) num_q_heads = q->shape[1];
  CUTILE_REQUIRE(num_q_heads >= 0 && num_q_heads <= q->shape[1] && ot.shape[0] <= q->shape[0] &&
                     ot.shape[1] <= num_q_heads + (k ? k->shape[1] : 0) && (!k || ot.shape[0] <= k->shape[0]),
                 CUTILE_ERR_KERNEL_LAUNCH, "rope: out [%d, %d, %d] does not fit the inputs", ot.shape[0], ot.shape[1], ot.shape[2]);
  if (position_start_dev) {
    if (cutile_status_t s = check_tensor(position_start_dev, "position_start", 1, 1)) return s;
    CUTILE_REQUIRE(position_start_dev->dtype == CUTILE_DTYPE_U32 && position_start_dev->shape[0] == 1 &&
                       ((uintptr_t)position_start_dev->ptr & 3) == 0,
                   CUTILE_ERR_KERNEL_LAUNCH, "rope: position_start must be one aligned u32");
  }
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(d), "D")) return s;
  if (cutile_status_t s = check_generic(opts, 1, std::to_string(half), "HALF_D")) return s;
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(out, opts, tg)) return s;
  CUTILE_REQUIRE(tg[2] == 2, CUTILE_ERR_KERNEL_LAUNCH, "rope: the launch grid must cover both halves of D (grid.z = 2, got %u)", tg[2]);
  Resolved res;
  if (cutile_status_t s = resolve_entry("rope", opts, "f16", {"f16"}, &res)) return s;
  ArgPacker args;
  args.push_tensor(*q);
  args.push_tensor(k ? *k : *q);
  args.push_tensor(*inv_freq);
  args.push_val<const void*>(position_start_dev ? position_start_dev->ptr : nullptr);
  args.push_partition(*out);
  args.push_val<int32_t>(position_start);
  args.push_val<int32_t>(num_q_heads);
  args.push_tile_grid(tg);
  // one workgroup per sequence position (it computes that position's angles once)
  uint32_t grid[3] = {std::max<uint32_t>(1, std::min<uint32_t>(std::min<uint32_t>(tg[0], ot.shape[0]), 1u << 20)), 1, 1};
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

// kv_cache_update_seq_f16 / kv_cache_update_seq_dynpos_f16: the start position by value or from device memory.
cutile_status_t cutile_launch_kv_cache_update_f16(cutile_stream_t stream, const cutile_tensor_arg_t* new_k,
                                                  const cutile_tensor_arg_t* new_v, const cutile_partition_arg_t* k_cache,
                                                  const cutile_partition_arg_t* v_cache,
                                                  const cutile_tensor_arg_t* position_start_dev, int32_t position_start,
                                                  int32_t seq_len, const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_tensor(new_k, "new_k", 3, 3)) return s;
  if (cutile_status_t s = check_tensor(new_v, "new_v", 3, 3)) return s;
  if (cutile_status_t s = check_partition(k_cache, "k_cache", 3, 3)) return s;
  if (cutile_status_t s = check_partition(v_cache, "v_cache", 3, 3)) return s;
  const cutile_tensor_arg_t& kc = k_cache->tensor;
  const cutile_tensor_arg_t& vc = v_cache->tensor;
  const int32_t d = new_k->shape[2];
  CUTILE_REQUIRE(new_k->dtype == CUTILE_DTYPE_F16 && new_v->dtype == CUTILE_DTYPE_F16 && kc.dtype == CUTILE_DTYPE_F16 &&
                     vc.dtype == CUTILE_DTYPE_F16,
                 CUTILE_ERR_KERNEL_LAUNCH, "kv_cache_update: every tensor must be f16");
  CUTILE_REQUIRE(new_v->shape[2] == d && kc.shape[2] == d && vc.shape[2] == d && new_v->shape[0] == new_k->shape[0] &&
                     new_v->shape[1] == new_k->shape[1] && vc.shape[0] == kc.shape[0] && kc.shape[0] <= new_k->shape[1],
                 CUTILE_ERR_KERNEL_LAUNCH, "kv_cache_update: new_k/new_v [seq, heads, D] and the caches [heads, max_seq, D] do not agree");
  CUTILE_REQUIRE(seq_len >= 0 && seq_len <= new_k->shape[0], CUTILE_ERR_KERNEL_LAUNCH,
                 "kv_cache_update: seq_len = %d but new_k holds %d positions", seq_len, new_k->shape[0]);
  const int32_t block = k_cache->partition_shape[2];
  CUTILE_REQUIRE(k_cache->partition_shape[0] == 1 && v_cache->partition_shape[0] == 1 && block > 0 && d % block == 0 &&
                     v_cache->partition_shape[1] == k_cache->partition_shape[1] && v_cache->partition_shape[2] == block,
                 CUTILE_ERR_KERNEL_LAUNCH, "kv_cache_update: caches must be partitioned [1, rows, BLOCK_SIZE] with BLOCK_SIZE dividing D = %d", d);
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(d), "D")) return s;
  if (cutile_status_t s = check_generic(opts, 1, std::to_string(block), "BLOCK_SIZE")) return s;
  uint32_t explicit_grid[3] = {0, 0, 0};
  if (opts) memcpy(explicit_grid, opts->grid, sizeof(explicit_grid));
  const cutile_partition_arg_t* parts[2] = {k_cache, v_cache};
  uint32_t tg[3];
  if (cutile_status_t s = cutile_infer_launch_grid(explicit_grid, parts, 2, tg)) return s;
  CUTILE_REQUIRE((int64_t)tg[2] * block >= d, CUTILE_ERR_KERNEL_LAUNCH, "kv_cache_update: the launch grid must cover all of D");
  if (position_start_dev) {
    if (cutile_status_t s = check_tensor(position_start_dev, "position_start", 1, 1)) return s;
    CUTILE_REQUIRE(position_start_dev->dtype == CUTILE_DTYPE_U32 && position_start_dev->shape[0] == 1 &&
                       ((uintptr_t)position_start_dev->ptr & 3) == 0,
                   CUTILE_ERR_KERNEL_LAUNCH, "kv_cache_update: position_start must be one aligned u32");
  } else {
    // kv_cache.rs:27 "_position_start ... asserted == 0 at call site": the prefill form writes rows 0..seq_len
    CUTILE_REQUIRE(position_start == 0, CUTILE_ERR_KERNEL_LAUNCH,
                   "kv_cache_update_seq_f16 writes cache rows 0..seq_len; position_start must be 0 (got %d), use the "
                   "device-position form for other offsets", position_start);
    CUTILE_REQUIRE((int64_t)seq_len <= std::min(kc.shape[1], vc.shape[1]) &&
                       (int64_t)seq_len <= (int64_t)tg[1] * k_cache->partition_shape[1],
                   CUTILE_ERR_KERNEL_LAUNCH, "kv_cache_update: %d rows do not fit the cache rows the launch covers", seq_len);
  }
  Resolved res;
  if (cutile_status_t s = resolve_entry("kv_cache_update", opts, "f16", {"f16"}, &res)) return s;
  ArgPacker args;
  args.push_tensor(*new_k);
  args.push_tensor(*new_v);
  args.push_partition(*k_cache);
  args.push_partition(*v_cache);
  args.push_val<const void*>(position_start_dev ? position_start_dev->ptr : nullptr);
  args.push_val<int32_t>(position_start);
  args.push_val<int32_t>(seq_len);
  args.push_tile_grid(tg);
  const uint64_t lanes = (uint64_t)seq_len * std::min<uint32_t>(tg[0], kc.shape[0]) * std::max(1, d / 8);
  uint32_t grid[3] = {std::max<uint32_t>(1, std::min<uint32_t>(div_up(lanes, 256), 1u << 16)), 1, 1};
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

// ---- greedy sampling and row gathers (cutile-kernels/src/argmax.rs, embeddings.rs, pointwise.rs:86-99) ----
// block_max / block_idx: rank-1 f32 / u32 outputs with tiles [1], one tile block per block.
static cutile_status_t argmax_outputs_grid(const char* fn, const cutile_partition_arg_t* block_max,
                                           const cutile_partition_arg_t* block_idx, const cutile_launch_opts_t* opts,
                                           uint32_t tg[3]) {
  if (cutile_status_t s = check_partition(block_max, "block_max", 1, 1)) return s;
  if (cutile_status_t s = check_partition(block_idx, "block_idx", 1, 1)) return s;
  CUTILE_REQUIRE(block_max->tensor.dtype == CUTILE_DTYPE_F32 && block_idx->tensor.dtype == CUTILE_DTYPE_U32 &&
                     block_max->partition_shape[0] == 1 && block_idx->partition_shape[0] == 1,
                 CUTILE_ERR_KERNEL_LAUNCH, "%s: block_max must be f32 and block_idx u32, both partitioned [1]", fn);
  uint32_t explicit_grid[3] = {0, 0, 0};
  if (opts) memcpy(explicit_grid, opts->grid, sizeof(explicit_grid));
  const cutile_partition_arg_t* parts[2] = {block_max, block_idx};
  return cutile_infer_launch_grid(explicit_grid, parts, 2, tg);
}

cutile_status_t cutile_launch_argmax_blocks_f16(cutile_stream_t stream, const cutile_tensor_arg_t* logits,
                                                const cutile_partition_arg_t* block_max,
                                                const cutile_partition_arg_t* block_idx, int32_t len,
                                                const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_tensor(logits, "logits", 1, 1)) return s;
  CUTILE_REQUIRE(logits->dtype == CUTILE_DTYPE_F16, CUTILE_ERR_KERNEL_LAUNCH, "argmax_blocks_f16: logits must be f16");
  uint32_t tg[3];
  if (cutile_status_t s = argmax_outputs_grid("argmax_blocks_f16", block_max, block_idx, opts, tg)) return s;
  const int block_size = generic_int(opts, 0, 1024);
  CUTILE_REQUIRE(block_size > 0 && len >= 0, CUTILE_ERR_KERNEL_LAUNCH, "argmax_blocks_f16: BLOCK_SIZE must be positive and len non-negative");
  Resolved res;
  if (cutile_status_t s = resolve_entry("argmax_blocks", opts, "f16", {"f16"}, &res)) return s;
  ArgPacker args;
  args.push_tensor(*logits);
  args.push_partition(*block_max);
  args.push_partition(*block_idx);
  args.push_val<int32_t>(len);
  args.push_val<int32_t>(block_size);
  args.push_tile_grid(tg);
  uint32_t grid[3] = {tg[0], 1, 1};
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

cutile_status_t cutile_launch_lm_head_argmax_blocks_f16(cutile_stream_t stream, const cutile_tensor_arg_t* weights,
                                                        const cutile_tensor_arg_t* hidden,
                                                        const cutile_partition_arg_t* block_max,
                                                        const cutile_partition_arg_t* block_idx, int32_t vocab_size,
                                                        const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_tensor(weights, "weights", 2, 2)) return s;
  if (cutile_status_t s = check_tensor(hidden, "hidden", 2, 2)) return s;
  const int32_t k = weights->shape[1];
  CUTILE_REQUIRE(weights->dtype == CUTILE_DTYPE_F16 && hidden->dtype == CUTILE_DTYPE_F16, CUTILE_ERR_KERNEL_LAUNCH,
                 "lm_head_argmax_blocks_f16: weights and hidden must be f16");
  CUTILE_REQUIRE(hidden->shape[0] == 1 && hidden->shape[1] == k, CUTILE_ERR_KERNEL_LAUNCH,
                 "lm_head_argmax_blocks_f16: weights are [%d, %d] but hidden is [%d, %d], expected [1, %d]", weights->shape[0], k,
                 hidden->shape[0], hidden->shape[1], k);
  // the tile program runs K / 32 whole tiles (argmax.rs:109-110)
  CUTILE_REQUIRE(k % 32 == 0, CUTILE_ERR_KERNEL_LAUNCH, "lm_head_argmax_blocks_f16: K = %d must be a multiple of 32", k);
  CUTILE_REQUIRE(k <= 30720, CUTILE_ERR_KERNEL_NOT_FOUND, "lm_head_argmax_blocks_f16: K = %d exceeds the 30720 the precompiled kernel keeps in LDS", k);
  CUTILE_REQUIRE(vocab_size >= 0, CUTILE_ERR_KERNEL_LAUNCH, "lm_head_argmax_blocks_f16: vocab_size must be non-negative");
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(k), "K")) return s;
  uint32_t tg[3];
  if (cutile_status_t s = argmax_outputs_grid("lm_head_argmax_blocks_f16", block_max, block_idx, opts, tg)) return s;
  Resolved res;
  if (cutile_status_t s = resolve_entry("lm_head_argmax_blocks", opts, "f16", {"f16"}, &res)) return s;
  ArgPacker args;
  args.push_tensor(*weights);
  args.push_tensor(*hidden);
  args.push_partition(*block_max);
  args.push_partition(*block_idx);
  args.push_val<int32_t>(vocab_size);
  args.push_tile_grid(tg);
  // two workgroups per compute unit, each walking a contiguous run of blocks
  cutile_device_t device = nullptr;
  if (cutile_status_t s = current_device(&device)) return s;
  int cus = 0;
  if (cutile_status_t s = compute_units(device, &cus)) return s;
  uint32_t grid[3] = {std::min(tg[0], (uint32_t)std::max(cus, 1) * 2u), 1, 1};
  return launch_packed(res.fn, grid, res.entry->block, (uint32_t)k * 2, stream, args);
}

cutile_status_t cutile_launch_argmax_reduce_blocks_to_u32(cutile_stream_t stream, const cutile_tensor_arg_t* block_max,
                                                          const cutile_tensor_arg_t* block_idx,
                                                          const cutile_partition_arg_t* out, int32_t num_blocks,
                                                          const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_tensor(block_max, "block_max", 1, 1)) return s;
  if (cutile_status_t s = check_tensor(block_idx, "block_idx", 1, 1)) return s;
  if (cutile_status_t s = check_partition(out, "out", 1, 1)) return s;
  CUTILE_REQUIRE(block_max->dtype == CUTILE_DTYPE_F32 && block_idx->dtype == CUTILE_DTYPE_U32 && out->tensor.dtype == CUTILE_DTYPE_U32,
                 CUTILE_ERR_KERNEL_LAUNCH, "argmax_reduce_blocks_to_u32: block_max is f32, block_idx and out are u32");
  CUTILE_REQUIRE(out->tensor.shape[0] == 1 && out->partition_shape[0] == 1 && ((uintptr_t)out->tensor.ptr & 3) == 0,
                 CUTILE_ERR_KERNEL_LAUNCH, "argmax_reduce_blocks_to_u32: out must be one u32 partitioned [1]");
  CUTILE_REQUIRE(num_blocks >= 0, CUTILE_ERR_KERNEL_LAUNCH, "argmax_reduce_blocks_to_u32: num_blocks must be non-negative");
  const int block_size = generic_int(opts, 0, std::max(256, (num_blocks + 255) / 256 * 256));
  CUTILE_REQUIRE(block_size > 0, CUTILE_ERR_KERNEL_LAUNCH, "argmax_reduce_blocks_to_u32: BLOCK_SIZE must be positive");
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(out, opts, tg)) return s;
  Resolved res;
  if (cutile_status_t s = resolve_entry("argmax_reduce_blocks", opts, "u32", {"u32"}, &res)) return s;
  ArgPacker args;
  args.push_tensor(*block_max);
  args.push_tensor(*block_idx);
  args.push_partition(*out);
  args.push_val<int32_t>(num_blocks);
  args.push_val<int32_t>(block_size);
  args.push_tile_grid(tg);
  uint32_t grid[3] = {1, 1, 1};
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

cutile_status_t cutile_launch_embedding_batch_f16(cutile_stream_t stream, const cutile_tensor_arg_t* token_ids,
                                                  const cutile_tensor_arg_t* table, const cutile_partition_arg_t* out,
                                                  const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_tensor(token_ids, "token_ids", 1, 1)) return s;
  if (cutile_status_t s = check_tensor(table, "table", 2, 2)) return s;
  if (cutile_status_t s = check_partition(out, "out", 2, 2)) return s;
  const cutile_tensor_arg_t& ot = out->tensor;
  CUTILE_REQUIRE(token_ids->dtype == CUTILE_DTYPE_U32 && table->dtype == CUTILE_DTYPE_F16 && ot.dtype == CUTILE_DTYPE_F16 &&
                     ((uintptr_t)token_ids->ptr & 3) == 0,
                 CUTILE_ERR_KERNEL_LAUNCH, "embedding_batch_f16: token_ids must be u32, table and out f16");
  const int32_t d = table->shape[1], block = out->partition_shape[1];
  CUTILE_REQUIRE(out->partition_shape[0] == 1 && ot.shape[1] == d && ot.shape[0] <= token_ids->shape[0], CUTILE_ERR_KERNEL_LAUNCH,
                 "embedding_batch_f16: out [%d, %d] tiles [%d, %d] must be [tokens <= %d, D = %d] partitioned [1, BLOCK_SIZE]",
                 ot.shape[0], ot.shape[1], out->partition_shape[0], block, token_ids->shape[0], d);
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(d), "D")) return s;
  if (cutile_status_t s = check_generic(opts, 1, std::to_string(block), "BLOCK_SIZE")) return s;
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(out, opts, tg)) return s;
  Resolved res;
  if (cutile_status_t s = resolve_entry("embedding_batch", opts, "f16", {"f16"}, &res)) return s;
  ArgPacker args;
  args.push_tensor(*token_ids);
  args.push_tensor(*table);
  args.push_partition(*out);
  args.push_tile_grid(tg);
  uint32_t grid[3] = {std::max<uint32_t>(1, std::min<uint32_t>(std::min<uint32_t>(tg[0], (uint32_t)ot.shape[0]), 1u << 20)), 1, 1};
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

cutile_status_t cutile_launch_gather_row_f16(cutile_stream_t stream, const cutile_tensor_arg_t* src,
                                             const cutile_partition_arg_t* out, int32_t row_idx,
                                             const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_tensor(src, "src", 2, 2)) return s;
  if (cutile_status_t s = check_partition(out, "out", 1, 1)) return s;
  CUTILE_REQUIRE(src->dtype == CUTILE_DTYPE_F16 && out->tensor.dtype == CUTILE_DTYPE_F16, CUTILE_ERR_KERNEL_LAUNCH,
                 "gather_row_f16: src and out must be f16");
  CUTILE_REQUIRE(row_idx >= 0, CUTILE_ERR_KERNEL_LAUNCH, "gather_row_f16: row_idx must be non-negative");
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(out->partition_shape[0]), "BLOCK_SIZE")) return s;
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(out, opts, tg)) return s;
  Resolved res;
  if (cutile_status_t s = resolve_entry("gather_row", opts, "f16", {"f16"}, &res)) return s;
  ArgPacker args;
  args.push_tensor(*src);
  args.push_partition(*out);
  args.push_val<int32_t>(row_idx);
  args.push_tile_grid(tg);
  const uint64_t width = std::min<uint64_t>((uint64_t)tg[0] * out->partition_shape[0], out->tensor.shape[0]);
  uint32_t grid[3] = {std::max<uint32_t>(1, std::min<uint32_t>(div_up(width, 256), 4096)), 1, 1};
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

// ---- fused Q/K norm + RoPE + KV-cache update (cutile-kernels/src/experimental/fused_transformer.rs) ----
static cutile_status_t launch_qk_norm_rope_kv(const char* name, cutile_stream_t stream, const void* q, const void* k, const void* v,
                                              const void* q_weight, const void* k_weight, const void* inv_freq, void* q_out,
                                              void* k_cache, void* v_cache, const void* pos_dev, float eps, int32_t position_start,
                                              int32_t seq_len, int32_t num_q_heads, int32_t num_kv_heads, int32_t d,
                                              int32_t max_seq, int64_t q_row_stride, int64_t kv_row_stride,
                                              const cutile_launch_opts_t* opts) {
  const void* ptrs[9] = {q, k, v, q_weight, k_weight, inv_freq, q_out, k_cache, v_cache};
  for (const void* p : ptrs) {
    CUTILE_REQUIRE(p, CUTILE_ERR_INVALID_ARGUMENT, "%s: null device pointer", name);
    CUTILE_REQUIRE(p == inv_freq ? ((uintptr_t)p & 3) == 0 : aligned16(p), CUTILE_ERR_KERNEL_LAUNCH,
                   "%s: device pointers must be 16-byte aligned (inv_freq: 4)", name);
  }
  CUTILE_REQUIRE(d > 0 && d % 16 == 0 && d <= 2048, CUTILE_ERR_KERNEL_NOT_FOUND,
                 "%s: D = %d must be a multiple of 16, at most 2048, with D/16 a power of two", name, d);
  CUTILE_REQUIRE(((d / 16) & (d / 16 - 1)) == 0 && d / 16 <= 64, CUTILE_ERR_KERNEL_NOT_FOUND,
                 "%s: D = %d must be a multiple of 16, at most 2048, with D/16 a power of two", name, d);
  CUTILE_REQUIRE(seq_len >= 0 && num_q_heads >= 0 && num_kv_heads >= 0 && max_seq > 0, CUTILE_ERR_KERNEL_LAUNCH,
                 "%s: seq_len, head counts must be non-negative and MAX_SEQ positive", name);
  if (!pos_dev)
    CUTILE_REQUIRE(position_start >= 0 && (int64_t)position_start + seq_len <= max_seq, CUTILE_ERR_KERNEL_LAUNCH,
                   "%s: positions %d .. %lld do not fit the %d rows of the caches", name, position_start,
                   (long long)position_start + seq_len, max_seq);
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(d), "D")) return s;
  if (cutile_status_t s = check_generic(opts, 1, std::to_string(d / 2), "HALF_D")) return s;
  if (cutile_status_t s = check_generic(opts, 2, std::to_string(max_seq), "MAX_SEQ")) return s;
  if (seq_len == 0 || num_q_heads + num_kv_heads == 0) return CUTILE_SUCCESS;
  cutile_launch_opts_t o = opts ? *opts : cutile_launch_opts_t{};
  o.generics = nullptr;
  o.n_generics = 0;
  Resolved res;
  if (cutile_status_t s = resolve_entry("qk_norm_rope_kv", &o, "f16", {"f16"}, &res)) return s;
  ArgPacker args;
  for (const void* p : ptrs) args.push_val<const void*>(p);
  args.push_val<const void*>(pos_dev);
  args.push_val<float>(eps);
  args.push_val<int32_t>(position_start);
  args.push_val<int32_t>(seq_len);
  args.push_val<int32_t>(num_q_heads);
  args.push_val<int32_t>(num_kv_heads);
  args.push_val<int32_t>(d);
  args.push_val<int32_t>(max_seq);
  args.push_val<int64_t>(q_row_stride);
  args.push_val<int64_t>(kv_row_stride);
  uint32_t grid[3] = {std::min<uint32_t>((uint32_t)seq_len, 1u << 20), 1, 1};   // one workgroup per position
  // lanes per workgroup: rows * D/16 lane slots per position; the size that idles the fewest lanes in the last pass
  const uint32_t lane_slots = (uint32_t)(num_q_heads + 2 * num_kv_heads) * (uint32_t)(d / 16);
  uint32_t block[3] = {256, 1, 1}, best_idle = UINT32_MAX;
  for (uint32_t b : {256u, 192u, 128u, 64u}) {
    const uint32_t idle = (lane_slots + b - 1) / b * b - lane_slots;
    if (idle < best_idle) best_idle = idle, block[0] = b;
  }
  return launch_packed(res.fn, grid, block, 0, stream, args);
}

cutile_status_t cutile_launch_qk_norm_rope_kv_prefill_raw_f16(cutile_stream_t stream, const void* q, const void* k,
                                                              const void* v, const void* q_weight, const void* k_weight,
                                                              const void* inv_freq, void* q_out, void* k_cache,
                                                              void* v_cache, float eps, int32_t position_start,
                                                              int32_t seq_len, int32_t num_q_heads, int32_t num_kv_heads,
                                                              int32_t d, int32_t max_seq, const cutile_launch_opts_t* opts) {
  return launch_qk_norm_rope_kv("qk_norm_rope_kv_prefill_raw_f16", stream, q, k, v, q_weight, k_weight, inv_freq, q_out, k_cache,
                                v_cache, nullptr, eps, position_start, seq_len, num_q_heads, num_kv_heads, d, max_seq,
                                (int64_t)num_q_heads * d, (int64_t)num_kv_heads * d, opts);
}

cutile_status_t cutile_launch_qk_norm_rope_kv_decode_raw_f16(cutile_stream_t stream, const void* qkv, const void* q_weight,
                                                             const void* k_weight, const void* inv_freq, void* q_out,
                                                             void* k_cache, void* v_cache,
                                                             const cutile_tensor_arg_t* position_start, float eps,
                                                             int32_t num_q_heads, int32_t num_kv_heads, int32_t d,
                                                             int32_t max_seq, const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_tensor(position_start, "position_start", 1, 1)) return s;
  CUTILE_REQUIRE(position_start->dtype == CUTILE_DTYPE_U32 && position_start->shape[0] == 1 && ((uintptr_t)position_start->ptr & 3) == 0,
                 CUTILE_ERR_KERNEL_LAUNCH, "qk_norm_rope_kv_decode_raw_f16: position_start must be one aligned u32");
  CUTILE_REQUIRE(qkv && num_q_heads >= 0 && num_kv_heads >= 0 && d > 0, CUTILE_ERR_INVALID_ARGUMENT,
                 "qk_norm_rope_kv_decode_raw_f16: null qkv or negative head count");
  const char* bytes = (const char*)qkv;
  const void* k = bytes + (size_t)num_q_heads * d * 2;
  const void* v = bytes + (size_t)(num_q_heads + num_kv_heads) * d * 2;
  return launch_qk_norm_rope_kv("qk_norm_rope_kv_decode_raw_f16", stream, qkv, k, v, q_weight, k_weight, inv_freq, q_out, k_cache,
                                v_cache, position_start->ptr, eps, 0, 1, num_q_heads, num_kv_heads, d, max_seq,
                                (int64_t)num_q_heads * d, (int64_t)num_kv_heads * d, opts);
}

// ---- KV block layout conversion (cutile-kernels/src/experimental/kvbm.rs) ----
static cutile_status_t launch_kvbm_copy(const char* name, cutile_stream_t stream, int32_t to_stacked, int32_t stacked_layout,
                                        int32_t contiguous_layout, int32_t num_blocks, const cutile_tensor_arg_t* stacked_tensors,
                                        const cutile_tensor_arg_t* contiguous_tensors, int32_t nh, int32_t nl, int32_t no, int32_t nt,
                                        int32_t hd, const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_tensor(stacked_tensors, "stacked_tensors", 1, 1)) return s;
  if (cutile_status_t s = check_tensor(contiguous_tensors, "contiguous_tensors", 1, 1)) return s;
  CUTILE_REQUIRE(num_blocks >= 0 && nh > 0 && nl > 0 && no > 0 && nt > 0 && hd > 0, CUTILE_ERR_KERNEL_LAUNCH,
                 "%s: num_blocks must be non-negative and the block extents positive", name);
  CUTILE_REQUIRE((stacked_layout == CUTILE_KVBM_STACKED_NHD || stacked_layout == CUTILE_KVBM_STACKED_HND) &&
                     (contiguous_layout == CUTILE_KVBM_UNIVERSAL ||
                      (stacked_layout == CUTILE_KVBM_STACKED_NHD && contiguous_layout == CUTILE_KVBM_OPERATIONAL_NHD) ||
                      (stacked_layout == CUTILE_KVBM_STACKED_HND && contiguous_layout == CUTILE_KVBM_OPERATIONAL_HND)),
                 CUTILE_ERR_KERNEL_LAUNCH, "unsupported KVBM %s layout map", to_stacked ? "contiguous-to-stacked" : "stacked-to-contiguous");
  const int64_t stacked_count = (int64_t)num_blocks * nl * no;
  CUTILE_REQUIRE(stacked_tensors->dtype == CUTILE_DTYPE_I64 && contiguous_tensors->dtype == CUTILE_DTYPE_I64 &&
                     stacked_tensors->strides[0] == 1 && contiguous_tensors->strides[0] == 1 &&
                     stacked_tensors->shape[0] >= stacked_count && contiguous_tensors->shape[0] >= num_blocks &&
                     (((uintptr_t)stacked_tensors->ptr | (uintptr_t)contiguous_tensors->ptr) & 7) == 0,
                 CUTILE_ERR_KERNEL_LAUNCH, "%s: the pointer tables must be dense aligned i64 tensors of %lld (stacked) and %d (contiguous) entries",
                 name, (long long)stacked_count, num_blocks);
  if (num_blocks == 0) return CUTILE_SUCCESS;
  Resolved res;
  if (cutile_status_t s = resolve_entry("kvbm_copy", nullptr, "f16", {"f16"}, &res)) return s;
  (void)opts;
  ArgPacker args;
  args.push_val<const void*>(stacked_tensors->ptr);
  args.push_val<const void*>(contiguous_tensors->ptr);
  args.push_val<int32_t>(to_stacked);
  args.push_val<int32_t>(stacked_layout == CUTILE_KVBM_STACKED_HND ? 1 : 0);
  args.push_val<int32_t>(contiguous_layout);
  args.push_val<int32_t>(num_blocks);
  args.push_val<int32_t>(nh);
  args.push_val<int32_t>(nl);
  args.push_val<int32_t>(no);
  args.push_val<int32_t>(nt);
  args.push_val<int32_t>(hd);
  const uint64_t lanes = (uint64_t)num_blocks * nh * nl * no * nt * (uint64_t)(hd % 8 == 0 ? hd / 8 : hd);
  uint32_t grid[3] = {std::max<uint32_t>(1, std::min<uint32_t>(div_up(lanes, 256 * 4), 1u << 16)), 1, 1};
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}
cutile_status_t cutile_launch_copy_stacked_to_contiguous_f16(cutile_stream_t stream, int32_t stacked_layout, int32_t contiguous_layout,
                                                             int32_t num_blocks, const cutile_tensor_arg_t* stacked_tensors,
                                                             const cutile_tensor_arg_t* contiguous_tensors, int32_t nh, int32_t nl,
                                                             int32_t no, int32_t nt, int32_t hd, const cutile_launch_opts_t* opts) {
  return launch_kvbm_copy("copy_stacked_to_contiguous_f16", stream, 0, stacked_layout, contiguous_layout, num_blocks, stacked_tensors,
                          contiguous_tensors, nh, nl, no, nt, hd, opts);
}
cutile_status_t cutile_launch_copy_contiguous_to_stacked_f16(cutile_stream_t stream, int32_t stacked_layout, int32_t contiguous_layout,
                                                             int32_t num_blocks, const cutile_tensor_arg_t* stacked_tensors,
                                                             const cutile_tensor_arg_t* contiguous_tensors, int32_t nh, int32_t nl,
                                                             int32_t no, int32_t nt, int32_t hd, const cutile_launch_opts_t* opts) {
  return launch_kvbm_copy("copy_contiguous_to_stacked_f16", stream, 1, stacked_layout, contiguous_layout, num_blocks, stacked_tensors,
                          contiguous_tensors, nh, nl, no, nt, hd, opts);
}

static bool decode_vec_layout(const cutile_tensor_arg_t& t) {
  return t.strides[2] == 1 && t.strides[1] % 8 == 0 && t.strides[0] % 8 == 0 && aligned16(t.ptr);
}

cutile_status_t cutile_launch_fmha_decode_gqa_split(cutile_stream_t stream, const cutile_tensor_arg_t* q,
                                                    const cutile_tensor_arg_t* k, const cutile_tensor_arg_t* v,
                                                    const cutile_partition_arg_t* att_out,
                                                    const cutile_partition_arg_t* lse_out, float qk_scale,
                                                    const cutile_tensor_arg_t* position_start,
                                                    const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_tensor(q, "q", 3, 3)) return s;
  if (cutile_status_t s = check_tensor(k, "k", 3, 3)) return s;
  if (cutile_status_t s = check_tensor(v, "v", 3, 3)) return s;
  if (cutile_status_t s = check_partition(att_out, "att_out", 3, 3)) return s;
  if (cutile_status_t s = check_partition(lse_out, "lse_out", 2, 2)) return s;
  if (cutile_status_t s = check_tensor(position_start, "position_start", 1, 1)) return s;
  const cutile_tensor_arg_t& at = att_out->tensor;
  const cutile_tensor_arg_t& lt = lse_out->tensor;
  const int32_t kv_heads = q->shape[0], group = q->shape[1], d = q->shape[2];
  CUTILE_REQUIRE(q->dtype == CUTILE_DTYPE_F16 && k->dtype == CUTILE_DTYPE_F16 && v->dtype == CUTILE_DTYPE_F16 &&
                     at.dtype == CUTILE_DTYPE_F16 && lt.dtype == CUTILE_DTYPE_F32 && position_start->dtype == CUTILE_DTYPE_U32,
                 CUTILE_ERR_KERNEL_LAUNCH, "fmha_decode_gqa_split: q, k, v, att_out are f16, lse_out f32, position_start u32");
  CUTILE_REQUIRE(k->shape[0] == kv_heads && v->shape[0] == kv_heads && k->shape[2] == d && v->shape[2] == d &&
                     at.shape[0] == kv_heads && at.shape[2] == d && lt.shape[0] == kv_heads && at.shape[1] == lt.shape[1] &&
                     at.shape[1] % group == 0 && position_start->shape[0] == 1,
                 CUTILE_ERR_KERNEL_LAUNCH, "fmha_decode_gqa_split: q [kv_heads, GROUP, D], k/v [kv_heads, max_seq, D], "
                 "att_out [kv_heads, NUM_KV_SPLITS*GROUP, D] and lse_out [kv_heads, NUM_KV_SPLITS*GROUP] do not agree");
  CUTILE_REQUIRE(att_out->partition_shape[0] == 1 && att_out->partition_shape[1] == group && att_out->partition_shape[2] == d &&
                     lse_out->partition_shape[0] == 1 && lse_out->partition_shape[1] == group,
                 CUTILE_ERR_KERNEL_LAUNCH, "fmha_decode_gqa_split: att_out must be partitioned [1, %d, %d] and lse_out [1, %d]", group, d, group);
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(group), "GROUP")) return s;
  if (cutile_status_t s = check_generic(opts, 2, std::to_string(d), "D")) return s;
  const int bn = generic_int(opts, 1, 64);
  CUTILE_REQUIRE(bn > 0, CUTILE_ERR_KERNEL_LAUNCH, "fmha_decode_gqa_split: BN must be positive");
  uint32_t explicit_grid[3] = {0, 0, 0};
  if (opts) memcpy(explicit_grid, opts->grid, sizeof(explicit_grid));
  const cutile_partition_arg_t* parts[2] = {att_out, lse_out};
  uint32_t tg[3];
  if (cutile_status_t s = cutile_infer_launch_grid(explicit_grid, parts, 2, tg)) return s;
  if (cutile_status_t s = check_generic(opts, 3, std::to_string(tg[1]), "NUM_KV_SPLITS")) return s;
  CUTILE_REQUIRE(decode_vec_layout(*q) && decode_vec_layout(*k) && decode_vec_layout(*v) && decode_vec_layout(at) &&
                     ((uintptr_t)position_start->ptr & 3) == 0 && ((uintptr_t)lt.ptr & 3) == 0,
                 CUTILE_ERR_KERNEL_NOT_FOUND, "fmha_decode_gqa_split: precompiled variants need unit head-dim stride and 16-byte aligned rows");
  // The matrix-core variant first: from GROUP 4 on the vector-ALU one no longer keeps up with HBM, and at D = 64 and
  // 256 it is the slower one for every group; only GROUP 1 and 2 at D = 128 measured (3 %) faster on the vector ALUs.
  const std::string plain = "f16_g" + std::to_string(group) + "_d" + std::to_string(d);
  std::vector<std::string> acceptable;
  const bool vector_first = group <= 2 && d == 128;
  for (const std::string& name : {vector_first ? plain : plain + "_mfma", vector_first ? plain + "_mfma" : plain})
    if (find_entry("fmha_decode_gqa_split", name)) acceptable.push_back(name);
  CUTILE_REQUIRE(!acceptable.empty(), CUTILE_ERR_KERNEL_NOT_FOUND,
                 "no precompiled variant of fmha_decode_gqa_split<GROUP=%d, D=%d>; available: %s", group, d,
                 list_variants("fmha_decode_gqa_split").c_str());
  Resolved res;
  if (cutile_status_t s = resolve_entry("fmha_decode_gqa_split", opts, acceptable[0], acceptable, &res)) return s;
  ArgPacker args;
  args.push_tensor(*q);
  args.push_tensor(*k);
  args.push_tensor(*v);
  args.push_partition(*att_out);
  args.push_partition(*lse_out);
  args.push_val<float>(qk_scale);
  args.push_val<const void*>(position_start->ptr);
  args.push_val<int32_t>(bn);
  args.push_tile_grid(tg);
  uint32_t grid[3] = {std::min<uint32_t>(tg[0], (uint32_t)kv_heads), tg[1], 1};
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

cutile_status_t cutile_launch_attention_decode_kernel_grouped_f16(
    cutile_stream_t stream, const void* q, const int32_t* q_shape, const int32_t* q_strides, const void* k,
    const int32_t* k_shape, const int32_t* k_strides, const void* v, const int32_t* v_shape, const int32_t* v_strides,
    void* att, const int32_t* att_shape, const int32_t* att_strides, void* lse, const int32_t* lse_shape,
    const int32_t* lse_strides, float softmax_scale, const void* s_kv, int32_t tile_n, int32_t kv_len_per_split,
    int32_t query_group_tile_size, const cutile_launch_opts_t* opts) {
  const char* fn = "attention_decode_kernel_grouped";
  CUTILE_REQUIRE(q && k && v && att && lse && s_kv && q_shape && q_strides && k_shape && k_strides && v_shape && v_strides &&
                     att_shape && att_strides && lse_shape && lse_strides,
                 CUTILE_ERR_INVALID_ARGUMENT, "%s: null argument", fn);
  for (int i = 0; i < 4; ++i)
    CUTILE_REQUIRE(q_shape[i] > 0 && k_shape[i] > 0 && v_shape[i] > 0 && lse_shape[i] > 0, CUTILE_ERR_TENSOR,
                   "%s: Shape dimensions must be positive.", fn);
  for (int i = 0; i < 5; ++i)
    CUTILE_REQUIRE(att_shape[i] > 0, CUTILE_ERR_TENSOR, "%s: Shape dimensions must be positive.", fn);
  const int32_t batch = q_shape[0], kv_heads = q_shape[1], group = q_shape[2], d = q_shape[3], splits = att_shape[3];
  CUTILE_REQUIRE(k_shape[0] == batch && k_shape[1] == kv_heads && k_shape[3] == d && v_shape[0] == batch && v_shape[1] == kv_heads &&
                     v_shape[3] == d && att_shape[0] == batch && att_shape[1] == kv_heads && att_shape[2] == group && att_shape[4] == d &&
                     lse_shape[0] == batch && lse_shape[1] == kv_heads && lse_shape[2] == group && lse_shape[3] == splits,
                 CUTILE_ERR_KERNEL_LAUNCH,
                 "%s: q [B, H_kv, G, D], k/v [B, H_kv, S, D], att [B, H_kv, G, NUM_KV_SPLITS, D] and lse [B, H_kv, G, NUM_KV_SPLITS] do not agree", fn);
  CUTILE_REQUIRE(tile_n > 0 && kv_len_per_split > 0 && query_group_tile_size >= group, CUTILE_ERR_KERNEL_LAUNCH,
                 "%s: TILE_N and KV_LEN_PER_SPLIT must be positive and QUERY_GROUP_TILE_SIZE (%d) at least NUM_Q_HEAD_PER_KV (%d)", fn,
                 query_group_tile_size, group);
  // with a remainder the tile program's splits overlap (its first tile is start / TILE_N rounded down, attention.rs:640-641)
  CUTILE_REQUIRE(kv_len_per_split % tile_n == 0, CUTILE_ERR_KERNEL_NOT_FOUND,
                 "%s: the precompiled kernels need KV_LEN_PER_SPLIT (%d) to be a multiple of TILE_N (%d)", fn, kv_len_per_split, tile_n);
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(d), "HEAD_DIM")) return s;
  if (cutile_status_t s = check_generic(opts, 1, std::to_string(tile_n), "TILE_N")) return s;
  if (cutile_status_t s = check_generic(opts, 2, std::to_string(kv_len_per_split), "KV_LEN_PER_SPLIT")) return s;
  if (cutile_status_t s = check_generic(opts, 3, std::to_string(group), "NUM_Q_HEAD_PER_KV")) return s;
  if (cutile_status_t s = check_generic(opts, 4, std::to_string(query_group_tile_size), "QUERY_GROUP_TILE_SIZE")) return s;
  if (cutile_status_t s = check_generic(opts, 5, std::to_string(splits), "NUM_KV_SPLITS")) return s;
  auto rows_ok = [&](const int32_t* strides, int n) {
    for (int i = 0; i < n; ++i)
      if (strides[i] < 0 || strides[i] % 8 != 0) return false;
    return true;
  };
  const int64_t v_extent = ((int64_t)(v_shape[2] - 1) * v_strides[2] + d) * 2;
  CUTILE_REQUIRE(rows_ok(q_strides, 3) && rows_ok(k_strides, 3) && rows_ok(v_strides, 3) && rows_ok(att_strides, 4) &&
                     lse_strides[0] >= 0 && lse_strides[1] >= 0 && lse_strides[2] >= 0 && aligned16(q) && aligned16(k) &&
                     aligned16(v) && aligned16(att) && ((uintptr_t)lse & 3) == 0 && ((uintptr_t)s_kv & 3) == 0 &&
                     v_extent <= 0xffffffffll,
                 CUTILE_ERR_KERNEL_NOT_FOUND,
                 "%s: precompiled variants need 16-byte aligned pointers, strides that are multiples of 8 elements and less than 4 GiB of V per head", fn);
  uint32_t tg[3] = {(uint32_t)batch, (uint32_t)kv_heads, (uint32_t)splits};
  if (opts && (opts->grid[0] || opts->grid[1] || opts->grid[2])) {
    CUTILE_REQUIRE(opts->grid[0] == tg[0] && opts->grid[1] == tg[1] && opts->grid[2] == tg[2], CUTILE_ERR_KERNEL_LAUNCH,
                   "%s: launch grid (%u, %u, %u) is not (batch, kv heads, NUM_KV_SPLITS) = (%u, %u, %u)", fn, opts->grid[0],
                   opts->grid[1], opts->grid[2], tg[0], tg[1], tg[2]);
  }
  const std::string name = "f16_g" + std::to_string(group) + "_d" + std::to_string(d);
  CUTILE_REQUIRE(find_entry(fn, name), CUTILE_ERR_KERNEL_NOT_FOUND,
                 "no precompiled variant of %s<NUM_Q_HEAD_PER_KV=%d, HEAD_DIM=%d>; available: %s", fn, group, d, list_variants(fn).c_str());
  Resolved res;
  if (cutile_status_t s = resolve_entry(fn, opts, name, {name}, &res)) return s;
  ArgPacker args;
  args.push_val<const void*>(q);
  args.push_val<const void*>(k);
  args.push_val<const void*>(v);
  args.push_val<void*>(att);
  args.push_val<void*>(lse);
  args.push_val<const void*>(s_kv);
  for (int i = 0; i < 3; ++i) args.push_val<int32_t>(q_strides[i]);
  for (int i = 0; i < 3; ++i) args.push_val<int32_t>(k_strides[i]);
  for (int i = 0; i < 3; ++i) args.push_val<int32_t>(v_strides[i]);
  for (int i = 0; i < 4; ++i) args.push_val<int32_t>(att_strides[i]);
  for (int i = 0; i < 3; ++i) args.push_val<int32_t>(lse_strides[i]);
  args.push_val<int32_t>(k_shape[2]);
  args.push_val<int32_t>(v_shape[2]);
  args.push_val<int32_t>(kv_len_per_split);
  args.push_val<float>(softmax_scale);
  args.push_tile_grid(tg);
  return launch_packed(res.fn, tg, res.entry->block, 0, stream, args);
}

cutile_status_t cutile_launch_splitk_reduce_merge(cutile_stream_t stream, const cutile_tensor_arg_t* att_partial,
                                                  const cutile_tensor_arg_t* lse_partial, const cutile_partition_arg_t* out,
                                                  const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_tensor(att_partial, "att_partial", 3, 3)) return s;
  if (cutile_status_t s = check_tensor(lse_partial, "lse_partial", 2, 2)) return s;
  if (cutile_status_t s = check_partition(out, "out", 3, 3)) return s;
  const cutile_tensor_arg_t& ot = out->tensor;
  const int32_t group = ot.shape[1], d = ot.shape[2];
  CUTILE_REQUIRE(att_partial->dtype == CUTILE_DTYPE_F16 && lse_partial->dtype == CUTILE_DTYPE_F32 && ot.dtype == CUTILE_DTYPE_F16,
                 CUTILE_ERR_KERNEL_LAUNCH, "splitk_reduce_merge: att_partial and out are f16, lse_partial f32");
  CUTILE_REQUIRE(group > 0 && att_partial->shape[0] >= ot.shape[0] && lse_partial->shape[0] >= ot.shape[0] &&
                     att_partial->shape[2] == d && att_partial->shape[1] == lse_partial->shape[1] &&
                     att_partial->shape[1] % group == 0 && att_partial->shape[1] >= group,
                 CUTILE_ERR_KERNEL_LAUNCH, "splitk_reduce_merge: att_partial [kv_heads, NUM_KV_SPLITS*GROUP, D], lse_partial "
                 "[kv_heads, NUM_KV_SPLITS*GROUP] and out [kv_heads, GROUP, D] do not agree");
  const int32_t chunk = out->partition_shape[2];
  CUTILE_REQUIRE(out->partition_shape[0] == 1 && out->partition_shape[1] == group && chunk > 0 && d % chunk == 0,
                 CUTILE_ERR_KERNEL_LAUNCH, "splitk_reduce_merge: out must be partitioned [1, %d, CHUNK_D] with CHUNK_D dividing D = %d", group, d);
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(group), "GROUP")) return s;
  if (cutile_status_t s = check_generic(opts, 1, std::to_string(d), "D")) return s;
  if (cutile_status_t s = check_generic(opts, 2, std::to_string(chunk), "CHUNK_D")) return s;
  if (cutile_status_t s = check_generic(opts, 3, std::to_string(att_partial->shape[1] / group), "NUM_KV_SPLITS")) return s;
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(out, opts, tg)) return s;
  CUTILE_REQUIRE((int64_t)tg[2] * chunk >= d, CUTILE_ERR_KERNEL_LAUNCH, "splitk_reduce_merge: the launch grid must cover all of D");
  Resolved res;
  if (cutile_status_t s = resolve_entry("splitk_reduce_merge", opts, "f16", {"f16"}, &res)) return s;
  ArgPacker args;
  args.push_tensor(*att_partial);
  args.push_tensor(*lse_partial);
  args.push_partition(*out);
  args.push_tile_grid(tg);
  // one workgroup per (KV head, query head of the group)
  uint32_t grid[3] = {std::min<uint32_t>(tg[0], (uint32_t)ot.shape[0]) * (uint32_t)group, 1, 1};
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

// ---- decode attention step that allocates nothing ----
// The partial results of the split kernel (att [kv_heads, NUM_KV_SPLITS*GROUP, D] f16 and lse [kv_heads,
// NUM_KV_SPLITS*GROUP] f32) live in the device-resident scratch array of scratch.hip instead of caller tensors.
// The side library that holds the array is opened on first use, after the HIP runtime is bound, so it attaches to the
// runtime this process already runs.
typedef int (*scratch_lookup_fn)(void**, size_t*, int*);
static std::mutex g_scratch_mutex;
static scratch_lookup_fn g_scratch_lookup = nullptr;
static std::string g_scratch_error;

static cutile_status_t scratch_memory(void** ptr, size_t* bytes) {
  if (cutile_status_t s = ensure_init()) return s;
  CUTILE_API_OR_RETURN(api);
  (void)api;
  scratch_lookup_fn fn;
  {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_lookup && g_scratch_error.empty()) {
      std::string path = CUTILE_SCRATCH_LIBRARY;
      Dl_info info;
      if (dladdr((const void*)&cutile_launch_fmha_decode_gqa_noalloc, &info) && info.dli_fname) {
        std::string self = info.dli_fname;
        size_t slash = self.rfind('/');
        if (slash != std::string::npos) path = self.substr(0, slash + 1) + CUTILE_SCRATCH_LIBRARY;
      }
      void* h = dlopen(path.c_str(), RTLD_NOW | RTLD_LOCAL);
      if (!h) {
        const char* e = dlerror();
        g_scratch_error = std::string("cannot load ") + path + ": " + (e ? e : "unknown");
      } else {
        g_scratch_lookup = (scratch_lookup_fn)dlsym(h, CUTILE_SCRATCH_LOOKUP_SYMBOL);
        if (!g_scratch_lookup) g_scratch_error = path + " lacks " CUTILE_SCRATCH_LOOKUP_SYMBOL;
      }
    }
    fn = g_scratch_lookup;
    if (!fn) return fail(CUTILE_ERR_LIBRARY_INIT, "shared object init failed: %s", g_scratch_error.c_str());
  }
  int ordinal = -1;
  const int err = fn(ptr, bytes, &ordinal);
  if (err != 0) return from_hip((hipError_t)err, "hipGetSymbolAddress(scratch)");
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_scratch_capacity(size_t* bytes) {
  CUTILE_REQUIRE(bytes, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  *bytes = CUTILE_SCRATCH_BYTES;
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_launch_fmha_decode_gqa_noalloc(cutile_stream_t stream, const cutile_tensor_arg_t* q,
                                                      const cutile_tensor_arg_t* k, const cutile_tensor_arg_t* v,
                                                      const cutile_partition_arg_t* out, float qk_scale,
                                                      const cutile_tensor_arg_t* position_start, int32_t num_kv_splits,
                                                      int32_t bn) {
  if (cutile_status_t s = check_tensor(q, "q", 3, 3)) return s;
  if (cutile_status_t s = check_partition(out, "out", 3, 3)) return s;
  const int32_t kv_heads = q->shape[0], group = q->shape[1], d = q->shape[2];
  CUTILE_REQUIRE(num_kv_splits > 0 && bn > 0, CUTILE_ERR_KERNEL_LAUNCH,
                 "fmha_decode_gqa_noalloc: NUM_KV_SPLITS and BN must be positive");
  CUTILE_REQUIRE(out->tensor.shape[0] == kv_heads && out->tensor.shape[1] == group && out->tensor.shape[2] == d,
                 CUTILE_ERR_KERNEL_LAUNCH, "fmha_decode_gqa_noalloc: out must be [kv_heads, GROUP, D] like q");
  // partials first, their log-sum-exp behind them on the next 256-byte boundary
  const uint64_t rows = (uint64_t)kv_heads * (uint64_t)num_kv_splits * (uint64_t)group;
  const uint64_t att_bytes = (rows * (uint64_t)d * 2 + 255) / 256 * 256;
  const uint64_t need = att_bytes + rows * 4;
  CUTILE_REQUIRE((uint64_t)num_kv_splits * (uint64_t)group <= 0x7fffffffull / (uint64_t)std::max(d, 1) && need <= CUTILE_SCRATCH_BYTES,
                 CUTILE_ERR_KERNEL_LAUNCH,
                 "fmha_decode_gqa_noalloc: %d KV heads x %d splits x GROUP %d x D %d needs %llu bytes of partial results, "
                 "the device-resident scratch holds %u; use fewer splits or the split + merge entry points with caller memory",
                 kv_heads, num_kv_splits, group, d, (unsigned long long)need, (unsigned)CUTILE_SCRATCH_BYTES);
  void* base = nullptr;
  size_t capacity = 0;
  if (cutile_status_t s = scratch_memory(&base, &capacity)) return s;
  CUTILE_REQUIRE(base && need <= capacity, CUTILE_ERR_STATE, "fmha_decode_gqa_noalloc: scratch lookup returned %zu bytes", capacity);
  const int32_t sg = num_kv_splits * group;
  cutile_partition_arg_t att;
  memset(&att, 0, sizeof(att));
  att.tensor.ptr = base;
  att.tensor.dtype = CUTILE_DTYPE_F16;
  att.tensor.rank = 3;
  att.tensor.shape[0] = kv_heads; att.tensor.shape[1] = sg; att.tensor.shape[2] = d;
  att.tensor.strides[0] = sg * d; att.tensor.strides[1] = d; att.tensor.strides[2] = 1;
  att.partition_shape[0] = 1; att.partition_shape[1] = group; att.partition_shape[2] = d;
  att.partition_strides[0] = att.partition_strides[1] = att.partition_strides[2] = 1;
  cutile_partition_arg_t lse;
  memset(&lse, 0, sizeof(lse));
  lse.tensor.ptr = (char*)base + att_bytes;
  lse.tensor.dtype = CUTILE_DTYPE_F32;
  lse.tensor.rank = 2;
  lse.tensor.shape[0] = kv_heads; lse.tensor.shape[1] = sg;
  lse.tensor.strides[0] = sg; lse.tensor.strides[1] = 1;
  lse.partition_shape[0] = 1; lse.partition_shape[1] = group;
  lse.partition_strides[0] = lse.partition_strides[1] = 1;
  const std::string g_s = std::to_string(group), bn_s = std::to_string(bn), d_s = std::to_string(d), n_s = std::to_string(num_kv_splits);
  const char* generics[4] = {g_s.c_str(), bn_s.c_str(), d_s.c_str(), n_s.c_str()};
  cutile_launch_opts_t split_opts;
  memset(&split_opts, 0, sizeof(split_opts));
  split_opts.generics = generics;
  split_opts.n_generics = 4;
  // Every (head, split) workgroup of the split kernel writes its GROUP rows and log-sum-exp values, an empty split
  // included, so nothing in the scratch has to start at zero and what an earlier call left there is never read.
  if (cutile_status_t s = cutile_launch_fmha_decode_gqa_split(stream, q, k, v, &att, &lse, qk_scale, position_start, &split_opts)) return s;
  return cutile_launch_splitk_reduce_merge(stream, &att.tensor, &lse.tensor, out, nullptr);
}

// Everything the entry point above does once per device and shape — opening the side library, the symbol lookup
// (the runtime places the array then), loading the two code objects — done ahead of time: the same call in
// compile-only mode, so every check runs and nothing is enqueued.
cutile_status_t cutile_fmha_decode_gqa_noalloc_prepare(const cutile_tensor_arg_t* q, const cutile_tensor_arg_t* k,
                                                       const cutile_tensor_arg_t* v, const cutile_partition_arg_t* out,
                                                       const cutile_tensor_arg_t* position_start, int32_t num_kv_splits,
                                                       int32_t bn) {
  const int saved = g_launch_mode;
  g_launch_mode = 1;
  cutile_status_t s = cutile_launch_fmha_decode_gqa_noalloc(nullptr, q, k, v, out, 1.0f, position_start, num_kv_splits, bn);
  g_launch_mode = saved;
  return s;
}

cutile_status_t cutile_launch_softmax(cutile_stream_t stream, const cutile_tensor_arg_t* x,
                                      const cutile_partition_arg_t* y, const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_tensor(x, "x", 2, 2)) return s;
  if (cutile_status_t s = check_partition(y, "y", 2, 2)) return s;
  const cutile_tensor_arg_t& yt = y->tensor;
  CUTILE_REQUIRE(x->dtype == yt.dtype && (x->dtype == CUTILE_DTYPE_F16 || x->dtype == CUTILE_DTYPE_F32),
                 CUTILE_ERR_KERNEL_LAUNCH, "softmax: x and y must both be f16 or both f32");
  const int32_t bm = y->partition_shape[0], bn = y->partition_shape[1];
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(bm), "BM")) return s;
  if (cutile_status_t s = check_generic(opts, 1, std::to_string(bn), "BN")) return s;
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(y, opts, tg)) return s;
  const std::string dt = cutile_dtype_name(x->dtype);
  const int e = 16 / (int)cutile_dtype_size(x->dtype);
  const uint64_t rows = std::min<uint64_t>((uint64_t)tg[0] * bm, yt.shape[0]);
  const bool vec_ok = bn % e == 0 && x->shape[1] % e == 0 && yt.shape[1] % e == 0 && x->strides[1] == 1 &&
                      yt.strides[1] == 1 && x->strides[0] % e == 0 && yt.strides[0] % e == 0 && aligned16(x->ptr) &&
                      aligned16(yt.ptr) && (uint64_t)x->shape[0] >= rows;
  std::vector<std::string> acceptable;
  if (vec_ok) acceptable = fitting_row_variants("softmax", dt + "_w", bn);
  acceptable.push_back(dt + "_generic");
  Resolved res;
  BucketScope bucket(dt + "|bn" + pow2_class(bn));
  if (cutile_status_t s = resolve_entry("softmax", opts, acceptable[0], acceptable, &res)) return s;
  ArgPacker args;
  args.push_tensor(*x);
  args.push_partition(*y);
  args.push_tile_grid(tg);
  const uint64_t segments = rows * tg[1];
  uint32_t grid[3];
  row_launch_grid(res.entry, segments, grid);
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

cutile_status_t cutile_launch_gemm(cutile_stream_t stream, const cutile_partition_arg_t* z, const cutile_tensor_arg_t* x,
                                   const cutile_tensor_arg_t* y, int32_t k, int32_t accumulate,
                                   const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_partition(z, "z", 2, 2)) return s;
  if (cutile_status_t s = check_tensor(x, "x", 2, 2)) return s;
  if (cutile_status_t s = check_tensor(y, "y", 2, 2)) return s;
  const cutile_tensor_arg_t& zt = z->tensor;
  const bool in_bf16 = x->dtype == CUTILE_DTYPE_BF16, in_f16 = x->dtype == CUTILE_DTYPE_F16, in_f32 = x->dtype == CUTILE_DTYPE_F32;
  CUTILE_REQUIRE(x->dtype == y->dtype && (in_bf16 || in_f16 || in_f32), CUTILE_ERR_KERNEL_NOT_FOUND,
                 "gemm: x and y must both be bf16, f16 or f32 (got %s, %s)", cutile_dtype_name(x->dtype),
                 cutile_dtype_name(y->dtype));
  CUTILE_REQUIRE((in_bf16 && (zt.dtype == CUTILE_DTYPE_BF16 || zt.dtype == CUTILE_DTYPE_F32)) ||
                     (in_f16 && zt.dtype == CUTILE_DTYPE_F16) || (in_f32 && zt.dtype == CUTILE_DTYPE_F32),
                 CUTILE_ERR_KERNEL_NOT_FOUND, "gemm: no kernel for %s operands with %s z (bf16 -> bf16 | f32, f16 -> f16, f32 -> f32)",
                 cutile_dtype_name(x->dtype), cutile_dtype_name(zt.dtype));
  const int32_t bm = z->partition_shape[0], bn = z->partition_shape[1];
  const int bk_user = generic_int(opts, 3, 64);
  if (cutile_status_t s = check_generic(opts, 1, std::to_string(bm), "BM")) return s;
  if (cutile_status_t s = check_generic(opts, 2, std::to_string(bn), "BN")) return s;
  CUTILE_REQUIRE(bk_user > 0, CUTILE_ERR_KERNEL_LAUNCH, "gemm: BK must be positive");
  CUTILE_REQUIRE(k >= 0, CUTILE_ERR_KERNEL_LAUNCH, "gemm: k must be non-negative");
  // The tile program runs k / BK whole K tiles (integer division).
  const int32_t k_total = (k / bk_user) * bk_user;
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(z, opts, tg)) return s;
  // The matrix-core variants need row-major operands with unit inner stride, 16-byte
  // aligned rows and K, N multiples of 8; everything else takes the any-layout kernel.
  const bool fast_layout = x->strides[1] == 1 && y->strides[1] == 1 && zt.strides[1] == 1 && x->strides[0] % 8 == 0 &&
                           y->strides[0] % 8 == 0 && zt.strides[0] % 4 == 0 && aligned16(x->ptr) && aligned16(y->ptr) &&
                           aligned16(zt.ptr) && x->shape[1] % 8 == 0 && y->shape[1] % 8 == 0 && zt.shape[1] % 4 == 0 &&
                           k_total % 8 == 0 && extent_bytes_2d(*x) < kDescriptorLimit && extent_bytes_2d(*y) < kDescriptorLimit &&
                           extent_bytes_2d(zt) < kDescriptorLimit;   // larger operands: the any-layout kernel (64-bit addresses)
  const std::string dt = in_f32 ? "f32" : in_f16 ? "f16" : zt.dtype == CUTILE_DTYPE_BF16 ? "bf16" : "bf16f32";
  // The ring-pipelined variants on 32 x 32 x 16 ("_r") fetch whole K tiles only ("_q" masks a ragged last tile).
  const int32_t k_valid = std::min(std::min(x->shape[1], y->shape[0]), k_total);
  // The streaming variants ("_s": one workgroup per compute unit walks its share of the tiles, the operand ring
  // running on from tile to tile) take whole tiles in M, N and K only, and at least three K tiles.
  const bool whole_tiles = (int64_t)tg[0] * bm == zt.shape[0] && (int64_t)tg[1] * bn == zt.shape[1] && x->shape[0] >= zt.shape[0] &&
                           y->shape[1] >= zt.shape[1] && k_valid == k_total && k_total % 64 == 0 && k_total >= 192;
  std::vector<std::string> acceptable;
  if (fast_layout)
    for (const auto& e : kernel_table())
      if (strcmp(e.function, "gemm") == 0 && dt == e.dtype && e.tile[0] == bm && e.tile[1] == bn &&
          (k_valid % 64 == 0 || strstr(e.variant, "_r") == nullptr) && strchr(e.variant, '+') == nullptr &&
          (whole_tiles || !is_stream_variant(e.variant)))
        acceptable.push_back(e.variant);
  acceptable.push_back(dt + "_generic");
  Resolved res;
  // shape class for tuning records: the tile, and whether the tiles fit one wave of workgroups over the 256 CUs
  BucketScope bucket(dt + "_" + std::to_string(bm) + "x" + std::to_string(bn) + ((uint64_t)tg[0] * tg[1] <= 256 ? "|tiles<=256" : "|tiles>256"));
  if (cutile_status_t s = resolve_entry("gemm", opts, acceptable[0], acceptable, &res)) return s;
  uint32_t stream_grid = 0;
  if (is_stream_variant(res.entry->variant)) {
    if (cutile_status_t s = stream_member(&res, "gemm", accumulate != 0, zt, (uint64_t)tg[0] * tg[1], &stream_grid)) return s;
  } else if (strstr(res.entry->variant, "_p2x4") != nullptr) {   // the walking form: one workgroup per compute unit
    int cus = 256;
    if (g_launch_mode != 2)
      if (cutile_status_t s = compute_units(res.device, &cus)) return s;
    stream_grid = (uint32_t)std::min<uint64_t>((uint64_t)tg[0] * tg[1], (uint64_t)std::max(cus, 1));
  }
  ArgPacker args;
  args.push_partition(*z);
  args.push_tensor(*x);
  args.push_tensor(*y);
  args.push_val<int32_t>(k_total);
  args.push_tile_grid(tg);
  args.push_val<int32_t>(accumulate ? 1 : 0);
  uint32_t grid[3] = {stream_grid ? stream_grid : tg[0] * tg[1], 1, 1};
  if (res.entry->tile[0] == 0) {   // any-layout kernel: 64x64 outputs per workgroup over the covered region
    const uint64_t cover_m = std::min<uint64_t>((uint64_t)tg[0] * bm, zt.shape[0]);
    const uint64_t cover_n = std::min<uint64_t>((uint64_t)tg[1] * bn, zt.shape[1]);
    grid[0] = std::max<uint32_t>(1, div_up(cover_m, 64));
    grid[1] = std::max<uint32_t>(1, div_up(cover_n, 64));
  }
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

// ---- mapped partitions (cutile/src/tensor.rs:314-401) ---------------------------------------------------------
cutile_status_t cutile_launch_batch_matmul(cutile_stream_t stream, const cutile_partition_arg_t* c, const cutile_tensor_arg_t* a,
                                           const cutile_tensor_arg_t* b, int32_t k, const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_partition(c, "c", 3, 3)) return s;
  if (cutile_status_t s = check_tensor(a, "a", 3, 3)) return s;
  if (cutile_status_t s = check_tensor(b, "b", 3, 3)) return s;
  const cutile_tensor_arg_t& ct = c->tensor;
  CUTILE_REQUIRE(a->dtype == b->dtype && a->dtype == ct.dtype &&
                     (ct.dtype == CUTILE_DTYPE_F32 || ct.dtype == CUTILE_DTYPE_F16 || ct.dtype == CUTILE_DTYPE_BF16),
                 CUTILE_ERR_KERNEL_NOT_FOUND, "batch_matmul: c, a and b must share one element type of f32, f16, bf16 (got %s, %s, %s)",
                 cutile_dtype_name(ct.dtype), cutile_dtype_name(a->dtype), cutile_dtype_name(b->dtype));
  CUTILE_REQUIRE(c->partition_shape[0] == 1, CUTILE_ERR_KERNEL_LAUNCH, "batch_matmul: c must be partitioned [1, BM, BN]");
  const int32_t bm = c->partition_shape[1], bn = c->partition_shape[2];
  const std::string dt = cutile_dtype_name(ct.dtype);
  if (cutile_status_t s = check_generic(opts, 0, dt, "E")) return s;
  if (cutile_status_t s = check_generic(opts, 1, std::to_string(bm), "BM")) return s;
  if (cutile_status_t s = check_generic(opts, 2, std::to_string(bn), "BN")) return s;
  const int bk_user = generic_int(opts, 3, 64);
  CUTILE_REQUIRE(bk_user > 0, CUTILE_ERR_KERNEL_LAUNCH, "batch_matmul: BK must be positive");
  CUTILE_REQUIRE(k >= 0, CUTILE_ERR_KERNEL_LAUNCH, "batch_matmul: k must be non-negative");
  if (cutile_status_t s = check_generic(opts, 4, std::to_string(k), "K")) return s;
  const int32_t k_total = (k / bk_user) * bk_user;
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(c, opts, tg)) return s;
  const uint32_t batches = std::min<uint32_t>(tg[0], (uint32_t)ct.shape[0]);
  // The matrix-core variants need what the plain GEMM's need of every rank-2 slice, 16-byte aligned batch strides, and
  // operands that have every batch the launch covers.
  const size_t es = cutile_dtype_size(ct.dtype);
  auto slice_ok = [&](const cutile_tensor_arg_t& t) {
    return t.strides[2] == 1 && t.strides[1] % 8 == 0 && t.strides[0] % 8 == 0 && aligned16(t.ptr) && t.shape[2] % 8 == 0 &&
           extent_bytes_2d(t.shape[1], t.shape[2], t.strides[1], (int64_t)es) < kDescriptorLimit;
  };
  const bool fast_layout = ct.dtype != CUTILE_DTYPE_F32 && slice_ok(*a) && slice_ok(*b) && slice_ok(ct) && k_total % 8 == 0 &&
                           (uint32_t)a->shape[0] >= batches && (uint32_t)b->shape[0] >= batches;
  const int32_t k_valid = std::min(std::min(a->shape[2], b->shape[1]), k_total);
  std::vector<std::string> acceptable;
  if (fast_layout)
    for (const auto& e : kernel_table())
      if (strcmp(e.function, "batch_matmul") == 0 && dt == e.dtype && e.tile[0] == bm && e.tile[1] == bn &&
          (k_valid % 64 == 0 || strstr(e.variant, "_r") == nullptr))
        acceptable.push_back(e.variant);
  acceptable.push_back(dt + "_generic");
  Resolved res;
  if (cutile_status_t s = resolve_entry("batch_matmul", opts, acceptable[0], acceptable, &res)) return s;
  ArgPacker args;
  args.push_partition(*c);
  args.push_tensor(*a);
  args.push_tensor(*b);
  args.push_val<int32_t>(k_total);
  args.push_tile_grid(tg);
  // The batch rides on HIP grid axis y (z for the any-layout kernel), which holds at most 65535 workgroups; the
  // tiles of one batch are folded into axis x.
  CUTILE_REQUIRE(batches <= 65535u, CUTILE_ERR_KERNEL_LAUNCH,
                 "batch_matmul: %u batches in one launch exceed the 65535 workgroups of the grid axis that carries the batch; split the launch",
                 batches);
  const uint64_t tiles_per_batch = (uint64_t)tg[1] * tg[2];
  CUTILE_REQUIRE(tiles_per_batch <= 0x7fffffffull, CUTILE_ERR_KERNEL_LAUNCH,
                 "batch_matmul: %llu output tiles per batch do not fit a launch grid axis", (unsigned long long)tiles_per_batch);
  uint32_t grid[3] = {(uint32_t)tiles_per_batch, batches, 1};
  if (res.entry->tile[0] == 0) {   // any-layout kernel: 64x64 outputs per workgroup over the covered region of each batch
    const uint64_t cover_m = std::min<uint64_t>((uint64_t)tg[1] * bm, ct.shape[1]);
    const uint64_t cover_n = std::min<uint64_t>((uint64_t)tg[2] * bn, ct.shape[2]);
    grid[0] = std::max<uint32_t>(1, div_up(cover_m, 64));
    grid[1] = std::max<uint32_t>(1, div_up(cover_n, 64));
    grid[2] = batches;
  }
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

static cutile_status_t mapped_record(const cutile_mapped_partition_arg_t* p, MappedArg* m, uint32_t grid[3]) {
  CUTILE_REQUIRE(p && grid, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  CUTILE_REQUIRE(!p->partition.prefix_coverage, CUTILE_ERR_TENSOR,
                 "a partial-coverage (prefix) partition cannot be mapped: a mapped schedule covers its full index space by construction");
  uint32_t pg[3];
  if (cutile_status_t s = cutile_partition_grid(&p->partition, pg)) return s;
  const int rank = p->map_rank;
  CUTILE_REQUIRE(rank >= 1 && rank <= 3, CUTILE_ERR_TENSOR, "mapped partitions require a rank-1 through rank-3 map shape.");
  bool all_owned = true;
  for (int a = 0; a < rank; ++a) {
    CUTILE_REQUIRE(p->map_shape[a] >= 0, CUTILE_ERR_TENSOR, "mapped partition map dimensions must be non-negative.");
    all_owned &= p->map_shape[a] == CUTILE_MAP_OWNED;
  }
  CUTILE_REQUIRE(!all_owned, CUTILE_ERR_TENSOR, "mapped partition requires at least one streamed (non-OWNED) map axis.");
  for (int a = 0; a < rank; ++a)
    CUTILE_REQUIRE(pg[a] != 0, CUTILE_ERR_TENSOR, "mapped partition requires a non-empty logical partition grid.");
  for (int a = rank; a < 3; ++a)
    CUTILE_REQUIRE(pg[a] == 1, CUTILE_ERR_TENSOR, "mapped partition map rank must match the logical partition grid rank.");
  uint64_t streamed = 1;
  int n_streamed = 0;
  for (int a = 0; a < rank; ++a)
    if (p->map_shape[a] != CUTILE_MAP_OWNED) {
      streamed *= pg[a];
      ++n_streamed;
      CUTILE_REQUIRE(streamed <= 0xFFFFFFFFull, CUTILE_ERR_TENSOR, "mapped partition logical grid is too large");
    }
  CUTILE_REQUIRE(p->num_tile_blocks > 0, CUTILE_ERR_TENSOR, "mapped partition requires num_tile_blocks > 0.");
  CUTILE_REQUIRE(p->num_tile_blocks <= streamed, CUTILE_ERR_TENSOR,
                 "mapped partition num_tile_blocks cannot exceed the streamed logical tile count.");
  // what the schedule itself accepts (emit_mapped_partition_schedule): only the trailing two streamed axes group
  int seen = 0;
  for (int a = 0; a < rank; ++a)
    if (p->map_shape[a] != CUTILE_MAP_OWNED) {
      ++seen;
      const bool leading = n_streamed - seen >= 2 || n_streamed == 1;
      CUTILE_REQUIRE(!leading || p->map_shape[a] == 1, CUTILE_ERR_TENSOR,
                     n_streamed == 1 ? "rank-1 mapped partition maps must be [1], got [%d]"
                                     : "mapped partition schedules group only the trailing two axes: a leading map axis must be 1, got %d",
                     p->map_shape[a]);
    }
  if (m) {
    for (int a = 0; a < 3; ++a) {
      m->map[a] = a < rank ? p->map_shape[a] : 1;
      m->grid[a] = pg[a];
    }
    m->rank = rank;
    m->total = (uint32_t)streamed;
  }
  grid[0] = p->num_tile_blocks;
  grid[1] = grid[2] = 1;
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_mapped_partition_grid(const cutile_mapped_partition_arg_t* p, uint32_t grid[3]) {
  return mapped_record(p, nullptr, grid);
}

cutile_status_t cutile_mapped_partition_index(const cutile_mapped_partition_arg_t* p, uint32_t item, uint32_t index[3],
                                              uint32_t* n_items) {
  CUTILE_REQUIRE(index, CUTILE_ERR_INVALID_ARGUMENT, "index is null");
  MappedArg m;
  uint32_t grid[3];
  if (cutile_status_t s = mapped_record(p, &m, grid)) return s;
  if (n_items) *n_items = m.total;
  CUTILE_REQUIRE(item < m.total, CUTILE_ERR_INVALID_ARGUMENT, "stream item %u is outside the %u items of the mapped partition", item, m.total);
  mapped_index(m, item, index);
  return CUTILE_SUCCESS;
}

// iter_indices_within: the (start_tile, num_tiles) pair of every axis checked against the grid as the reference's
// compile-time and run-time asserts do (cutile-compiler/src/compiler/compile_expression.rs:1403-1560), then the
// record of the narrowed schedule: lengths in m->grid, starts and the whole grid in *range.
static cutile_status_t mapped_subrange(const cutile_mapped_partition_arg_t* p, const int32_t* ranges, MappedArg* m,
                                       MappedRangeArg* range, uint32_t grid[3]) {
  CUTILE_REQUIRE(ranges, CUTILE_ERR_INVALID_ARGUMENT, "ranges is null");
  if (cutile_status_t s = mapped_record(p, m, grid)) return s;
  uint64_t total = 1;
  for (int a = 0; a < 3; ++a) {
    range->start[a] = 0;
    range->full_grid[a] = m->grid[a];
  }
  for (int a = 0; a < m->rank; ++a) {
    CUTILE_REQUIRE(m->map[a] != CUTILE_MAP_OWNED, CUTILE_ERR_TENSOR,
                   "sub-range iteration over a map with OWNED axes is not supported yet");
    const int32_t start = ranges[2 * a], len = ranges[2 * a + 1];
    CUTILE_REQUIRE(start >= 0, CUTILE_ERR_TENSOR, "sub-range axis %d start %d is negative", a, start);
    CUTILE_REQUIRE(len >= -1, CUTILE_ERR_TENSOR, "sub-range axis %d length %d is negative (-1 means the rest of the axis)", a, len);
    CUTILE_REQUIRE((uint32_t)start <= m->grid[a], CUTILE_ERR_TENSOR, "sub-range axis %d start %d exceeds the %u tiles of the axis", a,
                   start, m->grid[a]);
    const uint32_t n = len == -1 ? m->grid[a] - (uint32_t)start : (uint32_t)len;
    CUTILE_REQUIRE((uint64_t)start + n <= m->grid[a], CUTILE_ERR_TENSOR,
                   "sub-range axis %d (start %d, %u tiles) exceeds the %u tiles of the axis", a, start, n, m->grid[a]);
    range->start[a] = start;
    m->grid[a] = n;
    total *= n;
  }
  m->total = (uint32_t)total;
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_mapped_partition_index_within(const cutile_mapped_partition_arg_t* p, const int32_t* ranges, uint32_t item,
                                                     uint32_t index[3], uint32_t* n_items) {
  MappedArg m;
  MappedRangeArg range;
  uint32_t grid[3];
  if (cutile_status_t s = mapped_subrange(p, ranges, &m, &range, grid)) return s;
  if (n_items) *n_items = m.total;
  if (!index) return CUTILE_SUCCESS;                     // the count alone (an empty range has no item to ask for)
  CUTILE_REQUIRE(item < m.total, CUTILE_ERR_INVALID_ARGUMENT, "stream item %u is outside the %u items of the sub-range", item, m.total);
  mapped_index(m, item, index);
  for (int a = 0; a < 3; ++a) index[a] += (uint32_t)range.start[a];
  return CUTILE_SUCCESS;
}

// The launch grid of a mapped kernel: (num_tile_blocks, 1, 1); an explicit .grid() is a checked override.
static cutile_status_t mapped_launch_grid(const cutile_mapped_partition_arg_t* z, const cutile_launch_opts_t* opts, MappedArg* m,
                                          uint32_t grid[3]) {
  if (cutile_status_t s = mapped_record(z, m, grid)) return s;
  if (opts && (opts->grid[0] | opts->grid[1] | opts->grid[2]))
    CUTILE_REQUIRE(opts->grid[0] == grid[0] && opts->grid[1] == 1 && opts->grid[2] == 1, CUTILE_ERR_KERNEL_LAUNCH,
                   "launch grid (%u, %u, %u) does not match the inferred partition grid (%u, 1, 1)", opts->grid[0],
                   opts->grid[1], opts->grid[2], grid[0]);
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_launch_gemm_persistent(cutile_stream_t stream, const cutile_mapped_partition_arg_t* zm,
                                              const cutile_tensor_arg_t* x, const cutile_tensor_arg_t* y,
                                              const cutile_launch_opts_t* opts) {
  CUTILE_REQUIRE(zm, CUTILE_ERR_INVALID_ARGUMENT, "z is null");
  const cutile_partition_arg_t* z = &zm->partition;
  if (cutile_status_t s = check_partition(z, "z", 2, 2)) return s;
  if (cutile_status_t s = check_tensor(x, "x", 2, 2)) return s;
  if (cutile_status_t s = check_tensor(y, "y", 2, 2)) return s;
  const cutile_tensor_arg_t& zt = z->tensor;
  const bool in_bf16 = x->dtype == CUTILE_DTYPE_BF16, in_f16 = x->dtype == CUTILE_DTYPE_F16, in_f32 = x->dtype == CUTILE_DTYPE_F32;
  CUTILE_REQUIRE(x->dtype == y->dtype && zt.dtype == x->dtype && (in_bf16 || in_f16 || in_f32), CUTILE_ERR_KERNEL_NOT_FOUND,
                 "gemm_persistent: z, x and y must share one element type of bf16, f16, f32 (got %s, %s, %s)",
                 cutile_dtype_name(zt.dtype), cutile_dtype_name(x->dtype), cutile_dtype_name(y->dtype));
  CUTILE_REQUIRE(zm->map_rank == 2 && zm->map_shape[0] != CUTILE_MAP_OWNED && zm->map_shape[1] != CUTILE_MAP_OWNED,
                 CUTILE_ERR_KERNEL_LAUNCH, "gemm_persistent: z needs a rank-2 map with both axes streamed");
  const int32_t bm = z->partition_shape[0], bn = z->partition_shape[1];
  const char* dt = in_f32 ? "f32" : in_f16 ? "f16" : "bf16";
  if (cutile_status_t s = check_generic(opts, 0, dt, "T")) return s;
  if (cutile_status_t s = check_generic(opts, 1, std::to_string(bm), "BM")) return s;
  if (cutile_status_t s = check_generic(opts, 2, std::to_string(bn), "BN")) return s;
  if (cutile_status_t s = check_generic(opts, 4, std::to_string(zm->map_shape[0]), "MAP_SHAPE[0]")) return s;
  if (cutile_status_t s = check_generic(opts, 5, std::to_string(zm->map_shape[1]), "MAP_SHAPE[1]")) return s;
  const int bk_user = generic_int(opts, 3, 64);
  CUTILE_REQUIRE(bk_user > 0, CUTILE_ERR_KERNEL_LAUNCH, "gemm_persistent: BK must be positive");
  // launch checks the reference derives from the kernel body (persistent_gemm.rs:20-26): the K tiles of x must exist in y
  CUTILE_REQUIRE(div_up((uint32_t)x->shape[1], (uint32_t)bk_user) <= div_up((uint32_t)y->shape[0], (uint32_t)bk_user),
                 CUTILE_ERR_KERNEL_LAUNCH, "gemm_persistent: ceil(dim(x, 1)/BK) <= ceil(dim(y, 0)/BK) failed (%d, %d, BK = %d)",
                 x->shape[1], y->shape[0], bk_user);
  MappedArg m;
  uint32_t grid[3];
  if (cutile_status_t s = mapped_launch_grid(zm, opts, &m, grid)) return s;
  const bool fast_layout = (in_bf16 || in_f16) && x->strides[1] == 1 && y->strides[1] == 1 && zt.strides[1] == 1 && x->strides[0] % 8 == 0 &&
                           y->strides[0] % 8 == 0 && zt.strides[0] % 4 == 0 && aligned16(x->ptr) && aligned16(y->ptr) &&
                           aligned16(zt.ptr) && x->shape[1] % 8 == 0 && y->shape[1] % 8 == 0 && zt.shape[1] % 4 == 0 &&
                           extent_bytes_2d(*x) < kDescriptorLimit && extent_bytes_2d(*y) < kDescriptorLimit &&
                           extent_bytes_2d(zt) < kDescriptorLimit;
  // the streaming variant: whole tiles in M, N and K, at least three K tiles, the plain two-axis schedule
  const int32_t kx = x->shape[1];
  const bool whole_tiles = zt.shape[0] % bm == 0 && zt.shape[1] % bn == 0 && x->shape[0] >= zt.shape[0] && y->shape[1] >= zt.shape[1] &&
                           y->shape[0] >= kx && kx % 64 == 0 && kx >= 192 && m.rank == 2;
  std::vector<std::string> acceptable;
  if (fast_layout)
    for (const auto& e : kernel_table())
      if (strcmp(e.function, "gemm_persistent") == 0 && strcmp(e.dtype, dt) == 0 && e.tile[0] == bm && e.tile[1] == bn &&
          strchr(e.variant, '+') == nullptr && (whole_tiles || !is_stream_variant(e.variant)))
        acceptable.push_back(e.variant);
  acceptable.push_back(std::string(dt) + "_generic");
  Resolved res;
  if (cutile_status_t s = resolve_entry("gemm_persistent", opts, acceptable[0], acceptable, &res)) return s;
  if (is_stream_variant(res.entry->variant)) {
    uint32_t unused = 0;
    // (the member only; the launch grid stays the caller's num_tile_blocks, and the accumulators start from zero)
    if (cutile_status_t s = stream_member(&res, "gemm_persistent", true, zt, m.total, &unused)) return s;
  }
  ArgPacker args;
  args.push_partition(*z);
  args.push_tensor(*x);
  args.push_tensor(*y);
  args.push_val<MappedArg>(m);
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

// group_gemm_f16_nt_desc (cutile-kernels/src/experimental/moe.rs:67-128): no partition argument, so the launch grid
// (NUM_SM workgroups) comes from .grid() or the NUM_SM generic, and the tile shape from the BM / BN generics.
cutile_status_t cutile_launch_group_gemm_f16_nt_desc(cutile_stream_t stream, const cutile_tensor_arg_t* a_ptrs,
                                                     const cutile_tensor_arg_t* b_ptrs, const cutile_tensor_arg_t* c_ptrs,
                                                     const cutile_tensor_arg_t* a_metas, const cutile_tensor_arg_t* b_metas,
                                                     const cutile_tensor_arg_t* c_metas, int32_t num_groups,
                                                     const cutile_launch_opts_t* opts) {
  const cutile_tensor_arg_t* ptrs[3] = {a_ptrs, b_ptrs, c_ptrs};
  const cutile_tensor_arg_t* metas[3] = {a_metas, b_metas, c_metas};
  const char* names[3] = {"a", "b", "c"};
  CUTILE_REQUIRE(num_groups >= 0, CUTILE_ERR_KERNEL_LAUNCH, "group_gemm_f16_nt_desc: num_groups must be non-negative");
  for (int i = 0; i < 3; ++i) {
    if (cutile_status_t s = check_tensor(ptrs[i], "pointer table", 1, 1)) return s;
    if (cutile_status_t s = check_tensor(metas[i], "descriptor table", 2, 2)) return s;
    CUTILE_REQUIRE(ptrs[i]->dtype == CUTILE_DTYPE_I64 && ((uintptr_t)ptrs[i]->ptr & 7) == 0 && ptrs[i]->shape[0] >= num_groups,
                   CUTILE_ERR_KERNEL_LAUNCH, "group_gemm_f16_nt_desc: %s_ptrs must be an aligned i64 tensor of at least %d entries",
                   names[i], num_groups);
    CUTILE_REQUIRE(metas[i]->dtype == CUTILE_DTYPE_I32 && metas[i]->shape[1] == 8 && metas[i]->shape[0] >= num_groups &&
                       ((uintptr_t)metas[i]->ptr & 3) == 0,
                   CUTILE_ERR_KERNEL_LAUNCH, "group_gemm_f16_nt_desc: %s_metas must be an i32 tensor [>= %d, 8]", names[i], num_groups);
  }
  const int bm = generic_int(opts, 0, 128), bn = generic_int(opts, 1, 128), bk = generic_int(opts, 2, 64);
  const int num_sm_generic = generic_int(opts, 3, 0);
  CUTILE_REQUIRE(bk > 0, CUTILE_ERR_KERNEL_LAUNCH, "group_gemm_f16_nt_desc: BK must be positive");
  uint32_t grid[3] = {0, 1, 1};
  if (opts && (opts->grid[0] | opts->grid[1] | opts->grid[2])) {
    CUTILE_REQUIRE(opts->grid[0] > 0 && opts->grid[1] == 1 && opts->grid[2] == 1, CUTILE_ERR_KERNEL_LAUNCH,
                   "group_gemm_f16_nt_desc: the launch grid must be (NUM_SM, 1, 1), got (%u, %u, %u)", opts->grid[0], opts->grid[1],
                   opts->grid[2]);
    grid[0] = opts->grid[0];
  }
  CUTILE_REQUIRE(grid[0] || num_sm_generic > 0, CUTILE_ERR_KERNEL_LAUNCH, "Launch grid required.");
  // tiles advance by NUM_SM (moe.rs:121): a grid of another size would skip or repeat tiles
  CUTILE_REQUIRE(!grid[0] || num_sm_generic <= 0 || (uint32_t)num_sm_generic == grid[0], CUTILE_ERR_KERNEL_LAUNCH,
                 "group_gemm_f16_nt_desc: the launch grid (%u) must equal NUM_SM = %d", grid[0], num_sm_generic);
  if (!grid[0]) grid[0] = (uint32_t)num_sm_generic;
  std::vector<std::string> acceptable;
  for (const auto& e : kernel_table())
    if (strcmp(e.function, "group_gemm_nt_desc") == 0 && e.tile[0] == bm && e.tile[1] == bn) acceptable.push_back(e.variant);
  CUTILE_REQUIRE(!acceptable.empty(), CUTILE_ERR_KERNEL_NOT_FOUND,
                 "no precompiled variant of group_gemm_f16_nt_desc<BM=%d, BN=%d>; available: %s", bm, bn,
                 list_variants("group_gemm_nt_desc").c_str());
  cutile_launch_opts_t o = opts ? *opts : cutile_launch_opts_t{};
  o.generics = nullptr;
  o.n_generics = 0;
  Resolved res;
  if (cutile_status_t s = resolve_entry("group_gemm_nt_desc", &o, acceptable[0], acceptable, &res)) return s;
  ArgPacker args;
  for (int i = 0; i < 3; ++i) args.push_tensor(*ptrs[i]);
  for (int i = 0; i < 3; ++i) args.push_tensor(*metas[i]);
  args.push_val<int32_t>(num_groups);
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

cutile_status_t cutile_launch_mapped_tile_index(cutile_stream_t stream, const cutile_mapped_partition_arg_t* zm,
                                                const cutile_launch_opts_t* opts) {
  CUTILE_REQUIRE(zm, CUTILE_ERR_INVALID_ARGUMENT, "z is null");
  const cutile_partition_arg_t* z = &zm->partition;
  if (cutile_status_t s = check_partition(z, "z", 1, 3)) return s;
  CUTILE_REQUIRE(z->tensor.dtype == CUTILE_DTYPE_I32, CUTILE_ERR_KERNEL_NOT_FOUND, "mapped_tile_index: z must be i32");
  MappedArg m;
  uint32_t grid[3];
  if (cutile_status_t s = mapped_launch_grid(zm, opts, &m, grid)) return s;
  const std::string want = "i32_r" + std::to_string(z->tensor.rank);
  Resolved res;
  if (cutile_status_t s = resolve_entry("mapped_tile_index", opts, want, {want}, &res)) return s;
  ArgPacker args;
  args.push_partition(*z);
  args.push_val<MappedArg>(m);
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

cutile_status_t cutile_launch_mapped_tile_index_within(cutile_stream_t stream, const cutile_mapped_partition_arg_t* zm,
                                                       const int32_t* ranges, const cutile_launch_opts_t* opts) {
  CUTILE_REQUIRE(zm, CUTILE_ERR_INVALID_ARGUMENT, "z is null");
  const cutile_partition_arg_t* z = &zm->partition;
  if (cutile_status_t s = check_partition(z, "z", 1, 3)) return s;
  CUTILE_REQUIRE(z->tensor.dtype == CUTILE_DTYPE_I32, CUTILE_ERR_KERNEL_NOT_FOUND, "mapped_tile_index_within: z must be i32");
  MappedArg full, m;
  MappedRangeArg range;
  uint32_t grid[3];
  if (cutile_status_t s = mapped_launch_grid(zm, opts, &full, grid)) return s;
  if (cutile_status_t s = mapped_subrange(zm, ranges, &m, &range, grid)) return s;
  const std::string want = "i32_r" + std::to_string(z->tensor.rank);
  Resolved res;
  if (cutile_status_t s = resolve_entry("mapped_tile_index_within", opts, want, {want}, &res)) return s;
  ArgPacker args;
  args.push_partition(*z);
  args.push_val<MappedArg>(m);
  args.push_val<MappedRangeArg>(range);
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

// iter_indices_with: the type gives both partitions one tile and map shape; their logical grids must match too
// (cutile-compiler/src/compiler/compile_expression.rs:1318-1397).
cutile_status_t cutile_mapped_partitions_shared(const cutile_mapped_partition_arg_t* a, const cutile_mapped_partition_arg_t* b) {
  CUTILE_REQUIRE(a && b, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  uint32_t ga[3], gb[3], launch[3];
  if (cutile_status_t s = mapped_record(a, nullptr, launch)) return s;
  if (cutile_status_t s = mapped_record(b, nullptr, launch)) return s;
  bool same = a->map_rank == b->map_rank && a->partition.tensor.rank == b->partition.tensor.rank;
  for (int i = 0; same && i < a->map_rank; ++i) same = a->map_shape[i] == b->map_shape[i];
  for (int i = 0; same && i < a->partition.tensor.rank; ++i) same = a->partition.partition_shape[i] == b->partition.partition_shape[i];
  CUTILE_REQUIRE(same, CUTILE_ERR_TENSOR, "iter_indices_with requires both mapped partitions to share tile and map shapes");
  if (cutile_status_t s = cutile_partition_grid(&a->partition, ga)) return s;
  if (cutile_status_t s = cutile_partition_grid(&b->partition, gb)) return s;
  for (int i = 0; i < 3; ++i)
    CUTILE_REQUIRE(ga[i] == gb[i], CUTILE_ERR_TENSOR,
                   "shared mapped partitions require equal logical partition grids: axis %d has %u vs %u tiles", i, ga[i], gb[i]);
  CUTILE_REQUIRE(a->num_tile_blocks == b->num_tile_blocks, CUTILE_ERR_TENSOR,
                 "shared mapped partitions disagree on num_tile_blocks (%u vs %u)", a->num_tile_blocks, b->num_tile_blocks);
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_launch_mapped_shared_cache_update_f32(cutile_stream_t stream, const cutile_mapped_partition_arg_t* k_cache,
                                                             const cutile_mapped_partition_arg_t* v_cache,
                                                             const cutile_tensor_arg_t* new_k, int32_t source_seq_major,
                                                             const cutile_tensor_arg_t* position, int32_t start_tile,
                                                             int32_t n_tiles, const cutile_launch_opts_t* opts) {
  CUTILE_REQUIRE(k_cache && v_cache, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  if (cutile_status_t s = check_partition(&k_cache->partition, "k_cache", 3, 3)) return s;
  if (cutile_status_t s = check_partition(&v_cache->partition, "v_cache", 3, 3)) return s;
  if (cutile_status_t s = check_tensor(new_k, "new_k", 3, 3)) return s;
  CUTILE_REQUIRE(k_cache->partition.tensor.dtype == CUTILE_DTYPE_F32 && v_cache->partition.tensor.dtype == CUTILE_DTYPE_F32 &&
                     new_k->dtype == CUTILE_DTYPE_F32,
                 CUTILE_ERR_KERNEL_NOT_FOUND, "mapped_shared_cache_update: k_cache, v_cache and new_k must be f32");
  if (position) {
    if (cutile_status_t s = check_tensor(position, "position", 1, 1)) return s;
    CUTILE_REQUIRE(position->dtype == CUTILE_DTYPE_I32 && position->shape[0] == 1 && ((uintptr_t)position->ptr & 3) == 0,
                   CUTILE_ERR_KERNEL_LAUNCH, "mapped_shared_cache_update: position must be one i32 in device memory");
  }
  if (cutile_status_t s = cutile_mapped_partitions_shared(k_cache, v_cache)) return s;
  MappedArg full, m;
  MappedRangeArg range;
  uint32_t grid[3];
  if (cutile_status_t s = mapped_launch_grid(k_cache, opts, &full, grid)) return s;
  // a start read on the device is checked there; its length must fit the axis in any case
  const int32_t ranges[6] = {0, -1, position ? 0 : start_tile, n_tiles, 0, -1};
  CUTILE_REQUIRE(n_tiles >= 0, CUTILE_ERR_TENSOR, "sub-range axis 1 length %d is negative", n_tiles);
  if (cutile_status_t s = mapped_subrange(k_cache, ranges, &m, &range, grid)) return s;
  Resolved res;
  if (cutile_status_t s = resolve_entry("mapped_shared_cache_update", opts, "f32", {"f32"}, &res)) return s;
  ArgPacker args;
  args.push_partition(k_cache->partition);
  args.push_partition(v_cache->partition);
  args.push_tensor(*new_k);
  args.push_val<MappedArg>(m);
  args.push_val<MappedRangeArg>(range);
  args.push_val<const void*>(position ? position->ptr : nullptr);
  args.push_val<int32_t>(source_seq_major ? 1 : 0);
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

cutile_status_t cutile_launch_fmha(cutile_stream_t stream, const cutile_partition_arg_t* out, const cutile_tensor_arg_t* q,
                                   const cutile_tensor_arg_t* k, const cutile_tensor_arg_t* v, float qk_scale,
                                   int32_t input_pos, int32_t query_group_size, int32_t causal,
                                   const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_partition(out, "out", 3, 3)) return s;
  if (cutile_status_t s = check_tensor(q, "q", 4, 4)) return s;
  if (cutile_status_t s = check_tensor(k, "k", 4, 4)) return s;
  if (cutile_status_t s = check_tensor(v, "v", 4, 4)) return s;
  const cutile_tensor_arg_t& ot = out->tensor;
  CUTILE_REQUIRE((q->dtype == CUTILE_DTYPE_BF16 || q->dtype == CUTILE_DTYPE_F16) && k->dtype == q->dtype &&
                     v->dtype == q->dtype && ot.dtype == q->dtype,
                 CUTILE_ERR_KERNEL_NOT_FOUND, "fmha: precompiled variants take bf16 or f16 q, k, v, out of one type");
  const int32_t b = q->shape[0], h = q->shape[1], m = q->shape[2], d = q->shape[3];
  const int32_t bm = out->partition_shape[1], dd = out->partition_shape[2];
  CUTILE_REQUIRE(out->partition_shape[0] == 1 && dd == d, CUTILE_ERR_KERNEL_LAUNCH,
                 "fmha: out must be partitioned [1, BM, %d], got [%d, %d, %d]", d, out->partition_shape[0], bm, dd);
  CUTILE_REQUIRE(ot.shape[0] == b * h && ot.shape[1] == m && ot.shape[2] == d, CUTILE_ERR_KERNEL_LAUNCH,
                 "fmha: out is [%d, %d, %d], expected [b*h = %d, m = %d, d = %d]", ot.shape[0], ot.shape[1], ot.shape[2],
                 b * h, m, d);
  CUTILE_REQUIRE(query_group_size > 0 && h % query_group_size == 0 && k->shape[1] * query_group_size == h &&
                     v->shape[1] == k->shape[1],
                 CUTILE_ERR_KERNEL_LAUNCH, "fmha: %d query heads, %d kv heads, query_group_size %d do not agree", h,
                 k->shape[1], query_group_size);
  CUTILE_REQUIRE(k->shape[0] == b && v->shape[0] == b && k->shape[3] == d && v->shape[3] == d &&
                     k->shape[2] == v->shape[2],
                 CUTILE_ERR_KERNEL_LAUNCH, "fmha: k / v shapes do not match q");
  CUTILE_REQUIRE(input_pos >= 0, CUTILE_ERR_KERNEL_LAUNCH, "fmha: input_pos must be non-negative");
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(bm), "BM")) return s;
  if (cutile_status_t s = check_generic(opts, 2, std::to_string(d), "D")) return s;
  const int bn_user = generic_int(opts, 1, 0);
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(out, opts, tg)) return s;
  CUTILE_REQUIRE(q->strides[3] == 1 && k->strides[3] == 1 && v->strides[3] == 1 && ot.strides[2] == 1 &&
                     q->strides[2] % 8 == 0 && k->strides[2] % 8 == 0 && v->strides[2] % 8 == 0 &&
                     ot.strides[1] % 4 == 0 && aligned16(q->ptr) && aligned16(k->ptr) && aligned16(v->ptr) &&
                     aligned16(ot.ptr) && q->strides[0] % 8 == 0 && q->strides[1] % 8 == 0 && k->strides[0] % 8 == 0 &&
                     k->strides[1] % 8 == 0 && v->strides[0] % 8 == 0 && v->strides[1] % 8 == 0,
                 CUTILE_ERR_KERNEL_NOT_FOUND, "fmha: precompiled variants need unit head-dim stride and 16-byte aligned rows");
  // one descriptor per (batch, head): its rows must end below 2 GiB
  CUTILE_REQUIRE(extent_bytes_2d(m, d, q->strides[2], 2) < kDescriptorLimit && extent_bytes_2d(k->shape[2], d, k->strides[2], 2) < kDescriptorLimit &&
                     extent_bytes_2d(v->shape[2], d, v->strides[2], 2) < kDescriptorLimit && extent_bytes_2d(m, d, ot.strides[1], 2) < kDescriptorLimit,
                 CUTILE_ERR_KERNEL_NOT_FOUND, "fmha: the rows of one (batch, head) of q, k, v and out must each end below 2 GiB from the first");
  const std::string dt = cutile_dtype_name(q->dtype);
  std::vector<std::string> acceptable, same_bn;
  for (const auto& e : kernel_table())
    if (strcmp(e.function, "fmha") == 0 && dt == e.dtype && e.tile[0] == bm && e.tile[2] == d) {
      acceptable.push_back(e.variant);
      if (e.tile[1] == bn_user) same_bn.push_back(e.variant);
    }
  CUTILE_REQUIRE(!acceptable.empty(), CUTILE_ERR_KERNEL_NOT_FOUND,
                 "no precompiled variant of fmha<%s, BM=%d, D=%d>; available: %s", dt.c_str(), bm, d,
                 list_variants("fmha").c_str());
  Resolved res;
  BucketScope bucket(dt + "_bm" + std::to_string(bm) + "_d" + std::to_string(d) + (causal ? "|causal" : "|full"));
  if (cutile_status_t s = resolve_entry("fmha", opts, same_bn.empty() ? acceptable[0] : same_bn[0], acceptable, &res)) return s;
  ArgPacker args;
  args.push_partition(*out);
  args.push_tensor(*q);
  args.push_tensor(*k);
  args.push_tensor(*v);
  args.push_val<float>(qk_scale);
  args.push_val<int32_t>(input_pos);
  args.push_val<int32_t>(query_group_size);
  args.push_val<int32_t>(causal ? 1 : 0);
  args.push_tile_grid(tg);
  uint32_t grid[3] = {tg[0], tg[1], 1};
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

// Sequence-layout attention: q / out [q_len, q_heads, D] and k / v [kv_heads, max_seq, D] are handed to the
// (batch, head, row, d) kernels as permuted views (batch 1, head stride D, row stride q_heads * D); the
// kernel tile is chosen here, whatever BM the caller's partition names, because the output does not depend on it.
cutile_status_t cutile_launch_fmha_seq_f16(cutile_stream_t stream, const cutile_tensor_arg_t* q,
                                           const cutile_tensor_arg_t* k, const cutile_tensor_arg_t* v,
                                           const cutile_partition_arg_t* out, float qk_scale,
                                           int32_t query_group_size, int32_t kv_len, int32_t query_start,
                                           const cutile_tensor_arg_t* position_start, int32_t kv_len_from_position,
                                           int32_t causal, const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_tensor(q, "q", 3, 3)) return s;
  if (cutile_status_t s = check_tensor(k, "k", 3, 3)) return s;
  if (cutile_status_t s = check_tensor(v, "v", 3, 3)) return s;
  if (cutile_status_t s = check_partition(out, "out", 3, 3)) return s;
  const cutile_tensor_arg_t& ot = out->tensor;
  CUTILE_REQUIRE(q->dtype == CUTILE_DTYPE_F16 && k->dtype == CUTILE_DTYPE_F16 && v->dtype == CUTILE_DTYPE_F16 &&
                     ot.dtype == CUTILE_DTYPE_F16,
                 CUTILE_ERR_KERNEL_LAUNCH, "sequence attention: q, k, v and out must be f16");
  const int32_t q_len = q->shape[0], q_heads = q->shape[1], d = q->shape[2], kv_heads = k->shape[0];
  const int32_t max_seq = std::min(k->shape[1], v->shape[1]);
  CUTILE_REQUIRE(k->shape[2] == d && v->shape[2] == d && v->shape[0] == kv_heads && ot.shape[2] == d &&
                     ot.shape[0] <= q_len && ot.shape[1] <= q_heads,
                 CUTILE_ERR_KERNEL_LAUNCH, "sequence attention: q/out [q_len, q_heads, D] and k/v [kv_heads, kv_len, D] do not agree");
  CUTILE_REQUIRE(query_group_size > 0 && (int64_t)kv_heads * query_group_size == q_heads, CUTILE_ERR_KERNEL_LAUNCH,
                 "sequence attention: %d query heads, %d kv heads, query_group_size %d do not agree", q_heads, kv_heads,
                 query_group_size);
  const int32_t bm = out->partition_shape[0], pack = out->partition_shape[1];
  CUTILE_REQUIRE(out->partition_shape[2] == d && pack > 0 && query_group_size % pack == 0, CUTILE_ERR_KERNEL_LAUNCH,
                 "sequence attention: out must be partitioned [BM, G, %d] with G dividing query_group_size = %d, got [%d, %d, %d]",
                 d, query_group_size, bm, pack, out->partition_shape[2]);
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(bm), "BM")) return s;
  if (cutile_status_t s = check_generic(opts, 2, std::to_string(d), "D")) return s;
  if (position_start) {
    if (cutile_status_t s = check_tensor(position_start, "position_start", 1, 1)) return s;
    CUTILE_REQUIRE(position_start->dtype == CUTILE_DTYPE_U32 && position_start->shape[0] == 1 &&
                       ((uintptr_t)position_start->ptr & 3) == 0,
                   CUTILE_ERR_KERNEL_LAUNCH, "sequence attention: position_start must be one aligned u32");
    if (!kv_len_from_position) kv_len = max_seq;
  } else {
    CUTILE_REQUIRE(query_start >= 0 && kv_len >= 0 && kv_len <= max_seq, CUTILE_ERR_KERNEL_LAUNCH,
                   "sequence attention: query_start = %d and kv_len = %d must be non-negative and kv_len within the %d rows of k and v",
                   query_start, kv_len, max_seq);
  }
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(out, opts, tg)) return s;
  auto rows_ok = [&](const cutile_tensor_arg_t& t) {
    return t.strides[2] == 1 && t.strides[0] % 8 == 0 && t.strides[1] % 8 == 0 && aligned16(t.ptr);
  };
  CUTILE_REQUIRE(rows_ok(*q) && rows_ok(*k) && rows_ok(*v) && rows_ok(ot), CUTILE_ERR_KERNEL_NOT_FOUND,
                 "sequence attention: precompiled variants need unit head-dim stride and 16-byte aligned rows");
  CUTILE_REQUIRE(extent_bytes_2d(q->shape[0], d, q->strides[0], 2) < kDescriptorLimit && extent_bytes_2d(max_seq, d, k->strides[1], 2) < kDescriptorLimit &&
                     extent_bytes_2d(max_seq, d, v->strides[1], 2) < kDescriptorLimit && extent_bytes_2d(ot.shape[0], d, ot.strides[0], 2) < kDescriptorLimit,
                 CUTILE_ERR_KERNEL_NOT_FOUND, "sequence attention: the rows of one head of q, k, v and out must each end below 2 GiB from the first");
  // what the launch covers: rows 0 .. rows_cov and heads 0 .. heads_cov of out
  const int32_t rows_cov = (int32_t)std::min<int64_t>((int64_t)tg[0] * bm, ot.shape[0]);
  const int32_t heads_cov = (int32_t)std::min<int64_t>((int64_t)tg[1] * pack, ot.shape[1]);
  // views in the kernels' (batch, head, row, d) order
  cutile_tensor_arg_t qv{}, kv{}, vv{};
  qv.ptr = q->ptr; qv.dtype = q->dtype; qv.rank = 4;
  qv.shape[0] = 1; qv.shape[1] = q_heads; qv.shape[2] = rows_cov; qv.shape[3] = d;
  qv.strides[0] = 0; qv.strides[1] = q->strides[1]; qv.strides[2] = q->strides[0]; qv.strides[3] = 1;
  auto kv_view = [&](const cutile_tensor_arg_t& t, cutile_tensor_arg_t* o) {
    o->ptr = t.ptr; o->dtype = t.dtype; o->rank = 4;
    o->shape[0] = 1; o->shape[1] = kv_heads; o->shape[2] = position_start ? max_seq : kv_len; o->shape[3] = d;
    o->strides[0] = 0; o->strides[1] = t.strides[0]; o->strides[2] = t.strides[1]; o->strides[3] = 1;
  };
  kv_view(*k, &kv);
  kv_view(*v, &vv);
  cutile_partition_arg_t ov{};
  ov.tensor.ptr = ot.ptr; ov.tensor.dtype = ot.dtype; ov.tensor.rank = 3;
  ov.tensor.shape[0] = heads_cov; ov.tensor.shape[1] = rows_cov; ov.tensor.shape[2] = d;
  ov.tensor.strides[0] = ot.strides[1]; ov.tensor.strides[1] = ot.strides[0]; ov.tensor.strides[2] = 1;
  // kernel tile: the ping-pong kernel for long D = 128 prefills, else the largest tile of that D
  const char* function = position_start ? "fmha_seq" : "fmha";
  std::vector<const KernelEntry*> fit;
  for (const auto& e : kernel_table())
    if (strcmp(e.function, function) == 0 && strcmp(e.dtype, "f16") == 0 && e.tile[2] == d) fit.push_back(&e);
  CUTILE_REQUIRE(!fit.empty(), CUTILE_ERR_KERNEL_NOT_FOUND, "no precompiled sequence attention for f16, D = %d; available: %s", d,
                 list_variants(function).c_str());
  const bool long_prefill = rows_cov >= 256 && kv_len > 0;
  std::stable_sort(fit.begin(), fit.end(), [&](const KernelEntry* a, const KernelEntry* b) {
    const bool pa = strstr(a->variant, "_pp") != nullptr, pb = strstr(b->variant, "_pp") != nullptr;
    if (pa != pb) return long_prefill ? pa : pb;
    return a->tile[0] > b->tile[0];
  });
  std::vector<std::string> acceptable;
  for (auto* e : fit)
    if (kv_len > 0 || strstr(e->variant, "_pp") == nullptr) acceptable.push_back(e->variant);   // an empty key range: the plain kernels only
  CUTILE_REQUIRE(!acceptable.empty(), CUTILE_ERR_KERNEL_NOT_FOUND, "no precompiled sequence attention for f16, D = %d and an empty key range", d);
  cutile_launch_opts_t o = opts ? *opts : cutile_launch_opts_t{};
  o.generics = nullptr;
  o.n_generics = 0;
  Resolved res;
  if (cutile_status_t s = resolve_entry(function, &o, acceptable[0], acceptable, &res)) return s;
  const int32_t kbm = res.entry->tile[0];
  ov.partition_shape[0] = 1; ov.partition_shape[1] = kbm; ov.partition_shape[2] = d;
  for (int i = 0; i < 3; ++i) ov.partition_strides[i] = ov.tensor.strides[i];
  const uint32_t kg[3] = {(uint32_t)heads_cov, div_up((uint64_t)rows_cov, (uint64_t)kbm), 1};
  ArgPacker args;
  args.push_partition(ov);
  args.push_tensor(qv);
  args.push_tensor(kv);
  args.push_tensor(vv);
  args.push_val<float>(qk_scale);
  if (position_start) {
    args.push_val<const void*>(position_start->ptr);
    args.push_val<int32_t>(kv_len_from_position ? 1 : 0);
  } else {
    args.push_val<int32_t>(query_start);
  }
  args.push_val<int32_t>(query_group_size);
  args.push_val<int32_t>(causal ? 1 : 0);
  args.push_tile_grid(kg);
  uint32_t grid[3] = {kg[0], kg[1], 1};
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

// fmha_prefill_gqa_lpt (cutile-kernels/src/experimental/attention.rs:22-377): fmha_prefill_gqa on raw pointers, with the
// caller choosing the order in which tile blocks take (query block, head group) pairs (longest first, swizzled).  The
// order does not change the result; this library's kernels have their own (heaviest tiles first, heads that share a
// KV head side by side on one XCD), so the scheduling arguments of the reference have no counterpart here.
cutile_status_t cutile_launch_fmha_prefill_gqa_lpt_raw_f16(cutile_stream_t stream, const void* q, const void* k, const void* v,
                                                           void* out, float qk_scale, int32_t query_group_size, int32_t q_len,
                                                           int32_t kv_len, int32_t query_start, int32_t num_head_groups,
                                                           int32_t group, int32_t d, int32_t causal,
                                                           const cutile_launch_opts_t* opts) {
  CUTILE_REQUIRE(q && k && v && out, CUTILE_ERR_INVALID_ARGUMENT, "fmha_prefill_gqa_lpt: null device pointer");
  CUTILE_REQUIRE(q_len > 0 && kv_len >= 0 && num_head_groups > 0 && group > 0 && d > 0 && query_group_size > 0 &&
                     ((int64_t)num_head_groups * group) % query_group_size == 0,
                 CUTILE_ERR_KERNEL_LAUNCH, "fmha_prefill_gqa_lpt: q_len, head groups, GROUP and D must be positive and the heads a multiple of query_group_size");
  const int32_t q_heads = num_head_groups * group, kv_heads = q_heads / query_group_size;
  auto t3 = [&](const void* p, int32_t a, int32_t b) {
    cutile_tensor_arg_t t{};
    t.ptr = const_cast<void*>(p);
    t.dtype = CUTILE_DTYPE_F16;
    t.rank = 3;
    t.shape[0] = a, t.shape[1] = b, t.shape[2] = d;
    t.strides[0] = b * d, t.strides[1] = d, t.strides[2] = 1;
    return t;
  };
  // the reference views k and v as [kv_heads, kv_len, D] with kv_len rows per head (:66-72)
  cutile_tensor_arg_t qt = t3(q, q_len, q_heads), kt = t3(k, kv_heads, std::max(kv_len, 1)), vt = t3(v, kv_heads, std::max(kv_len, 1));
  cutile_partition_arg_t op{};
  op.tensor = t3(out, q_len, q_heads);
  const int32_t bm = std::max(1, generic_int(opts, 0, 64));
  op.partition_shape[0] = bm, op.partition_shape[1] = group, op.partition_shape[2] = d;
  for (int i = 0; i < 3; ++i) op.partition_strides[i] = op.tensor.strides[i];
  if (cutile_status_t s = check_generic(opts, 2, std::to_string(d), "D")) return s;
  if (cutile_status_t s = check_generic(opts, 3, std::to_string(group), "GROUP")) return s;
  cutile_launch_opts_t o = opts ? *opts : cutile_launch_opts_t{};
  o.generics = nullptr;
  o.n_generics = 0;
  return cutile_launch_fmha_seq_f16(stream, &qt, &kt, &vt, &op, qk_scale, query_group_size, kv_len, query_start, nullptr, 0, causal, &o);
}

cutile_status_t cutile_launch_linear_tile_mxfp8(cutile_stream_t stream, const cutile_partition_arg_t* z,
                                                const cutile_tensor_arg_t* x, const cutile_tensor_arg_t* y,
                                                const cutile_tensor_arg_t* xs, const cutile_tensor_arg_t* ys, float alpha,
                                                const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_partition(z, "z", 2, 2)) return s;
  if (cutile_status_t s = check_tensor(x, "x", 2, 2)) return s;
  if (cutile_status_t s = check_tensor(y, "y", 2, 2)) return s;
  if (cutile_status_t s = check_tensor(xs, "x_scales", 2, 2)) return s;
  if (cutile_status_t s = check_tensor(ys, "y_scales", 2, 2)) return s;
  const cutile_tensor_arg_t& zt = z->tensor;
  CUTILE_REQUIRE(x->dtype == CUTILE_DTYPE_F8E4M3FN && y->dtype == CUTILE_DTYPE_F8E4M3FN &&
                     xs->dtype == CUTILE_DTYPE_F8E8M0FNU && ys->dtype == CUTILE_DTYPE_F8E8M0FNU,
                 CUTILE_ERR_KERNEL_NOT_FOUND, "linear_tile: precompiled variants take f8e4m3fn data with f8e8m0fnu scales");
  CUTILE_REQUIRE(zt.dtype == CUTILE_DTYPE_F32 || zt.dtype == CUTILE_DTYPE_BF16, CUTILE_ERR_KERNEL_NOT_FOUND,
                 "linear_tile: z must be f32 or bf16");
  const int32_t M = x->shape[0], K = x->shape[1], N = y->shape[0];
  CUTILE_REQUIRE(y->shape[1] == K, CUTILE_ERR_KERNEL_LAUNCH, "linear_tile: x is [%d, %d] but y is [%d, %d]", M, K, N, y->shape[1]);
  CUTILE_REQUIRE(K % 32 == 0 && xs->shape[0] == M && xs->shape[1] == K / 32 && ys->shape[0] == N && ys->shape[1] == K / 32,
                 CUTILE_ERR_KERNEL_LAUNCH, "linear_tile: scales must be [M, K/32] and [N, K/32] with K a multiple of 32");
  CUTILE_REQUIRE(zt.shape[0] == M && zt.shape[1] == N, CUTILE_ERR_KERNEL_LAUNCH, "linear_tile: z is [%d, %d], expected [%d, %d]",
                 zt.shape[0], zt.shape[1], M, N);
  const int32_t bm = z->partition_shape[0], bn = z->partition_shape[1];
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(bm), "BM")) return s;
  if (cutile_status_t s = check_generic(opts, 1, std::to_string(bn), "BN")) return s;
  const int bk_user = generic_int(opts, 2, 128);
  CUTILE_REQUIRE(bk_user > 0 && bk_user % 32 == 0 && generic_int(opts, 3, bk_user / 32) == bk_user / 32,
                 CUTILE_ERR_KERNEL_LAUNCH, "linear_tile: BK must be a multiple of 32 and BK_SCALES = BK/32");
  CUTILE_REQUIRE(K % bk_user == 0, CUTILE_ERR_KERNEL_LAUNCH, "linear_tile: K = %d is not a multiple of BK = %d", K, bk_user);
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(z, opts, tg)) return s;
  uint32_t full[3];
  cutile_partition_grid(z, full);
  const bool full_cover = tg[0] == full[0] && tg[1] == full[1];
  CUTILE_REQUIRE(K % 128 == 0 && x->strides[1] == 1 && y->strides[1] == 1 && xs->strides[1] == 1 && ys->strides[1] == 1 &&
                     zt.strides[1] == 1 && x->strides[0] % 16 == 0 && y->strides[0] % 16 == 0 && xs->strides[0] % 4 == 0 &&
                     ys->strides[0] % 4 == 0 && zt.strides[0] % 4 == 0 && zt.shape[1] % 4 == 0 && aligned16(x->ptr) &&
                     aligned16(y->ptr) && aligned16(zt.ptr) && ((uintptr_t)xs->ptr & 3) == 0 && ((uintptr_t)ys->ptr & 3) == 0,
                 CUTILE_ERR_KERNEL_NOT_FOUND,
                 "linear_tile: precompiled variants need K a multiple of 128, unit inner strides and aligned rows");
  CUTILE_REQUIRE(extent_bytes_2d(*x) < kDescriptorLimit && extent_bytes_2d(*y) < kDescriptorLimit && extent_bytes_2d(*xs) < kDescriptorLimit &&
                     extent_bytes_2d(*ys) < kDescriptorLimit && extent_bytes_2d(zt) < kDescriptorLimit,
                 CUTILE_ERR_KERNEL_NOT_FOUND,
                 "linear_tile: precompiled variants address an operand with 32-bit byte offsets: x, y, the scales and z must each end "
                 "below 2 GiB from their first element (x spans %lld bytes, y %lld, z %lld)",
                 (long long)extent_bytes_2d(*x), (long long)extent_bytes_2d(*y), (long long)extent_bytes_2d(zt));
  const std::string dt = zt.dtype == CUTILE_DTYPE_F32 ? "f32" : "bf16";
  // A kernel tile that is a whole multiple of the partition tile computes the
  // same output when the launch covers the whole tensor.
  std::vector<const KernelEntry*> fit;
  for (const auto& e : kernel_table())
    if (strcmp(e.function, "linear_tile") == 0 && dt == e.dtype &&
        ((e.tile[0] == bm && e.tile[1] == bn) || (full_cover && e.tile[0] % bm == 0 && e.tile[1] % bn == 0)))
      fit.push_back(&e);
  std::stable_sort(fit.begin(), fit.end(), [&](const KernelEntry* a, const KernelEntry* b) {
    bool ea = a->tile[0] == bm && a->tile[1] == bn, eb = b->tile[0] == bm && b->tile[1] == bn;
    if (ea != eb) return ea;
    return a->tile[0] * a->tile[1] < b->tile[0] * b->tile[1];
  });
  std::vector<std::string> acceptable;
  for (auto* e : fit) acceptable.push_back(e->variant);
  CUTILE_REQUIRE(!acceptable.empty(), CUTILE_ERR_KERNEL_NOT_FOUND,
                 "no precompiled variant of linear_tile<%d, %d, %d, %d> -> %s; available: %s", bm, bn, bk_user,
                 bk_user / 32, dt.c_str(), list_variants("linear_tile").c_str());
  Resolved res;
  BucketScope bucket("mxfp8_" + dt + "_" + std::to_string(bm) + "x" + std::to_string(bn));
  if (cutile_status_t s = resolve_entry("linear_tile", opts, acceptable[0], acceptable, &res)) return s;
  uint32_t kg[3] = {tg[0], tg[1], 1};
  if (res.entry->tile[0] != bm || res.entry->tile[1] != bn) {
    kg[0] = div_up(M, res.entry->tile[0]);
    kg[1] = div_up(N, res.entry->tile[1]);
  }
  ArgPacker args;
  args.push_partition(*z);
  args.push_tensor(*x);
  args.push_tensor(*y);
  args.push_tensor(*xs);
  args.push_tensor(*ys);
  args.push_val<float>(alpha);
  args.push_tile_grid(kg);
  uint32_t grid[3] = {kg[0] * kg[1], 1, 1};
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

cutile_status_t cutile_launch_linear_tile_nvfp4(cutile_stream_t stream, const cutile_partition_arg_t* z,
                                                const cutile_tensor_arg_t* x, const cutile_tensor_arg_t* y,
                                                const cutile_tensor_arg_t* xs, const cutile_tensor_arg_t* ys, float alpha,
                                                const cutile_launch_opts_t* opts) {
  if (cutile_status_t s = check_partition(z, "z", 2, 2)) return s;
  if (cutile_status_t s = check_tensor(x, "x", 2, 2)) return s;
  if (cutile_status_t s = check_tensor(y, "y", 2, 2)) return s;
  if (cutile_status_t s = check_tensor(xs, "x_scales", 2, 2)) return s;
  if (cutile_status_t s = check_tensor(ys, "y_scales", 2, 2)) return s;
  const cutile_tensor_arg_t& zt = z->tensor;
  CUTILE_REQUIRE(x->dtype == CUTILE_DTYPE_F4E2M1FNX2 && y->dtype == CUTILE_DTYPE_F4E2M1FNX2 &&
                     xs->dtype == CUTILE_DTYPE_F8E4M3FN && ys->dtype == CUTILE_DTYPE_F8E4M3FN,
                 CUTILE_ERR_KERNEL_NOT_FOUND, "linear_tile (nvfp4): precompiled variants take f4e2m1fnx2 data with f8e4m3fn scales");
  CUTILE_REQUIRE(zt.dtype == CUTILE_DTYPE_F32 || zt.dtype == CUTILE_DTYPE_BF16, CUTILE_ERR_KERNEL_NOT_FOUND,
                 "linear_tile (nvfp4): z must be f32 or bf16");
  const int32_t M = x->shape[0], KP = x->shape[1], N = y->shape[0];
  const int64_t K = 2 * (int64_t)KP;
  CUTILE_REQUIRE(y->shape[1] == KP, CUTILE_ERR_KERNEL_LAUNCH, "linear_tile (nvfp4): x is [%d, %d] but y is [%d, %d] (packed bytes)", M,
                 KP, N, y->shape[1]);
  CUTILE_REQUIRE(K % 16 == 0 && xs->shape[0] == M && xs->shape[1] == K / 16 && ys->shape[0] == N && ys->shape[1] == K / 16,
                 CUTILE_ERR_KERNEL_LAUNCH, "linear_tile (nvfp4): scales must be [M, K/16] and [N, K/16] with K = %lld a multiple of 16",
                 (long long)K);
  CUTILE_REQUIRE(zt.shape[0] == M && zt.shape[1] == N, CUTILE_ERR_KERNEL_LAUNCH,
                 "linear_tile (nvfp4): z is [%d, %d], expected [%d, %d]", zt.shape[0], zt.shape[1], M, N);
  const int32_t bm = z->partition_shape[0], bn = z->partition_shape[1];
  if (cutile_status_t s = check_generic(opts, 0, std::to_string(bm), "BM")) return s;
  if (cutile_status_t s = check_generic(opts, 1, std::to_string(bn), "BN")) return s;
  const int bk_user = generic_int(opts, 2, 64);
  CUTILE_REQUIRE(bk_user > 0 && bk_user % 16 == 0 && generic_int(opts, 3, bk_user / 2) == bk_user / 2 &&
                     generic_int(opts, 4, bk_user / 16) == bk_user / 16,
                 CUTILE_ERR_KERNEL_LAUNCH, "linear_tile (nvfp4): BK must be a multiple of 16, BK_PACKED = BK/2 and BK_SCALES = BK/16");
  // the tile program runs K / BK whole K tiles
  CUTILE_REQUIRE(K % bk_user == 0, CUTILE_ERR_KERNEL_LAUNCH, "linear_tile (nvfp4): K = %lld is not a multiple of BK = %d", (long long)K,
                 bk_user);
  uint32_t tg[3];
  if (cutile_status_t s = resolve_grid(z, opts, tg)) return s;
  uint32_t full[3];
  cutile_partition_grid(z, full);
  const bool full_cover = tg[0] == full[0] && tg[1] == full[1];
  CUTILE_REQUIRE(K % 64 == 0 && x->strides[1] == 1 && y->strides[1] == 1 && xs->strides[1] == 1 && ys->strides[1] == 1 &&
                     zt.strides[1] == 1 && x->strides[0] % 16 == 0 && y->strides[0] % 16 == 0 && xs->strides[0] % 2 == 0 &&
                     ys->strides[0] % 2 == 0 && zt.strides[0] % 4 == 0 && zt.shape[1] % 4 == 0 && aligned16(x->ptr) &&
                     aligned16(y->ptr) && aligned16(zt.ptr) && ((uintptr_t)xs->ptr & 1) == 0 && ((uintptr_t)ys->ptr & 1) == 0,
                 CUTILE_ERR_KERNEL_NOT_FOUND,
                 "linear_tile (nvfp4): precompiled variants need K a multiple of 64, unit inner strides and aligned rows");
  CUTILE_REQUIRE(extent_bytes_2d(*x) < kDescriptorLimit && extent_bytes_2d(*y) < kDescriptorLimit && extent_bytes_2d(*xs) < kDescriptorLimit &&
                     extent_bytes_2d(*ys) < kDescriptorLimit && extent_bytes_2d(zt) < kDescriptorLimit,
                 CUTILE_ERR_KERNEL_NOT_FOUND,
                 "linear_tile (nvfp4): precompiled variants address an operand with 32-bit byte offsets: x, y, the scales and z must each "
                 "end below 2 GiB from their first element (x spans %lld bytes, y %lld, z %lld)",
                 (long long)extent_bytes_2d(*x), (long long)extent_bytes_2d(*y), (long long)extent_bytes_2d(zt));
  const std::string dt = zt.dtype == CUTILE_DTYPE_F32 ? "f32" : "bf16";
  // A kernel tile that is a whole multiple of the partition tile computes the same output when the
  // launch covers the whole tensor (the reference example's 16x16 tiles run on the 32x32 kernel).
  std::vector<const KernelEntry*> fit;
  for (const auto& e : kernel_table())
    if (strcmp(e.function, "linear_tile_nvfp4") == 0 && dt == e.dtype &&
        ((e.tile[0] == bm && e.tile[1] == bn) || (full_cover && e.tile[0] % bm == 0 && e.tile[1] % bn == 0)))
      fit.push_back(&e);
  std::stable_sort(fit.begin(), fit.end(), [&](const KernelEntry* a, const KernelEntry* b) {
    bool ea = a->tile[0] == bm && a->tile[1] == bn, eb = b->tile[0] == bm && b->tile[1] == bn;
    if (ea != eb) return ea;
    return a->tile[0] * a->tile[1] < b->tile[0] * b->tile[1];
  });
  std::vector<std::string> acceptable;
  for (auto* e : fit) acceptable.push_back(e->variant);
  CUTILE_REQUIRE(!acceptable.empty(), CUTILE_ERR_KERNEL_NOT_FOUND,
                 "no precompiled variant of nvfp4 linear_tile<%d, %d, %d, %d, %d> -> %s; available: %s", bm, bn, bk_user, bk_user / 2,
                 bk_user / 16, dt.c_str(), list_variants("linear_tile_nvfp4").c_str());
  Resolved res;
  if (cutile_status_t s = resolve_entry("linear_tile_nvfp4", opts, acceptable[0], acceptable, &res)) return s;
  uint32_t kg[3] = {tg[0], tg[1], 1};
  if (res.entry->tile[0] != bm || res.entry->tile[1] != bn) {
    kg[0] = div_up(M, res.entry->tile[0]);
    kg[1] = div_up(N, res.entry->tile[1]);
  }
  ArgPacker args;
  args.push_partition(*z);
  args.push_tensor(*x);
  args.push_tensor(*y);
  args.push_tensor(*xs);
  args.push_tensor(*ys);
  args.push_val<float>(alpha);
  args.push_tile_grid(kg);
  uint32_t grid[3] = {kg[0] * kg[1], 1, 1};
  return launch_packed(res.fn, grid, res.entry->block, 0, stream, args);
}

}  // extern "C"

// ---- RNG (cuda-core/src/api.rs:214-293) --------------------------------------------------------------------------
struct cutile_rng {
  uint64_t seed = 0;
  uint64_t offset = 0;   // next Philox block of the stream
};

static cutile_status_t rng_fill(cutile_rng_t rng, const char* dtype, void* ptr, size_t n, int32_t kind, double mean, double std,
                                cutile_stream_t stream) {
  CUTILE_REQUIRE(rng, CUTILE_ERR_INVALID_ARGUMENT, "rng is null");
  CUTILE_REQUIRE(ptr || n == 0, CUTILE_ERR_INVALID_ARGUMENT, "rng fill: null device pointer");
  const bool is_f32 = strcmp(dtype, "f32") == 0;
  CUTILE_REQUIRE(((uintptr_t)ptr & (is_f32 ? 3u : 7u)) == 0, CUTILE_ERR_INVALID_ARGUMENT, "rng fill: misaligned device pointer");
  if (n == 0) return CUTILE_SUCCESS;
  Resolved res;
  if (cutile_status_t s = resolve_entry("rng_fill", nullptr, dtype, {dtype}, &res)) return s;
  const uint64_t per_block = is_f32 ? 4 : 2, blocks = ((uint64_t)n + per_block - 1) / per_block;
  ArgPacker args;
  args.push_val<void*>(ptr);
  args.push_val<uint64_t>((uint64_t)n);
  args.push_val<uint64_t>(rng->seed);
  args.push_val<uint64_t>(rng->offset);
  args.push_val<int32_t>(kind);
  if (is_f32) {
    args.push_val<float>((float)mean);
    args.push_val<float>((float)std);
  } else {
    args.push_val<double>(mean);
    args.push_val<double>(std);
  }
  // enough lanes to keep the stores streaming; each lane walks its blocks with the grid's stride
  uint32_t grid[3] = {std::max<uint32_t>(1, std::min<uint32_t>(div_up(blocks, 256), 8192)), 1, 1};
  if (cutile_status_t s = launch_packed(res.fn, grid, res.entry->block, 0, stream, args)) return s;
  // compile-only and specialize-only launches enqueue nothing and write no values: the stream position stays put
  if (g_launch_mode == 0) rng->offset += blocks;
  return CUTILE_SUCCESS;
}

extern "C" {
cutile_status_t cutile_rng_create(cutile_rng_t* rng) {
  CUTILE_REQUIRE(rng, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  *rng = new cutile_rng();
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_rng_set_seed(cutile_rng_t rng, uint64_t seed) {
  CUTILE_REQUIRE(rng, CUTILE_ERR_INVALID_ARGUMENT, "rng is null");
  rng->seed = seed;
  rng->offset = 0;
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_rng_set_offset(cutile_rng_t rng, uint64_t offset) {
  CUTILE_REQUIRE(rng, CUTILE_ERR_INVALID_ARGUMENT, "rng is null");
  rng->offset = offset;
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_rng_get_offset(cutile_rng_t rng, uint64_t* offset) {
  CUTILE_REQUIRE(rng && offset, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  *offset = rng->offset;
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_rng_normal_f32(cutile_rng_t rng, void* device_ptr, size_t num_elements, float mean, float std,
                                      cutile_stream_t stream) {
  return rng_fill(rng, "f32", device_ptr, num_elements, 1, mean, std, stream);
}
cutile_status_t cutile_rng_normal_f64(cutile_rng_t rng, void* device_ptr, size_t num_elements, double mean, double std,
                                      cutile_stream_t stream) {
  return rng_fill(rng, "f64", device_ptr, num_elements, 1, mean, std, stream);
}
cutile_status_t cutile_rng_uniform_f32(cutile_rng_t rng, void* device_ptr, size_t num_elements, cutile_stream_t stream) {
  return rng_fill(rng, "f32", device_ptr, num_elements, 0, 0.0, 1.0, stream);
}
cutile_status_t cutile_rng_uniform_f64(cutile_rng_t rng, void* device_ptr, size_t num_elements, cutile_stream_t stream) {
  return rng_fill(rng, "f64", device_ptr, num_elements, 0, 0.0, 1.0, stream);
}
cutile_status_t cutile_rng_destroy(cutile_rng_t rng) {
  delete rng;
  return CUTILE_SUCCESS;
}
}  // extern "C"

// ---- launch modes of the generated launcher (cutile-macro/src/_module.rs:852-900) -------------------------------
extern "C" {
cutile_status_t cutile_set_launch_mode(int32_t mode) {
  CUTILE_REQUIRE(mode >= 0 && mode <= 2, CUTILE_ERR_INVALID_ARGUMENT, "launch mode must be 0 (launch), 1 (compile only) or 2 (specialize only)");
  g_launch_mode = mode;
  return CUTILE_SUCCESS;
}
cutile_status_t cutile_get_launch_mode(int32_t* mode) {
  CUTILE_REQUIRE(mode, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  *mode = g_launch_mode;
  return CUTILE_SUCCESS;
}
const char* cutile_last_resolved_source(void) { return g_last_source.c_str(); }
const char* cutile_last_resolved_bucket(void) { return g_last_bucket.c_str(); }
cutile_status_t cutile_last_resolved_kernel(const char** function, cutile_kernel_info_t* info) {
  CUTILE_REQUIRE(function && info, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  CUTILE_REQUIRE(g_last_entry, CUTILE_ERR_STATE, "no launcher call has resolved a kernel on this thread yet");
  *function = g_last_entry->function;
  info->function = (cutile_function_t)g_last_fn;
  info->symbol = g_last_entry->symbol;
  info->variant = g_last_entry->variant;
  memcpy(info->block, g_last_entry->block, sizeof(info->block));
  info->lds_bytes = g_last_entry->lds_bytes;
  memcpy(info->tile, g_last_entry->tile, sizeof(info->tile));
  return CUTILE_SUCCESS;
}
}  // extern "C"

