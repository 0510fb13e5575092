// Launch-site specialization identity: CompileOptions, SpecializationBits, TileFunctionKey and Specialization,
// mirroring cutile-compiler/src/hints.rs:91-127, cutile-compiler/src/specialization.rs:21-174 and
// cutile/src/tile_kernel.rs:76-312.
//
// In the reference the key is the identity of a JIT-compiled kernel in the in-memory cache (L1) and, hashed
// together with the serialized Tile IR, of the on-disk cache (L2).  Here kernels are precompiled gfx950 code
// objects, so the key names *which* precompiled kernel a launch site resolves to and everything that could make
// another launch resolve differently: function, generics, stride / divisibility facts of every tensor argument,
// scalar hints, a constant grid, compile options, the code object's fingerprint (source_hash), the device and
// its architecture, the library version and the device compiler's identity.  Tensor extents are absent, as in
// the reference.  Keys are compared as whole structs; display_hash() is a 64-bit digest for log lines only.
#pragma once
#include <array>
#include <cstdint>
#include <cstdio>
#include <optional>
#include <string>
#include <utility>
#include <vector>

#include "../cutile_hip.h"

namespace cutile {

// hints.rs:91-127.  The hints steer NVIDIA's assembler in the reference; the precompiled kernels here were built
// with fixed choices, so the options only take part in the key (different options never share a key).
struct CompileOptions {
  std::optional<int32_t> occupancy_, num_cta_in_cga_, max_divisibility_, num_worker_warps_per_cta_;
  CompileOptions occupancy(int32_t v) && { occupancy_ = v; return std::move(*this); }
  CompileOptions num_cta_in_cga(int32_t v) && { num_cta_in_cga_ = v; return std::move(*this); }
  CompileOptions max_divisibility(int32_t v) && { max_divisibility_ = v; return std::move(*this); }
  CompileOptions num_worker_warps_per_cta(int32_t v) && { num_worker_warps_per_cta_ = v; return std::move(*this); }
  bool operator==(const CompileOptions& o) const {
    return occupancy_ == o.occupancy_ && num_cta_in_cga_ == o.num_cta_in_cga_ && max_divisibility_ == o.max_divisibility_ &&
           num_worker_warps_per_cta_ == o.num_worker_warps_per_cta_;
  }
  bool operator!=(const CompileOptions& o) const { return !(*this == o); }
};

// specialization.rs:21-72: the largest power of two dividing a value, clamped to `max` (16 unless overridden).
struct DivHint {
  int32_t divisor = 1;
  int32_t max = 16;
  static DivHint from_value(int64_t v) {
    uint64_t a = v < 0 ? (uint64_t)(-v) : (uint64_t)v;
    int32_t d = 1;
    if (a == 0) d = 16;                          // zero is divisible by everything: the clamp decides
    else while (d < 16 && (a & 1) == 0) { d *= 2; a >>= 1; }
    return DivHint{d, 16};
  }
  static DivHint from_ptr(uint64_t p) { return from_value((int64_t)(p & 0xffu) | (p ? 0x100 : 0)); }   // in bytes
  DivHint with_max(int32_t m) const { return DivHint{divisor < m ? divisor : m, m}; }
  bool operator==(const DivHint& o) const { return divisor == o.divisor && max == o.max; }
  bool operator!=(const DivHint& o) const { return !(*this == o); }
};

// specialization.rs:62-174
struct SpecializationBits {
  std::vector<DivHint> shape_div, stride_div;
  std::vector<bool> stride_one;
  DivHint base_ptr_div;
  bool elements_disjoint = true;
  // from the C ABI's record of a tensor argument (cutile_compute_spec)
  static SpecializationBits from_tensor_arg(const cutile_tensor_arg_t& t, int32_t max_divisibility = 16) {
    cutile_spec_bits_t b{};
    SpecializationBits s;
    if (cutile_compute_spec(&t, &b) != CUTILE_SUCCESS) return s;
    auto cap = [&](int32_t v) { return DivHint{v, 16}.with_max(max_divisibility); };
    for (int i = 0; i < t.rank; ++i) {
      s.shape_div.push_back(cap(b.shape_div[i]));
      s.stride_div.push_back(cap(b.stride_div[i]));
      s.stride_one.push_back(b.stride_one[i] != 0);
    }
    s.base_ptr_div = cap(b.base_ptr_div);
    s.elements_disjoint = b.elements_disjoint != 0;
    return s;
  }
  bool operator==(const SpecializationBits& o) const {
    return shape_div == o.shape_div && stride_div == o.stride_div && stride_one == o.stride_one && base_ptr_div == o.base_ptr_div &&
           elements_disjoint == o.elements_disjoint;
  }
  bool operator!=(const SpecializationBits& o) const { return !(*this == o); }
};

class TileFunctionKeyBuilder;

// tile_kernel.rs:76-114
class TileFunctionKey {
 public:
  static TileFunctionKeyBuilder builder(std::string module_name, std::string function_name);
  const std::string& module_name() const { return module_name_; }
  const std::string& function_name() const { return function_name_; }
  std::vector<std::string> function_generics;
  std::vector<std::pair<std::string, std::vector<int32_t>>> stride_args;   // per tensor: 1 where the stride is 1, else 0
  std::vector<std::pair<std::string, SpecializationBits>> spec_args;
  std::vector<std::pair<std::string, DivHint>> scalar_hints;
  std::optional<std::array<uint32_t, 3>> grid;
  CompileOptions compile_options;
  const std::string& source_hash() const { return source_hash_; }
  size_t device_id() const { return device_id_; }
  const std::string& gpu_name() const { return gpu_name_; }
  const std::string& compiler_version() const { return compiler_version_; }
  const std::string& toolchain_fingerprint() const { return toolchain_fingerprint_; }

  bool operator==(const TileFunctionKey& o) const {
    return module_name_ == o.module_name_ && function_name_ == o.function_name_ && function_generics == o.function_generics &&
           stride_args == o.stride_args && spec_args == o.spec_args && scalar_hints == o.scalar_hints && grid == o.grid &&
           compile_options == o.compile_options && source_hash_ == o.source_hash_ && device_id_ == o.device_id_ &&
           gpu_name_ == o.gpu_name_ && compiler_version_ == o.compiler_version_ && toolchain_fingerprint_ == o.toolchain_fingerprint_;
  }
  bool operator!=(const TileFunctionKey& o) const { return !(*this == o); }

  // Every field, each behind its length, so that no two different keys serialize alike ("sm_9" + "0" vs "sm_90" + "").
  std::string canonical() const {
    std::string out;
    auto str = [&](const std::string& s) { out += std::to_string(s.size()); out += ':'; out += s; out += ';'; };
    auto num = [&](int64_t v) { out += std::to_string(v); out += ';'; };
    str(module_name_); str(function_name_);
    num((int64_t)function_generics.size());
    for (auto& g : function_generics) str(g);
    num((int64_t)stride_args.size());
    for (auto& [n, v] : stride_args) { str(n); num((int64_t)v.size()); for (int32_t x : v) num(x); }
    num((int64_t)spec_args.size());
    for (auto& [n, b] : spec_args) {
      str(n); num((int64_t)b.shape_div.size());
      for (auto d : b.shape_div) num(d.divisor);
      for (auto d : b.stride_div) num(d.divisor);
      for (bool x : b.stride_one) num(x);
      num(b.base_ptr_div.divisor); num(b.elements_disjoint);
    }
    num((int64_t)scalar_hints.size());
    for (auto& [n, d] : scalar_hints) { str(n); num(d.divisor); }
    if (grid) { out += "g;"; num((*grid)[0]); num((*grid)[1]); num((*grid)[2]); } else out += "-;";
    auto opt = [&](const std::optional<int32_t>& v) { if (v) num(*v); else out += "-;"; };
    opt(compile_options.occupancy_); opt(compile_options.num_cta_in_cga_); opt(compile_options.max_divisibility_);
    opt(compile_options.num_worker_warps_per_cta_);
    str(source_hash_); num((int64_t)device_id_); str(gpu_name_); str(compiler_version_); str(toolchain_fingerprint_);
    return out;
  }
  // 64-bit FNV-1a of the canonical form: for log lines, never for identity.
  uint64_t display_hash() const {
    uint64_t h = 0xcbf29ce484222325ull;
    for (unsigned char c : canonical()) { h ^= c; h *= 0x100000001b3ull; }
    return h;
  }

 private:
  friend class TileFunctionKeyBuilder;
  std::string module_name_, function_name_, source_hash_;
  size_t device_id_ = 0;
  std::string gpu_name_, compiler_version_, toolchain_fingerprint_;
};

// tile_kernel.rs:116-215
class TileFunctionKeyBuilder {
 public:
  TileFunctionKeyBuilder(std::string module_name, std::string function_name) {
    k_.module_name_ = std::move(module_name);
    k_.function_name_ = std::move(function_name);
  }
  TileFunctionKeyBuilder generics(std::vector<std::string> g) && { k_.function_generics = std::move(g); return std::move(*this); }
  TileFunctionKeyBuilder stride_args(std::vector<std::pair<std::string, std::vector<int32_t>>> v) && { k_.stride_args = std::move(v); return std::move(*this); }
  TileFunctionKeyBuilder spec_args(std::vector<std::pair<std::string, SpecializationBits>> v) && { k_.spec_args = std::move(v); return std::move(*this); }
  TileFunctionKeyBuilder scalar_hints(std::vector<std::pair<std::string, DivHint>> v) && { k_.scalar_hints = std::move(v); return std::move(*this); }
  TileFunctionKeyBuilder grid(uint32_t x, uint32_t y, uint32_t z) && { k_.grid = std::array<uint32_t, 3>{x, y, z}; return std::move(*this); }
  TileFunctionKeyBuilder compile_options(CompileOptions o) && { k_.compile_options = std::move(o); return std::move(*this); }
  TileFunctionKeyBuilder source_hash(std::string h) && { k_.source_hash_ = std::move(h); return std::move(*this); }
  TileFunctionKeyBuilder device_id(size_t id) && { k_.device_id_ = id; return std::move(*this); }
  TileFunctionKeyBuilder gpu_name(std::string n) && { k_.gpu_name_ = std::move(n); return std::move(*this); }
  TileFunctionKeyBuilder compiler_version(std::string v) && { k_.compiler_version_ = std::move(v); return std::move(*this); }
  // identity of the device compiler that built the code objects (the reference's `tileiras --version`)
  TileFunctionKeyBuilder toolchain_fingerprint(std::string f) && { k_.toolchain_fingerprint_ = std::move(f); return std::move(*this); }
  TileFunctionKey build() && { return std::move(k_); }

 private:
  TileFunctionKey k_;
};
inline TileFunctionKeyBuilder TileFunctionKey::builder(std::string module_name, std::string function_name) {
  return TileFunctionKeyBuilder(std::move(module_name), std::move(function_name));
}

// tile_kernel.rs:231-312: a resolved launch-site specialization.  l1_cache_key() is the structured key; the
// persistent key names the precompiled kernel the launch resolved to (function, variant, entry symbol, code object
// fingerprint) instead of hashing Tile IR bytecode, which does not exist here.
class Specialization {
 public:
  Specialization(TileFunctionKey key, std::string variant, std::string symbol) : key_(std::move(key)), variant_(std::move(variant)), symbol_(std::move(symbol)) {}
  const TileFunctionKey& l1_cache_key() const { return key_; }
  TileFunctionKey into_l1_cache_key() && { return std::move(key_); }
  const std::string& variant() const { return variant_; }
  const std::string& symbol() const { return symbol_; }
  std::string l2_cache_key() const {
    char buf[17];
    snprintf(buf, sizeof(buf), "%016llx", (unsigned long long)key_.display_hash());
    return key_.function_name() + ":" + variant_ + ":" + key_.source_hash() + ":" + buf;
  }

 private:
  TileFunctionKey key_;
  std::string variant_, symbol_;
};

}  // namespace cutile
