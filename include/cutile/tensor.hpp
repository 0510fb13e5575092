// Tensor, Partition, TensorView: device memory with shape/stride metadata and the
// ownership forms a kernel launcher accepts and hands back.
//
// Mirrors cutile/src/tensor.rs: Storage :589-646, Tensor :649-1234, TensorView
// :1252-1397, Partition :252-527,1417-1541, KernelInput/KernelOutput
// :1687-2107; DeviceBuffer cuda-async/src/device_buffer.rs:40-226.
//
// Ownership forms (the reference's "you get back what you put in"):
//   read-only kernel parameter   Tensor<T> (moved in, moved back out),
//                                std::shared_ptr<Tensor<T>> (Arc), const Tensor<T>* (borrow),
//                                TensorView<T> (borrowed sub-region)
//   mutable kernel parameter     Partition<Tensor<T>> (owned, unique storage) or
//                                Partition<Tensor<T>*> (in-place, "(&mut t).partition(..)")
#pragma once
#include <array>
#include <cstring>
#include <limits>
#include <optional>
#include <memory>
#include <numeric>
#include <vector>

#include "device_op.hpp"

namespace cutile {

// ---- element types (cuda-core/src/dtype.rs:25-47,123-229) ------------------------------------
struct f16 { uint16_t bits; };
struct bf16 { uint16_t bits; };
struct f8e4m3fn { uint8_t bits; };
struct f8e8m0fnu { uint8_t bits; };
// Packed pair of e2m1 values in one byte: the low nibble is the first logical value (dtype.rs:60-99).
struct f4e2m1fnx2 {
  uint8_t bits;
  static constexpr f4e2m1fnx2 from_bits(uint8_t b) { return {b}; }
  static constexpr f4e2m1fnx2 from_nibbles(uint8_t low, uint8_t high) { return {(uint8_t)((low & 0x0F) | ((high & 0x0F) << 4))}; }
  constexpr uint8_t low() const { return bits & 0x0F; }
  constexpr uint8_t high() const { return bits >> 4; }
};

template <class T> struct DType;
#define CUTILE_DTYPE(T, CODE) \
  template <> struct DType<T> { static constexpr cutile_dtype_t id = CODE; static const char* name() { return cutile_dtype_name(CODE); } };
CUTILE_DTYPE(float, CUTILE_DTYPE_F32)
CUTILE_DTYPE(double, CUTILE_DTYPE_F64)
CUTILE_DTYPE(f16, CUTILE_DTYPE_F16)
CUTILE_DTYPE(bf16, CUTILE_DTYPE_BF16)
CUTILE_DTYPE(int8_t, CUTILE_DTYPE_I8)
CUTILE_DTYPE(int16_t, CUTILE_DTYPE_I16)
CUTILE_DTYPE(int32_t, CUTILE_DTYPE_I32)
CUTILE_DTYPE(int64_t, CUTILE_DTYPE_I64)
CUTILE_DTYPE(uint8_t, CUTILE_DTYPE_U8)
CUTILE_DTYPE(uint16_t, CUTILE_DTYPE_U16)
CUTILE_DTYPE(uint32_t, CUTILE_DTYPE_U32)
CUTILE_DTYPE(uint64_t, CUTILE_DTYPE_U64)
CUTILE_DTYPE(bool, CUTILE_DTYPE_BOOL)
CUTILE_DTYPE(f8e4m3fn, CUTILE_DTYPE_F8E4M3FN)
CUTILE_DTYPE(f8e8m0fnu, CUTILE_DTYPE_F8E8M0FNU)
CUTILE_DTYPE(f4e2m1fnx2, CUTILE_DTYPE_F4E2M1FNX2)
#undef CUTILE_DTYPE
// Host-side conversions of the 16-bit float storage types (round to nearest even).
inline bf16 bf16_from_f32(float f) {
  uint32_t x;
  std::memcpy(&x, &f, 4);
  if ((x & 0x7fffffffu) > 0x7f800000u) return {(uint16_t)((x >> 16) | 0x40u)};
  x += 0x7fffu + ((x >> 16) & 1u);
  return {(uint16_t)(x >> 16)};
}
inline float f32_from_bf16(bf16 h) {
  uint32_t x = (uint32_t)h.bits << 16;
  float f;
  std::memcpy(&f, &x, 4);
  return f;
}
inline f16 f16_from_f32(float f) {
  uint32_t x;
  std::memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u, abs = x & 0x7fffffffu;
  if (abs >= 0x7f800000u) return {(uint16_t)(sign | 0x7c00u | (abs > 0x7f800000u ? 0x0200u : 0))};
  if (abs >= 0x477ff000u) return {(uint16_t)(sign | 0x7c00u)};
  if (abs < 0x38800000u) {
    if (abs < 0x33000000u) return {(uint16_t)sign};
    int e = (int)(abs >> 23);
    uint32_t man = (abs & 0x7fffffu) | 0x800000u;
    int shift = 126 - e;
    uint32_t q = man >> shift, rem = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return {(uint16_t)(sign | q)};
  }
  uint32_t h = (((abs >> 23) - 112u) << 10) | ((abs & 0x7fffffu) >> 13);
  uint32_t rem = abs & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
  return {(uint16_t)(sign | h)};
}
inline float f32_from_f16(f16 h) {
  uint32_t sign = ((uint32_t)h.bits & 0x8000u) << 16, e = (h.bits >> 10) & 0x1fu, man = h.bits & 0x3ffu, x;
  if (e == 0) {
    float v = (float)man * (1.0f / 16777216.0f);
    return sign ? -v : v;
  }
  x = e == 31 ? (sign | 0x7f800000u | (man << 13)) : (sign | ((e + 112u) << 23) | (man << 13));
  float f;
  std::memcpy(&f, &x, 4);
  return f;
}
// one(): the value tests fill operands with (dtype.rs:225-227)
inline f8e4m3fn f8e4m3fn_one() { return {0x38}; }
inline f8e8m0fnu f8e8m0fnu_one() { return {0x7F}; }
inline f4e2m1fnx2 f4e2m1fnx2_one() { return f4e2m1fnx2::from_nibbles(0x2, 0x2); }   // dtype.rs:228

// ---- device allocations (device_buffer.rs:40-226) --------------------------------------------
// An allocation owned by another runtime, lent to a tensor (DeviceAllocation trait).
struct DeviceAllocation {
  virtual ~DeviceAllocation() = default;
  virtual void* device_ptr() const = 0;
  virtual size_t len_bytes() const = 0;
  virtual int device_id() const = 0;
};

class Storage {
 public:
  enum class Kind { Owned, Borrowed, Foreign, Meta };
  static constexpr uintptr_t kMetaSpecPtr = 16;  // Storage::META_SPEC_PTR

  static std::shared_ptr<Storage> owned(void* p, size_t bytes, int device) { return make(Kind::Owned, p, bytes, device, nullptr); }
  static std::shared_ptr<Storage> borrowed(void* p, size_t bytes, int device) { return make(Kind::Borrowed, p, bytes, device, nullptr); }
  static std::shared_ptr<Storage> foreign(std::shared_ptr<DeviceAllocation> owner, size_t bytes) {
    void* p = owner->device_ptr();
    int dev = owner->device_id();
    return make(Kind::Foreign, p, bytes, dev, std::move(owner));
  }
  static std::shared_ptr<Storage> meta(size_t bytes, int device) { return make(Kind::Meta, nullptr, bytes, device, nullptr); }

  // Owned memory is freed asynchronously on the thread's deallocator stream;
  // borrowed and foreign memory is left alone (device_buffer.rs:128-149).
  ~Storage() {
    if (kind_ == Kind::Owned && ptr_) {
      cutile_stream_t s = nullptr;
      if (cutile_deallocator_stream(device_, &s) == CUTILE_SUCCESS) cutile_free_async(ptr_, s);
    }
  }
  Storage(const Storage&) = delete;
  Kind kind() const { return kind_; }
  size_t len_bytes() const { return bytes_; }
  int device_id() const { return device_; }
  // Reading the pointer of a meta tensor is a programmer error (tensor.rs:612-624).
  void* device_ptr() const {
    if (kind_ == Kind::Meta)
      throw std::logic_error(
          "cutile: read of a meta tensor's device pointer. Meta tensors carry only shape/stride metadata; they have "
          "no device memory and cannot be launched or copied.");
    return ptr_;
  }
  uintptr_t spec_ptr() const { return kind_ == Kind::Meta ? kMetaSpecPtr : (uintptr_t)ptr_; }

 private:
  static std::shared_ptr<Storage> make(Kind k, void* p, size_t b, int d, std::shared_ptr<DeviceAllocation> o) {
    auto s = std::shared_ptr<Storage>(new Storage());
    s->kind_ = k; s->ptr_ = p; s->bytes_ = b; s->device_ = d; s->owner_ = std::move(o);
    return s;
  }
  Storage() = default;
  Kind kind_ = Kind::Meta;
  void* ptr_ = nullptr;
  size_t bytes_ = 0;
  int device_ = 0;
  std::shared_ptr<DeviceAllocation> owner_;
};

// ---- shape helpers ---------------------------------------------------------------------------
inline std::vector<int32_t> contiguous_strides(const std::vector<int32_t>& shape) {
  std::vector<int32_t> st(shape.size());
  int64_t s = 1;
  for (size_t i = shape.size(); i-- > 0;) {
    st[i] = (int32_t)s;
    s *= shape[i];
  }
  return st;
}
inline std::optional<size_t> checked_num_elements(const std::vector<int32_t>& shape) {
  size_t n = 1;
  for (int32_t d : shape) {
    if (d < 0) return std::nullopt;
    if (d != 0 && n > std::numeric_limits<size_t>::max() / (size_t)d) return std::nullopt;
    n *= (size_t)d;
  }
  return n;
}
// Bytes a (shape, strides) pair can address, from the base pointer (tensor.rs addressable_bytes).
template <class T>
size_t addressable_bytes(const std::vector<int32_t>& shape, const std::vector<int32_t>& strides) {
  unsigned __int128 last = 0;
  for (size_t i = 0; i < shape.size(); ++i) {
    if (shape[i] == 0) return 0;
    last += (unsigned __int128)(shape[i] - 1) * (unsigned __int128)(strides[i] < 0 ? 0 : strides[i]);
  }
  unsigned __int128 bytes = (last + 1) * sizeof(T);
  if (bytes > (unsigned __int128)std::numeric_limits<size_t>::max()) throw std::logic_error("addressable extent overflowed");
  return (size_t)bytes;
}

template <class T> class Tensor;
template <class T> class TensorView;
template <class X> class Partition;
template <class P> class MappedLaunchPartition;

// ---- Tensor ----------------------------------------------------------------------------------
template <class T>
class Tensor {
 public:
  using Elem = T;
  Tensor(Tensor&&) = default;
  Tensor& operator=(Tensor&&) = default;
  Tensor(const Tensor&) = delete;  // tensors move; share with shared_ptr<Tensor<T>>

  // from_raw_parts: takes ownership of an allocation (tensor.rs:781-795).
  static Tensor from_raw_parts(void* ptr, size_t len_bytes, int device, std::vector<int32_t> shape, std::vector<int32_t> strides) {
    assert_valid_metadata(shape, strides, len_bytes);
    return Tensor(Storage::owned(ptr, len_bytes, device), std::move(shape), std::move(strides));
  }
  // borrow_raw_parts: memory owned elsewhere, never freed here (tensor.rs:797-810).
  static Tensor borrow_raw_parts(void* ptr, int device, std::vector<int32_t> shape, std::vector<int32_t> strides) {
    auto n = checked_num_elements(shape);
    if (!n) throw std::logic_error("Tensor shape contains invalid dimensions or overflows.");
    return Tensor(Storage::borrowed(ptr, *n * sizeof(T), device), std::move(shape), std::move(strides));
  }
  // from_foreign: validates the ADDRESSABLE extent against the owner's size (tensor.rs:812-833).
  static Tensor from_foreign(std::shared_ptr<DeviceAllocation> owner, std::vector<int32_t> shape, std::vector<int32_t> strides) {
    auto n = checked_num_elements(shape);
    if (!n) throw std::logic_error("Tensor shape contains invalid dimensions or overflows.");
    size_t extent = addressable_bytes<T>(shape, strides);
    if (owner->len_bytes() < extent)
      throw std::logic_error("foreign allocation (" + std::to_string(owner->len_bytes()) +
                             " bytes) is smaller than the tensor's addressable extent (" + std::to_string(extent) +
                             " bytes for the given shape/strides)");
    return Tensor(Storage::foreign(std::move(owner), *n * sizeof(T)), std::move(shape), std::move(strides));
  }
  // from_meta: shape/stride metadata only, no memory (tensor.rs:915-936; api::meta).
  static Tensor from_meta(std::vector<int32_t> shape, int device = 0) {
    auto n = checked_num_elements(shape);
    if (!n) throw std::logic_error("Tensor shape contains invalid dimensions or overflows.");
    auto strides = contiguous_strides(shape);
    return Tensor(Storage::meta(*n * sizeof(T), device), std::move(shape), std::move(strides));
  }

  const std::vector<int32_t>& shape() const { return shape_; }
  const std::vector<int32_t>& strides() const { return strides_; }
  size_t size() const { return std::accumulate(shape_.begin(), shape_.end(), (size_t)1, [](size_t a, int32_t b) { return a * (size_t)b; }); }
  size_t num_bytes() const { return size() * sizeof(T); }
  int rank() const { return (int)shape_.size(); }
  int device_id() const { return storage_->device_id(); }
  bool is_contiguous() const { return strides_ == contiguous_strides(shape_); }
  bool is_meta() const { return storage_->kind() == Storage::Kind::Meta; }
  void* device_pointer() const { return storage_->device_ptr(); }
  long storage_use_count() const { return storage_.use_count(); }

  cutile_tensor_arg_t arg() const { return make_arg(storage_->device_ptr()); }
  cutile_spec_bits_t spec() const {
    cutile_tensor_arg_t a = make_arg((void*)storage_->spec_ptr());
    cutile_spec_bits_t s;
    cutile_compute_spec(&a, &s);
    return s;
  }

  // reshape: zero-copy, element count preserved, contiguous only (tensor.rs:1212-1234).
  Result<Tensor> reshape(std::vector<int32_t> new_shape) && {
    auto n = checked_num_elements(new_shape);
    if (!n || *n != size()) return DeviceError::tensor("reshape: element count must be preserved");
    if (!is_contiguous()) return DeviceError::tensor("reshape: tensor must be contiguous");
    auto st = contiguous_strides(new_shape);
    return Tensor(std::move(storage_), std::move(new_shape), std::move(st));
  }
  // (&arc).reshape: a new handle sharing the allocation.
  static Result<std::shared_ptr<Tensor>> reshape_shared(const std::shared_ptr<Tensor>& t, std::vector<int32_t> new_shape) {
    auto n = checked_num_elements(new_shape);
    if (!n || *n != t->size()) return DeviceError::tensor("reshape: element count must be preserved");
    if (!t->is_contiguous()) return DeviceError::tensor("reshape: tensor must be contiguous");
    auto st = contiguous_strides(new_shape);
    return std::shared_ptr<Tensor>(new Tensor(t->storage_, std::move(new_shape), std::move(st)));
  }
  // reinterpret<U>: same bytes, another element type (tensor.rs:1145-1165).
  template <class U>
  static Result<std::shared_ptr<Tensor<U>>> reinterpret(const std::shared_ptr<Tensor>& t, std::vector<int32_t> new_shape) {
    auto n = checked_num_elements(new_shape);
    if (!t->is_contiguous()) return DeviceError::tensor("reinterpret: tensor must be contiguous");
    if (!n || *n * sizeof(U) != t->num_bytes()) return DeviceError::tensor("reinterpret: total byte size must match");
    if (t->storage_->spec_ptr() % alignof(U) != 0) return DeviceError::tensor("reinterpret: pointer alignment is incompatible");
    auto st = contiguous_strides(new_shape);
    return std::shared_ptr<Tensor<U>>(new Tensor<U>(t->storage_, std::move(new_shape), std::move(st)));
  }
  // view / slice: borrowed sub-regions (tensor.rs:1252-1397).
  Result<TensorView<T>> view(std::vector<int32_t> new_shape) const;
  Result<TensorView<T>> slice(const std::vector<std::pair<int32_t, int32_t>>& ranges) const;

  // partition: consume the tensor into a mutable output partition; the storage
  // must be uniquely owned (tensor.rs:990-995,1417-1429).
  Partition<Tensor<T>> partition(std::vector<int32_t> tile) &&;
  Partition<Tensor<T>> partition_prefix(std::vector<int32_t> tile) &&;
  // (&mut t).partition(..): in-place partition of a tensor that stays with the caller.
  Partition<Tensor<T>*> partition_mut(std::vector<int32_t> tile) &;

 private:
  template <class U> friend class Tensor;
  template <class U> friend class TensorView;
  Tensor(std::shared_ptr<Storage> s, std::vector<int32_t> shape, std::vector<int32_t> strides)
      : storage_(std::move(s)), shape_(std::move(shape)), strides_(std::move(strides)) {
    if (shape_.size() != strides_.size() || shape_.size() > CUTILE_MAX_RANK)
      throw std::logic_error("Tensor: shape and strides must have the same rank (at most 4)");
  }
  static void assert_valid_metadata(const std::vector<int32_t>& shape, const std::vector<int32_t>&, size_t len_bytes) {
    auto n = checked_num_elements(shape);
    if (!n || *n * sizeof(T) != len_bytes)  // tensor.rs:739-752
      throw std::logic_error("Tensor: prod(shape) * sizeof(T) must equal the storage size in bytes");
  }
  cutile_tensor_arg_t make_arg(void* ptr) const {
    cutile_tensor_arg_t a{};
    a.ptr = ptr;
    a.dtype = DType<T>::id;
    a.rank = rank();
    for (int i = 0; i < rank(); ++i) {
      a.shape[i] = shape_[i];
      a.strides[i] = strides_[i];
    }
    return a;
  }
  std::shared_ptr<Storage> storage_;
  std::vector<int32_t> shape_, strides_;
};

// ---- TensorView ------------------------------------------------------------------------------
template <class T>
class TensorView {
 public:
  using Elem = T;
  const std::vector<int32_t>& shape() const { return shape_; }
  const std::vector<int32_t>& strides() const { return strides_; }
  size_t offset_bytes() const { return offset_bytes_; }
  // A view is pushed to a kernel as base pointer + byte offset (tensor.rs:2094-2107).
  cutile_tensor_arg_t arg() const {
    cutile_tensor_arg_t a{};
    a.ptr = static_cast<char*>(base_->device_pointer()) + offset_bytes_;
    a.dtype = DType<T>::id;
    a.rank = (int)shape_.size();
    for (size_t i = 0; i < shape_.size(); ++i) {
      a.shape[i] = shape_[i];
      a.strides[i] = strides_[i];
    }
    return a;
  }
  Result<TensorView> slice(const std::vector<std::pair<int32_t, int32_t>>& ranges) const {
    if (ranges.size() > shape_.size()) return DeviceError::tensor("slice: more ranges than dimensions");
    TensorView v = *this;
    for (size_t i = 0; i < ranges.size(); ++i) {
      auto [lo, hi] = ranges[i];
      if (lo < 0 || hi < lo || hi > shape_[i]) return DeviceError::tensor("slice: range out of bounds");
      v.offset_bytes_ += (size_t)lo * (size_t)strides_[i] * sizeof(T);
      v.shape_[i] = hi - lo;
    }
    return v;
  }

 private:
  friend class Tensor<T>;
  TensorView(const Tensor<T>* base, std::vector<int32_t> shape, std::vector<int32_t> strides, size_t off)
      : base_(base), shape_(std::move(shape)), strides_(std::move(strides)), offset_bytes_(off) {}
  const Tensor<T>* base_;
  std::vector<int32_t> shape_, strides_;
  size_t offset_bytes_;
};

template <class T>
Result<TensorView<T>> Tensor<T>::view(std::vector<int32_t> new_shape) const {
  auto n = checked_num_elements(new_shape);
  if (!n || *n != size()) return DeviceError::tensor("view: element count must be preserved");
  if (!is_contiguous()) return DeviceError::tensor("view: tensor must be contiguous");
  auto st = contiguous_strides(new_shape);
  return TensorView<T>(this, std::move(new_shape), std::move(st), 0);
}
template <class T>
Result<TensorView<T>> Tensor<T>::slice(const std::vector<std::pair<int32_t, int32_t>>& ranges) const {
  return TensorView<T>(this, shape_, strides_, 0).slice(ranges);
}

// ---- Partition -------------------------------------------------------------------------------
// GridBound (tensor.rs:1677-1685): an exact cover defines the launch grid, a prefix only bounds it.
template <class X>
class Partition {
 public:
  using Inner = X;  // Tensor<T> (owned) or Tensor<T>* (in place)
  Partition(X object, std::vector<int32_t> tile, bool prefix) : object_(std::move(object)), tile_(std::move(tile)), prefix_(prefix) {
    if ((int)tile_.size() != tensor().rank()) throw std::logic_error("partition: tile rank must match tensor rank");
    for (int32_t t : tile_)
      if (t <= 0) throw std::logic_error("partition: tile extents must be positive");
  }
  Partition(Partition&&) = default;
  Partition& operator=(Partition&&) = default;

  const auto& tensor() const {
    if constexpr (std::is_pointer_v<X>) return *object_;
    else return object_;
  }
  const std::vector<int32_t>& partition_shape() const { return tile_; }
  bool prefix_coverage() const { return prefix_; }
  // prefix(): turn an exact cover into an upper bound (tensor.rs:275-278).
  Partition prefix() && { prefix_ = true; return std::move(*this); }

  cutile_partition_arg_t arg() const {
    cutile_partition_arg_t p{};
    p.tensor = tensor().arg();
    for (int i = 0; i < tensor().rank(); ++i) {
      p.partition_shape[i] = tile_[i];
      p.partition_strides[i] = tensor().strides()[i];
    }
    p.prefix_coverage = prefix_ ? 1 : 0;
    return p;
  }
  // grid(): per-axis div_ceil, rank <= 3 (tensor.rs:447-468).
  Result<std::array<uint32_t, 3>> grid() const {
    std::array<uint32_t, 3> g{};
    cutile_partition_arg_t p = arg();
    CUTILE_TRY_STATUS(cutile_partition_grid(&p, g.data()));
    return g;
  }
  // unpartition(): recover the tensor (owned form), tensor.rs:1519-1541.
  X unpartition() && { return std::move(object_); }
  // map(): attach a host-side partition map (tensor.rs:314-329); defined after MappedLaunchPartition.
  MappedLaunchPartition<Partition<X>> map(std::vector<int32_t> map_shape, uint32_t num_tile_blocks) &&;

 private:
  X object_;
  std::vector<int32_t> tile_;
  bool prefix_;
};

// Map-shape sentinel of an owned axis (tensor.rs:331-337): the axis is not traversed by the stream of
// work items; each item owns its full extent and the kernel walks it.
constexpr int32_t OWNED = CUTILE_MAP_OWNED;

// MappedLaunchPartition (tensor.rs:339-401): the logical tile grid of `partition` is walked by
// `num_tile_blocks` tile blocks; the launch grid is (num_tile_blocks, 1, 1).  A kernel hands the inner
// partition back (tensor.rs:1945-1969).
template <class P>
class MappedLaunchPartition {
 public:
  using Inner = P;
  MappedLaunchPartition(P partition, std::vector<int32_t> map_shape, uint32_t num_tile_blocks)
      : partition_(std::move(partition)), map_shape_(std::move(map_shape)), num_tile_blocks_(num_tile_blocks) {}
  MappedLaunchPartition(MappedLaunchPartition&&) = default;
  MappedLaunchPartition& operator=(MappedLaunchPartition&&) = default;

  const P& partition() const { return partition_; }
  const std::vector<int32_t>& map_shape() const { return map_shape_; }
  uint32_t num_tile_blocks() const { return num_tile_blocks_; }

  cutile_mapped_partition_arg_t arg() const {
    cutile_mapped_partition_arg_t m{};
    m.partition = partition_.arg();
    m.map_rank = (int32_t)map_shape_.size();
    for (size_t i = 0; i < map_shape_.size() && i < 3; ++i) m.map_shape[i] = map_shape_[i];
    m.num_tile_blocks = num_tile_blocks_;
    return m;
  }
  // validate (tensor.rs:352-400): the launch grid, or the reason the map cannot traverse the partition
  Result<std::array<uint32_t, 3>> grid() const {
    std::array<uint32_t, 3> g{};
    cutile_mapped_partition_arg_t m = arg();
    CUTILE_TRY_STATUS(cutile_mapped_partition_grid(&m, g.data()));
    return g;
  }
  // the block id per partition axis that stream item `item` maps to (tile block b visits b, b + n, ...)
  Result<std::array<uint32_t, 3>> index(uint32_t item) const {
    std::array<uint32_t, 3> idx{};
    cutile_mapped_partition_arg_t m = arg();
    CUTILE_TRY_STATUS(cutile_mapped_partition_index(&m, item, idx.data(), nullptr));
    return idx;
  }
  // the block ids of `for index in z.iter_indices_within(ranges)` in stream order (cutile/src/_core.rs:912-930):
  // one (start_tile, num_tiles) pair per map axis, num_tiles -1 = the rest of the axis
  Result<std::vector<std::array<uint32_t, 3>>> indices_within(const std::vector<std::pair<int32_t, int32_t>>& ranges) const {
    if (ranges.size() != map_shape_.size())
      return DeviceError::tensor("sub-range iteration expects " + std::to_string(map_shape_.size()) +
                                 " (start_tile, num_tiles) pairs, got " + std::to_string(ranges.size()));
    std::vector<int32_t> flat;
    for (auto& r : ranges) {
      flat.push_back(r.first);
      flat.push_back(r.second);
    }
    cutile_mapped_partition_arg_t m = arg();
    uint32_t n = 0;
    CUTILE_TRY_STATUS(cutile_mapped_partition_index_within(&m, flat.data(), 0, nullptr, &n));
    std::vector<std::array<uint32_t, 3>> out(n);
    for (uint32_t t = 0; t < n; ++t) CUTILE_TRY_STATUS(cutile_mapped_partition_index_within(&m, flat.data(), t, out[t].data(), nullptr));
    return out;
  }
  P into_partition() && { return std::move(partition_); }

 private:
  P partition_;
  std::vector<int32_t> map_shape_;
  uint32_t num_tile_blocks_;
};

template <class X>
MappedLaunchPartition<Partition<X>> Partition<X>::map(std::vector<int32_t> map_shape, uint32_t num_tile_blocks) && {
  if (prefix_)
    throw std::logic_error("a partial-coverage (prefix) partition cannot be mapped: a mapped schedule covers its full "
                           "index space by construction");
  return MappedLaunchPartition<Partition<X>>(std::move(*this), std::move(map_shape), num_tile_blocks);
}

template <class T>
Partition<Tensor<T>> Tensor<T>::partition(std::vector<int32_t> tile) && {
  if (storage_.use_count() != 1)
    throw std::logic_error("partition: the tensor's storage must be uniquely owned (it is shared by views or clones)");
  return Partition<Tensor<T>>(std::move(*this), std::move(tile), false);
}
template <class T>
Partition<Tensor<T>> Tensor<T>::partition_prefix(std::vector<int32_t> tile) && {
  return std::move(*this).partition(std::move(tile)).prefix();
}
template <class T>
Partition<Tensor<T>*> Tensor<T>::partition_mut(std::vector<int32_t> tile) & {
  if (storage_.use_count() != 1)
    throw std::logic_error("partition: the tensor's storage must be uniquely owned (it is shared by views or clones)");
  return Partition<Tensor<T>*>(this, std::move(tile), false);
}
// try_partition: consume an Arc only if it has a single owner (tensor.rs:1476-1517).
template <class T>
Result<Partition<Tensor<T>>> try_partition(std::shared_ptr<Tensor<T>> t, std::vector<int32_t> tile) {
  if (t.use_count() != 1) return DeviceError::tensor("try_partition: the Arc has multiple owners");
  if (t->storage_use_count() != 1) return DeviceError::tensor("try_partition: the storage is shared");
  Tensor<T> owned = std::move(*t);
  return std::move(owned).partition(std::move(tile));
}

// ---- kernel argument traits ------------------------------------------------------------------
// How each accepted host form is pushed as a read-only tensor argument.
template <class T> const cutile_tensor_arg_t input_arg(const Tensor<T>& t) { return t.arg(); }
template <class T> const cutile_tensor_arg_t input_arg(const std::shared_ptr<Tensor<T>>& t) { return t->arg(); }
template <class T> const cutile_tensor_arg_t input_arg(const Tensor<T>* t) { return t->arg(); }
template <class T> const cutile_tensor_arg_t input_arg(const TensorView<T>& v) { return v.arg(); }

}  // namespace cutile
