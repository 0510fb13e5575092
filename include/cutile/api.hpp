// api::* — lazy tensor constructors and transfers, and the kernel launchers of
// the hot path.
//
// Constructors mirror cutile/src/api.rs:215-735 (zeros/ones/full :483-528,
// arange :552-559, copy_host_vec_to_device / to_host_vec / dup / memcpy
// :215-460, convert :654-666, randn :683-719, meta :450-462).  Everything is a
// DeviceOp: nothing is allocated or launched until the op executes.
//
// Launchers mirror the macro-generated unified launcher of each entry kernel
// (cutile-macro/src/kernel_launcher_generator.rs:1056-1202): arguments may be
// plain values or DeviceOps, the builder methods .generics() / .grid() are kept,
// and the output is the tuple of the arguments, in signature order, in the
// ownership form they were given.
#pragma once
#include <array>
#include <cmath>
#include <optional>
#include <stdexcept>
#include <string>

#include "runtime.hpp"
#include "specialization.hpp"
#include "tensor.hpp"

namespace cutile {
namespace api {

// ---- allocation ----------------------------------------------------------------------------
template <class T>
class Uninitialized : public DeviceOp<Uninitialized<T>, Tensor<T>> {
 public:
  explicit Uninitialized(std::vector<int32_t> shape) : shape_(std::move(shape)) {}
  Result<Tensor<T>> execute(const ExecutionContext& ctx) && {
    auto n = checked_num_elements(shape_);
    if (!n) return DeviceError::tensor("Tensor shape contains invalid dimensions or overflows.");
    auto p = ctx.alloc_async(*n * sizeof(T));  // tensor.rs:1016-1030
    if (p.is_err()) return p.error();
    auto strides = contiguous_strides(shape_);
    return Tensor<T>::from_raw_parts(p.value(), *n * sizeof(T), ctx.device_id(), std::move(shape_), std::move(strides));
  }

 private:
  std::vector<int32_t> shape_;
};

inline cutile_partition_arg_t flat_partition(const cutile_tensor_arg_t& t, size_t n, int32_t tile) {
  cutile_partition_arg_t p{};
  p.tensor = t;
  p.tensor.rank = 1;
  p.tensor.shape[0] = (int32_t)n;
  p.tensor.strides[0] = 1;
  p.partition_shape[0] = tile;
  p.partition_strides[0] = 1;
  return p;
}

// full: allocate, then launch the library kernel creation::full over tiles of 128
// (api.rs:518-528; kernel cutile/src/kernels/_creation.rs:44-47).
template <class T>
class Full : public DeviceOp<Full<T>, Tensor<T>> {
 public:
  Full(double v, int64_t iv, std::vector<int32_t> shape) : v_(v), iv_(iv), shape_(std::move(shape)) {}
  Result<Tensor<T>> execute(const ExecutionContext& ctx) && {
    auto t = Uninitialized<T>(std::move(shape_)).execute(ctx);
    if (t.is_err()) return t.error();
    if (t.value().size() == 0) return t;
    cutile_partition_arg_t p = flat_partition(t.value().arg(), t.value().size(), 128);
    CUTILE_TRY_STATUS(cutile_launch_full(ctx.stream()->raw(), v_, iv_, &p, nullptr));
    return t;
  }

 private:
  double v_;
  int64_t iv_;
  std::vector<int32_t> shape_;
};
template <class T> Full<T> full(double value, std::vector<int32_t> shape) { return Full<T>(value, (int64_t)value, std::move(shape)); }
template <class T> Full<T> zeros(std::vector<int32_t> shape) { return Full<T>(0.0, 0, std::move(shape)); }
template <class T> Full<T> ones(std::vector<int32_t> shape) { return Full<T>(1.0, 1, std::move(shape)); }

template <class T>
class Arange : public DeviceOp<Arange<T>, Tensor<T>> {
 public:
  explicit Arange(size_t n) : n_(n) {}
  Result<Tensor<T>> execute(const ExecutionContext& ctx) && {
    auto t = Uninitialized<T>({(int32_t)n_}).execute(ctx);
    if (t.is_err()) return t.error();
    cutile_partition_arg_t p = flat_partition(t.value().arg(), n_, 128);
    CUTILE_TRY_STATUS(cutile_launch_arange(ctx.stream()->raw(), &p, nullptr));
    return t;
  }

 private:
  size_t n_;
};
template <class T> Arange<T> arange(size_t n) { return Arange<T>(n); }

// eye / eye_rect: allocate [rows, cols] f32, then creation::eye over tiles of 16 x 16
// (api.rs:613-639; kernel cutile/src/kernels/_creation.rs:110-138).
class Eye : public DeviceOp<Eye, Tensor<float>> {
 public:
  Eye(size_t rows, size_t cols) : rows_(rows), cols_(cols) {}
  Result<Tensor<float>> execute(const ExecutionContext& ctx) && {
    auto t = Uninitialized<float>({(int32_t)rows_, (int32_t)cols_}).execute(ctx);
    if (t.is_err()) return t.error();
    if (t.value().size() == 0) return t;
    cutile_partition_arg_t p{};
    p.tensor = t.value().arg();
    for (int i = 0; i < 2; ++i) {
      p.partition_shape[i] = 16;
      p.partition_strides[i] = p.tensor.strides[i];
    }
    CUTILE_TRY_STATUS(cutile_launch_eye(ctx.stream()->raw(), &p, nullptr));
    return t;
  }

 private:
  size_t rows_, cols_;
};
inline Eye eye_rect(size_t rows, size_t cols) { return Eye(rows, cols); }
inline Eye eye(size_t n) { return Eye(n, n); }

class Linspace : public DeviceOp<Linspace, Tensor<float>> {
 public:
  Linspace(float start, float stop, size_t n) : start_(start), stop_(stop), n_(n) {}
  Result<Tensor<float>> execute(const ExecutionContext& ctx) && {
    auto t = Uninitialized<float>({(int32_t)n_}).execute(ctx);
    if (t.is_err()) return t.error();
    float step = n_ > 1 ? (stop_ - start_) / (float)(n_ - 1) : 0.0f;
    cutile_partition_arg_t p = flat_partition(t.value().arg(), n_, 128);
    CUTILE_TRY_STATUS(cutile_launch_linspace(ctx.stream()->raw(), &p, start_, step, nullptr));
    return t;
  }

 private:
  float start_, stop_;
  size_t n_;
};
inline Linspace linspace(float start, float stop, size_t n) { return Linspace(start, stop, n); }

// meta: shape/stride metadata without memory (api.rs:450-462).
template <class T> Value<Tensor<T>> meta(std::vector<int32_t> shape) { return value(Tensor<T>::from_meta(std::move(shape))); }

// ---- transfers -----------------------------------------------------------------------------
template <class T>
class CopyHostVecToDevice : public DeviceOp<CopyHostVecToDevice<T>, Tensor<T>> {
 public:
  explicit CopyHostVecToDevice(std::shared_ptr<std::vector<T>> host) : host_(std::move(host)) {}
  Result<Tensor<T>> execute(const ExecutionContext& ctx) && {
    auto t = Uninitialized<T>({(int32_t)host_->size()}).execute(ctx);
    if (t.is_err()) return t.error();
    CUTILE_TRY_STATUS(cutile_memcpy_htod_async(t.value().device_pointer(), host_->data(), host_->size() * sizeof(T), ctx.stream()->raw()));
    return t;
  }

 private:
  std::shared_ptr<std::vector<T>> host_;  // must stay alive until the stream is synchronised
};
template <class T>
CopyHostVecToDevice<T> copy_host_vec_to_device(std::shared_ptr<std::vector<T>> host) { return CopyHostVecToDevice<T>(std::move(host)); }

// to_host_vec: the vector is valid once the stream has been synchronised.
template <class Src>
class ToHostVec : public DeviceOp<ToHostVec<Src>, std::vector<typename std::decay_t<decltype(*std::declval<Src>())>::Elem>> {
 public:
  using T = typename std::decay_t<decltype(*std::declval<Src>())>::Elem;
  explicit ToHostVec(Src src) : src_(std::move(src)) {}
  Result<std::vector<T>> execute(const ExecutionContext& ctx) && {
    const Tensor<T>& t = *src_;
    if (!t.is_contiguous()) return DeviceError::tensor("to_host_vec: tensor must be contiguous");
    std::vector<T> out(t.size());
    CUTILE_TRY_STATUS(cutile_memcpy_dtoh_async(out.data(), t.device_pointer(), t.num_bytes(), ctx.stream()->raw()));
    return out;
  }

 private:
  Src src_;  // shared_ptr<Tensor<T>> or const Tensor<T>*
};
template <class T> ToHostVec<std::shared_ptr<Tensor<T>>> to_host_vec(std::shared_ptr<Tensor<T>> t) { return ToHostVec<std::shared_ptr<Tensor<T>>>(std::move(t)); }
template <class T> ToHostVec<const Tensor<T>*> to_host_vec(const Tensor<T>& t) { return ToHostVec<const Tensor<T>*>(&t); }
// device_op.to_host_vec(): copy the tensor an op produces.
template <class Op>
auto to_host_vec_op(Op op) {
  using T = typename Op::Output::Elem;
  return std::move(op).then([](Tensor<T> t) { return to_host_vec(std::make_shared<Tensor<T>>(std::move(t))); });
}

template <class T>
class Dup : public DeviceOp<Dup<T>, Tensor<T>> {
 public:
  explicit Dup(const Tensor<T>* src) : src_(src) {}
  Result<Tensor<T>> execute(const ExecutionContext& ctx) && {
    if (!src_->is_contiguous()) return DeviceError::tensor("dup: tensor must be contiguous");
    auto t = Uninitialized<T>(src_->shape()).execute(ctx);
    if (t.is_err()) return t.error();
    CUTILE_TRY_STATUS(cutile_memcpy_dtod_async(t.value().device_pointer(), src_->device_pointer(), src_->num_bytes(), ctx.stream()->raw()));
    return t;
  }

 private:
  const Tensor<T>* src_;
};
template <class T> Dup<T> dup(const Tensor<T>& t) { return Dup<T>(&t); }

// memcpy: device-to-device into an existing tensor; sizes must agree; a graph node (api.rs:298).
template <class T>
class Memcpy : public DeviceOp<Memcpy<T>, Unit> {
 public:
  Memcpy(Tensor<T>* dst, const Tensor<T>* src) : dst_(dst), src_(src) {
    if (dst->size() != src->size()) throw std::logic_error("memcpy: source and destination must have the same number of elements");
  }
  Result<Unit> execute(const ExecutionContext& ctx) && {
    return check(cutile_memcpy_dtod_async(dst_->device_pointer(), src_->device_pointer(), src_->num_bytes(), ctx.stream()->raw()));
  }

 private:
  Tensor<T>* dst_;
  const Tensor<T>* src_;
};
template <class T> Memcpy<T> memcpy(Tensor<T>& dst, const Tensor<T>& src) { return Memcpy<T>(&dst, &src); }

// convert<From, To>: new tensor of another element type (api.rs:654-666).
template <class To, class From>
class Convert : public DeviceOp<Convert<To, From>, Tensor<To>> {
 public:
  explicit Convert(std::shared_ptr<Tensor<From>> src) : src_(std::move(src)) {}
  Result<Tensor<To>> execute(const ExecutionContext& ctx) && {
    auto t = Uninitialized<To>({(int32_t)src_->size()}).execute(ctx);
    if (t.is_err()) return t.error();
    cutile_tensor_arg_t s = src_->arg();
    s.rank = 1; s.shape[0] = (int32_t)src_->size(); s.strides[0] = 1;
    cutile_partition_arg_t d = flat_partition(t.value().arg(), src_->size(), 128);
    CUTILE_TRY_STATUS(cutile_launch_convert(ctx.stream()->raw(), &s, &d, nullptr));
    return std::move(t).unwrap().reshape(src_->shape());
  }

 private:
  std::shared_ptr<Tensor<From>> src_;
};
template <class To, class From> Convert<To, From> convert(std::shared_ptr<Tensor<From>> src) { return Convert<To, From>(std::move(src)); }

// randn / rand / randn_f16 (api.rs:683-735): the values are drawn on the device by the library's generator
// (cutile_rng_*: Philox4x32-10, one generator per op, seeded when a seed is given, as the reference creates one RNG
// per call).  The op is a stream-ordered fill of a freshly allocated tensor: nothing blocks and nothing crosses the
// host.  The value stream is this library's own; cuRAND's does not exist on this platform.
template <class T> struct RngFill;
template <> struct RngFill<float> {
  static cutile_status_t normal(cutile_rng_t g, void* p, size_t n, float mean, float std, cutile_stream_t s) { return cutile_rng_normal_f32(g, p, n, mean, std, s); }
  static cutile_status_t uniform(cutile_rng_t g, void* p, size_t n, cutile_stream_t s) { return cutile_rng_uniform_f32(g, p, n, s); }
};
template <> struct RngFill<double> {
  static cutile_status_t normal(cutile_rng_t g, void* p, size_t n, double mean, double std, cutile_stream_t s) { return cutile_rng_normal_f64(g, p, n, mean, std, s); }
  static cutile_status_t uniform(cutile_rng_t g, void* p, size_t n, cutile_stream_t s) { return cutile_rng_uniform_f64(g, p, n, s); }
};
// RAII generator (cuda-core/src/api.rs:214-293 `RNG`)
class Rng {
 public:
  explicit Rng(std::optional<uint64_t> seed = std::nullopt) {
    if (cutile_rng_create(&g_) != CUTILE_SUCCESS) throw std::runtime_error("cutile_rng_create failed");
    if (seed) cutile_rng_set_seed(g_, *seed);
  }
  ~Rng() { cutile_rng_destroy(g_); }
  Rng(const Rng&) = delete;
  Rng& operator=(const Rng&) = delete;
  cutile_rng_t raw() const { return g_; }

 private:
  cutile_rng_t g_ = nullptr;
};

template <class T>
class RandomFill : public DeviceOp<RandomFill<T>, Tensor<T>> {
 public:
  RandomFill(bool normal, T mean, T std, std::vector<int32_t> shape, std::optional<uint64_t> seed)
      : normal_(normal), mean_(mean), std_(std), shape_(std::move(shape)), seed_(seed) {}
  Result<Tensor<T>> execute(const ExecutionContext& ctx) && {
    auto t = Uninitialized<T>(shape_).execute(ctx);
    if (t.is_err()) return t.error();
    Rng rng(seed_);
    const size_t n = t.value().size();
    if (normal_) CUTILE_TRY_STATUS(RngFill<T>::normal(rng.raw(), t.value().device_pointer(), n, mean_, std_, ctx.stream()->raw()));
    else CUTILE_TRY_STATUS(RngFill<T>::uniform(rng.raw(), t.value().device_pointer(), n, ctx.stream()->raw()));
    return t;
  }

 private:
  bool normal_;
  T mean_, std_;
  std::vector<int32_t> shape_;
  std::optional<uint64_t> seed_;
};
// randn<T>(mean, std, shape, seed): T = float | double (api.rs:683-696)
template <class T = float>
RandomFill<T> randn(T mean, T std, std::vector<int32_t> shape, std::optional<uint64_t> seed = std::nullopt) {
  return RandomFill<T>(true, mean, std, std::move(shape), seed);
}
// rand<T>(shape, seed): uniform in [0, 1) (api.rs:722-735)
template <class T = float>
RandomFill<T> rand(std::vector<int32_t> shape, std::optional<uint64_t> seed = std::nullopt) {
  return RandomFill<T>(false, T(0), T(1), std::move(shape), seed);
}
// randn_f16: f32 values drawn, then converted (api.rs:698-719: the generator has no f16 form)
inline auto randn_f16(float mean, float std, std::vector<int32_t> shape, std::optional<uint64_t> seed = std::nullopt) {
  const size_t n = checked_num_elements(shape).value_or(0);
  return randn<float>(mean, std, {(int32_t)n}, seed).then([shape = std::move(shape)](Tensor<float> src) mutable {
    return convert<f16>(std::make_shared<Tensor<float>>(std::move(src))).then([shape = std::move(shape)](Tensor<f16> t) mutable {
      return value(std::move(t).reshape(std::move(shape)).unwrap());
    });
  });
}

}  // namespace api

// reshape on an op's output (api::DeviceOpReshape).
template <class Op>
auto reshape_op(Op op, std::vector<int32_t> shape) {
  using TT = typename Op::Output;
  return std::move(op).then([shape = std::move(shape)](TT t) mutable { return value(std::move(t).reshape(std::move(shape)).unwrap()); });
}
// partition on an op's output (tile_kernel.rs:1236-1316 PartitionOp).
template <class Op>
auto partition_op(Op op, std::vector<int32_t> tile) {
  using TT = typename Op::Output;
  return std::move(op).then([tile = std::move(tile)](TT t) mutable { return value(std::move(t).partition(std::move(tile))); });
}
// unpartition on an op that yields a partition.
template <class Op>
auto unpartition_op(Op op) {
  using P = typename Op::Output;
  return std::move(op).map([](P p) { return std::move(p).unpartition(); });
}

// ---- kernel launchers ------------------------------------------------------------------------
// What a launcher hands back for a stored argument (KernelOutput::recover, tensor.rs:1945-1969): the argument itself,
// except that a mapped partition gives back its inner partition.
template <class T>
struct Recovered {
  using type = T;
  static T get(T&& v) { return std::move(v); }
};
template <class P>
struct Recovered<MappedLaunchPartition<P>> {
  using type = P;
  static P get(MappedLaunchPartition<P>&& v) { return std::move(v).into_partition(); }
};

// How one stored argument enters the specialization identity (kernel_launcher_generator.rs:600-700): a tensor-like
// argument contributes its stride-one pattern and SpecializationBits, an integer scalar a divisibility hint, a
// floating-point scalar nothing.
namespace detail {
template <class A, class = void> struct has_input_arg : std::false_type {};
template <class A> struct has_input_arg<A, std::void_t<decltype(input_arg(std::declval<const A&>()))>> : std::true_type {};
template <class A, class = void> struct has_arg_method : std::false_type {};
template <class A> struct has_arg_method<A, std::void_t<decltype(std::declval<const A&>().arg())>> : std::true_type {};
inline const cutile_tensor_arg_t& tensor_of(const cutile_tensor_arg_t& t) { return t; }
inline const cutile_tensor_arg_t& tensor_of(const cutile_partition_arg_t& p) { return p.tensor; }
inline const cutile_tensor_arg_t& tensor_of(const cutile_mapped_partition_arg_t& m) { return m.partition.tensor; }
template <class A>
void describe_arg(const A& a, size_t index, int32_t max_div, std::vector<std::pair<std::string, std::vector<int32_t>>>* strides,
                  std::vector<std::pair<std::string, SpecializationBits>>* specs, std::vector<std::pair<std::string, DivHint>>* scalars) {
  const std::string name = "arg" + std::to_string(index);
  if constexpr (std::is_integral_v<A>) {
    scalars->emplace_back(name, DivHint::from_value((int64_t)a).with_max(max_div));
  } else if constexpr (std::is_floating_point_v<A>) {
  } else {
    cutile_tensor_arg_t t{};
    if constexpr (has_input_arg<A>::value) t = input_arg(a);
    else if constexpr (has_arg_method<A>::value) { auto rec = a.arg(); t = tensor_of(rec); }
    else return;
    std::vector<int32_t> one;
    for (int i = 0; i < t.rank; ++i) one.push_back(t.strides[i] == 1 ? 1 : 0);
    strides->emplace_back(name, std::move(one));
    specs->emplace_back(name, SpecializationBits::from_tensor_arg(t, max_div));
  }
}
template <class Fn, class = void> struct kernel_name { static constexpr const char* value = "kernel"; };
template <class Fn> struct kernel_name<Fn, std::void_t<decltype(Fn::name)>> { static constexpr const char* value = Fn::name; };
}  // namespace detail

template <class Fn, class... ArgOps>
class KernelLauncher : public DeviceOp<KernelLauncher<Fn, ArgOps...>, std::tuple<typename Recovered<typename ArgOps::Output>::type...>> {
 public:
  using Stored = std::tuple<typename ArgOps::Output...>;
  using Out = std::tuple<typename Recovered<typename ArgOps::Output>::type...>;
  explicit KernelLauncher(ArgOps&&... ops) : ops_(std::move(ops)...) {}
  KernelLauncher(KernelLauncher&&) = default;
  // Builder methods of the generated launcher (cutile-macro/src/_module.rs:901-923).
  KernelLauncher generics(std::vector<std::string> g) && { generics_ = std::move(g); return std::move(*this); }
  KernelLauncher grid(uint32_t x, uint32_t y, uint32_t z) && { grid_ = {x, y, z}; const_grid_ = false; return std::move(*this); }
  // const_grid: the same launch grid, and the grid becomes part of the specialization identity.
  KernelLauncher const_grid(uint32_t x, uint32_t y, uint32_t z) && { grid_ = {x, y, z}; const_grid_ = true; return std::move(*this); }
  std::array<uint32_t, 3> get_launch_grid() const { return grid_; }
  KernelLauncher compile_options(CompileOptions o) && { compile_options_ = std::move(o); return std::move(*this); }
  KernelLauncher variant(std::string v) && { variant_ = std::move(v); return std::move(*this); }

  // compile / compile_on (_module.rs:852-866): everything a launch does except the launch block; afterwards the
  // kernel's code object is loaded on the device, so the first real launch loads nothing.
  Result<Unit> compile_on(const std::shared_ptr<Stream>& stream) && {
    ExecutionContext ctx(stream);
    auto r = std::move(*this).run(ctx, CUTILE_LAUNCH_MODE_COMPILE_ONLY, nullptr);
    if (r.is_err()) return r.error();
    return ok();
  }
  Result<Unit> compile() && {
    auto stream = next_stream();
    if (stream.is_err()) return stream.error();
    return std::move(*this).compile_on(stream.value());
  }
  // specialize / specialize_on (_module.rs:868-878): the identity of this launch, nothing compiled or launched.
  Result<Specialization> specialize_on(const std::shared_ptr<Stream>& stream) && {
    ExecutionContext ctx(stream);
    std::optional<Specialization> spec;
    auto r = std::move(*this).run(ctx, CUTILE_LAUNCH_MODE_SPECIALIZE_ONLY, &spec);
    if (r.is_err()) return r.error();
    return std::move(*spec);
  }
  Result<Specialization> specialize() && {
    auto stream = next_stream();
    if (stream.is_err()) return stream.error();
    return std::move(*this).specialize_on(stream.value());
  }
  Result<TileFunctionKey> l1_cache_key_on(const std::shared_ptr<Stream>& stream) && {
    auto s = std::move(*this).specialize_on(stream);
    if (s.is_err()) return s.error();
    return std::move(s).unwrap().into_l1_cache_key();
  }
  Result<TileFunctionKey> l1_cache_key() && {
    auto s = std::move(*this).specialize();
    if (s.is_err()) return s.error();
    return std::move(s).unwrap().into_l1_cache_key();
  }
  Result<std::string> l2_cache_key_on(const std::shared_ptr<Stream>& stream) && {
    auto s = std::move(*this).specialize_on(stream);
    if (s.is_err()) return s.error();
    return s.value().l2_cache_key();
  }
  Result<std::string> l2_cache_key() && {
    auto s = std::move(*this).specialize();
    if (s.is_err()) return s.error();
    return s.value().l2_cache_key();
  }

  Result<Out> execute(const ExecutionContext& ctx) && { return std::move(*this).run(ctx, CUTILE_LAUNCH_MODE_LAUNCH, nullptr); }

 private:
  enum : int32_t { CUTILE_LAUNCH_MODE_LAUNCH = 0, CUTILE_LAUNCH_MODE_COMPILE_ONLY = 1, CUTILE_LAUNCH_MODE_SPECIALIZE_ONLY = 2 };
  struct ModeGuard {   // the mode is a property of the thread for the duration of one launcher call
    explicit ModeGuard(int32_t m) { cutile_set_launch_mode(m); }
    ~ModeGuard() { cutile_set_launch_mode(0); }
  };
  Result<Out> run(const ExecutionContext& ctx, int32_t mode, std::optional<Specialization>* spec) && {
    // 1. run the argument ops in signature order; 2. validate + launch; 3. hand the arguments back.
    auto args = std::move(ops_).execute(ctx);
    if (args.is_err()) return args.error();
    Stored vals = std::move(args).unwrap();
    std::vector<const char*> gptrs;
    for (auto& s : generics_) gptrs.push_back(s.c_str());
    cutile_launch_opts_t opts{};
    opts.grid[0] = grid_[0]; opts.grid[1] = grid_[1]; opts.grid[2] = grid_[2];
    opts.generics = gptrs.empty() ? nullptr : gptrs.data();
    opts.n_generics = (int32_t)gptrs.size();
    opts.variant = variant_.empty() ? nullptr : variant_.c_str();
    cutile_status_t s;
    {
      ModeGuard guard(mode);
      s = std::apply([&](auto&... a) { return Fn::launch(ctx.stream()->raw(), &opts, a...); }, vals);
    }
    if (s != CUTILE_SUCCESS) return DeviceError::from_status(s);
    if (spec) {
      const char* fn_name = nullptr;
      cutile_kernel_info_t info{};
      CUTILE_TRY_STATUS(cutile_last_resolved_kernel(&fn_name, &info));
      const int32_t max_div = compile_options_.max_divisibility_.value_or(16);
      std::vector<std::pair<std::string, std::vector<int32_t>>> strides;
      std::vector<std::pair<std::string, SpecializationBits>> specs;
      std::vector<std::pair<std::string, DivHint>> scalars;
      size_t index = 0;
      std::apply([&](auto&... a) { (detail::describe_arg(a, index++, max_div, &strides, &specs, &scalars), ...); }, vals);
      char fp[17] = {0};
      CUTILE_TRY_STATUS(cutile_kernel_fingerprint(fn_name, info.variant, fp));
      char arch[256] = {0};
      cutile_device_t dev = nullptr;
      CUTILE_TRY_STATUS(cutile_device_get(ctx.device_id(), &dev));
      CUTILE_TRY_STATUS(cutile_device_arch(dev, arch, sizeof(arch)));
      auto b = TileFunctionKey::builder("cutile_kernels", detail::kernel_name<Fn>::value)
                   .generics(generics_)
                   .stride_args(std::move(strides))
                   .spec_args(std::move(specs))
                   .scalar_hints(std::move(scalars))
                   .compile_options(compile_options_)
                   .source_hash(fp)
                   .device_id((size_t)ctx.device_id())
                   .gpu_name(arch)
                   .compiler_version(cutile_version())
                   .toolchain_fingerprint(cutile_toolchain_fingerprint());
      if (const_grid_) b = std::move(b).grid(grid_[0], grid_[1], grid_[2]);
      spec->emplace(std::move(b).build(), info.variant ? info.variant : "", info.symbol ? info.symbol : "");
    }
    return std::apply([](auto&... a) { return Out(Recovered<std::decay_t<decltype(a)>>::get(std::move(a))...); }, vals);
  }

  Zip<ArgOps...> ops_;
  std::vector<std::string> generics_;
  std::array<uint32_t, 3> grid_{0, 0, 0};
  bool const_grid_ = false;
  CompileOptions compile_options_;
  std::string variant_;
};
template <class Fn, class... ArgOps>
struct is_graph_node<KernelLauncher<Fn, ArgOps...>> : std::bool_constant<(is_graph_node_v<ArgOps> && ...)> {};

template <class Fn, class... Xs>
auto make_launcher(Xs&&... xs) {
  return KernelLauncher<Fn, into_op_t<Xs>...>(into_op(std::forward<Xs>(xs))...);
}

// <kernel>_apply(tuple): the launcher over a tuple of materialised arguments (kernel_launcher_generator.rs:1036-1044).
template <class Fn, class... Xs>
auto apply_launcher(std::tuple<Xs...> args) {
  return std::apply([](auto&&... xs) { return make_launcher<Fn>(std::move(xs)...); }, std::move(args));
}

namespace kernels {
struct SaxpyFn {
  static constexpr const char* name = "saxpy";
  template <class Y, class X>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, Y& y, double a, X& x) {
    auto yp = y.arg();
    auto xa = input_arg(x);
    return cutile_launch_saxpy(s, &yp, a, &xa, o);
  }
};
struct AxpyFn {
  static constexpr const char* name = "axpy";
  template <class Z, class X, class Yv>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, Z& z, double a, X& x, Yv& y) {
    auto zp = z.arg();
    auto xa = input_arg(x), ya = input_arg(y);
    return cutile_launch_axpy(s, &zp, a, &xa, &ya, o);
  }
};
struct AddFn {
  static constexpr const char* name = "add";
  template <class Z, class X, class Yv>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, Z& z, X& x, Yv& y) {
    auto zp = z.arg();
    auto xa = input_arg(x), ya = input_arg(y);
    return cutile_launch_add(s, &zp, &xa, &ya, o);
  }
};
struct RmsNormF16Fn {
  static constexpr const char* name = "rms_norm_f16";
  template <class X, class W, class O>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, X& x, W& w, O& out, float eps) {
    auto xa = input_arg(x), wa = input_arg(w);
    auto op = out.arg();
    return cutile_launch_rms_norm_f16(s, &xa, &wa, &op, eps, o);
  }
};
struct RmsNormF32Fn {
  static constexpr const char* name = "rms_norm";
  template <class X, class W, class O>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, X& x, W& w, O& out, float eps) {
    auto xa = input_arg(x), wa = input_arg(w);
    auto op = out.arg();
    return cutile_launch_rms_norm_f32(s, &xa, &wa, &op, eps, o);
  }
};
// The benchmark programs with their own all-f16 arithmetic (cutile-benchmarks/benches/rmsnorm.rs:20-66,
// benches/softmax.rs:19-35); .generics({N, BLOCK_SIZE}) is required for the RMSNorm form.
struct RmsNormAllF16Fn {
  static constexpr const char* name = "rms_norm";
  template <class X, class W, class O>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, X& x, W& w, O& out, float eps) {
    auto xa = input_arg(x), wa = input_arg(w);
    auto op = out.arg();
    return cutile_launch_rms_norm_all_f16(s, &xa, &wa, &op, eps, o);
  }
};
struct SoftmaxAllF16Fn {
  static constexpr const char* name = "softmax";
  template <class X, class Yv>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, X& x, Yv& y) {
    auto xa = input_arg(x);
    auto yp = y.arg();
    return cutile_launch_softmax_all_f16(s, &xa, &yp, o);
  }
};
struct SoftmaxFn {
  static constexpr const char* name = "softmax";
  template <class X, class Yv>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, X& x, Yv& y) {
    auto xa = input_arg(x);
    auto yp = y.arg();
    return cutile_launch_softmax(s, &xa, &yp, o);
  }
};
// the example programs' small kernels
struct ReluFn {
  static constexpr const char* name = "relu";
  template <class IO>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, IO& io) {
    auto p = io.arg();
    return cutile_launch_relu(s, &p, o);
  }
};
struct DropoutFn {
  static constexpr const char* name = "dropout";
  template <class X, class XK, class O>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, float p, X& x, XK& x_keep, O& out) {
    auto op = out.arg();
    auto xa = input_arg(x), ka = input_arg(x_keep);
    return cutile_launch_dropout(s, p, &xa, &ka, &op, o);
  }
};
struct ScalePtrFn {
  static constexpr const char* name = "scale_ptr";
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, void* out_ptr, void* in_ptr, float scale, int32_t len) {
    return cutile_launch_scale_ptr(s, out_ptr, in_ptr, scale, len, o);
  }
};
struct MatvecFn {
  static constexpr const char* name = "matvec";
  template <class Z, class X, class Yv>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, Z& z, X& x, Yv& y, int32_t k) {
    auto zp = z.arg();
    auto xa = input_arg(x), ya = input_arg(y);
    return cutile_launch_matvec(s, &zp, &xa, &ya, k, o);
  }
};
struct BatchMatmulFn {
  static constexpr const char* name = "batch_matmul";
  template <class Cp, class A, class B>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, Cp& c, A& a, B& b, int32_t k) {
    auto cp = c.arg();
    auto aa = input_arg(a), ba = input_arg(b);
    return cutile_launch_batch_matmul(s, &cp, &aa, &ba, k, o);
  }
};
template <bool Accumulate>
struct GemmFn {
  static constexpr const char* name = "gemm";
  template <class Z, class X, class Yv>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, Z& z, X& x, Yv& y, int32_t k) {
    auto zp = z.arg();
    auto xa = input_arg(x), ya = input_arg(y);
    return cutile_launch_gemm(s, &zp, &xa, &ya, k, Accumulate ? 1 : 0, o);
  }
};
template <bool Causal>
struct FmhaFn {
  static constexpr const char* name = "fmha";
  // fmha(out, q, k, v, qk_scale, input_pos, query_group_size) — flash_attention_causal.rs:32-40
  template <class O, class Q, class K, class V>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, O& out, Q& q, K& k, V& v, float scale,
                                int32_t input_pos, int32_t group) {
    auto op = out.arg();
    auto qa = input_arg(q), ka = input_arg(k), va = input_arg(v);
    return cutile_launch_fmha(s, &op, &qa, &ka, &va, scale, input_pos, group, Causal ? 1 : 0, o);
  }
};
struct LinearTileMxfp8Fn {
  static constexpr const char* name = "linear_tile";
  template <class Z, class X, class Yv, class XS, class YS>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, Z& z, X& x, Yv& y, XS& xs, YS& ys, float alpha) {
    auto zp = z.arg();
    auto xa = input_arg(x), ya = input_arg(y), xsa = input_arg(xs), ysa = input_arg(ys);
    // the reference has one `linear_tile` per module (mxfp8.rs, nvfp4.rs); here the operand type picks the kernel
    if (xa.dtype == CUTILE_DTYPE_F4E2M1FNX2) return cutile_launch_linear_tile_nvfp4(s, &zp, &xa, &ya, &xsa, &ysa, alpha, o);
    return cutile_launch_linear_tile_mxfp8(s, &zp, &xa, &ya, &xsa, &ysa, alpha, o);
  }
};
// ---- transformer-block kernels (cutile-kernels/src/{norms,pointwise,positional}.rs) ----
struct AddRmsNormF16Fn {
  static constexpr const char* name = "add_rms_norm_f16";
  template <class R, class X, class W, class O, class RO>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, R& residual, X& x, W& w, O& out, RO& residual_out, float eps) {
    auto ra = input_arg(residual), xa = input_arg(x), wa = input_arg(w);
    auto op = out.arg(), rop = residual_out.arg();
    return cutile_launch_add_rms_norm_f16(s, &ra, &xa, &wa, &op, &rop, eps, o);
  }
};
struct QkNormF16Fn {
  static constexpr const char* name = "qk_norm_f16";
  template <class Q, class K, class QW, class KW, class O>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, Q& q, K& k, QW& qw, KW& kw, O& out, float eps, int32_t num_q_rows) {
    auto qa = input_arg(q), ka = input_arg(k), qwa = input_arg(qw), kwa = input_arg(kw);
    auto op = out.arg();
    return cutile_launch_qk_norm_f16(s, &qa, &ka, &qwa, &kwa, &op, eps, num_q_rows, o);
  }
};
template <bool Silu>
struct Pointwise2dF16Fn {
  static constexpr const char* name = Silu ? "silu_mul_2d_f16" : "add_2d_f16";
  template <class O, class A, class B>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, O& out, A& a, B& b) {
    auto op = out.arg();
    auto aa = input_arg(a), ba = input_arg(b);
    return Silu ? cutile_launch_silu_mul_2d_f16(s, &op, &aa, &ba, o) : cutile_launch_add_2d_f16(s, &op, &aa, &ba, o);
  }
};
struct RopeSeqF16Fn {
  static constexpr const char* name = "rope_seq_f16";
  template <class X, class F, class O>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, X& x, F& inv_freq, O& out, int32_t position_start) {
    auto xa = input_arg(x), fa = input_arg(inv_freq);
    auto op = out.arg();
    return cutile_launch_rope_f16(s, &xa, nullptr, &fa, nullptr, position_start, &op, 0, o);
  }
};
struct RopeSeqDynposF16Fn {
  static constexpr const char* name = "rope_seq_dynpos_f16";
  template <class X, class F, class P, class O>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, X& x, F& inv_freq, P& position_start, O& out) {
    auto xa = input_arg(x), fa = input_arg(inv_freq), pa = input_arg(position_start);
    auto op = out.arg();
    return cutile_launch_rope_f16(s, &xa, nullptr, &fa, &pa, 0, &op, 0, o);
  }
};
struct QkRopeDynposF16Fn {
  static constexpr const char* name = "qk_rope_dynpos_f16";
  template <class Q, class K, class F, class P, class O>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, Q& q, K& k, F& inv_freq, P& position_start, O& out, int32_t num_q_heads) {
    auto qa = input_arg(q), ka = input_arg(k), fa = input_arg(inv_freq), pa = input_arg(position_start);
    auto op = out.arg();
    return cutile_launch_rope_f16(s, &qa, &ka, &fa, &pa, 0, &op, num_q_heads, o);
  }
};
struct KvCacheUpdateSeqF16Fn {
  static constexpr const char* name = "kv_cache_update_seq_f16";
  template <class NK, class NV, class KC, class VC>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, NK& new_k, NV& new_v, KC& k_cache, VC& v_cache, int32_t position_start, int32_t seq_len) {
    auto ka = input_arg(new_k), va = input_arg(new_v);
    auto kp = k_cache.arg(), vp = v_cache.arg();
    return cutile_launch_kv_cache_update_f16(s, &ka, &va, &kp, &vp, nullptr, position_start, seq_len, o);
  }
};
struct KvCacheUpdateSeqDynposF16Fn {
  static constexpr const char* name = "kv_cache_update_seq_dynpos_f16";
  template <class NK, class NV, class KC, class VC, class P>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, NK& new_k, NV& new_v, KC& k_cache, VC& v_cache, P& position_start, int32_t seq_len) {
    auto ka = input_arg(new_k), va = input_arg(new_v), pa = input_arg(position_start);
    auto kp = k_cache.arg(), vp = v_cache.arg();
    return cutile_launch_kv_cache_update_f16(s, &ka, &va, &kp, &vp, &pa, 0, seq_len, o);
  }
};
struct FmhaDecodeGqaSplitFn {
  static constexpr const char* name = "fmha_decode_gqa_split";
  template <class Q, class K, class V, class A, class L, class P>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, Q& q, K& k, V& v, A& att_out, L& lse_out, float qk_scale, P& position_start) {
    auto qa = input_arg(q), ka = input_arg(k), va = input_arg(v), pa = input_arg(position_start);
    auto ap = att_out.arg(), lp = lse_out.arg();
    return cutile_launch_fmha_decode_gqa_split(s, &qa, &ka, &va, &ap, &lp, qk_scale, &pa, o);
  }
};
struct SplitkReduceMergeFn {
  static constexpr const char* name = "splitk_reduce_merge";
  template <class A, class L, class O>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, A& att_partial, L& lse_partial, O& out) {
    auto aa = input_arg(att_partial), la = input_arg(lse_partial);
    auto op = out.arg();
    return cutile_launch_splitk_reduce_merge(s, &aa, &la, &op, o);
  }
};
struct GroupGemmF16NtDescFn {
  static constexpr const char* name = "group_gemm_f16_nt_desc";
  template <class AP, class BP, class CP, class AM, class BM_, class CM>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, AP& a_ptrs, BP& b_ptrs, CP& c_ptrs, AM& a_metas,
                                BM_& b_metas, CM& c_metas, int32_t num_groups) {
    auto ap = input_arg(a_ptrs), bp = input_arg(b_ptrs), cp = input_arg(c_ptrs);
    auto am = input_arg(a_metas), bm = input_arg(b_metas), cm = input_arg(c_metas);
    return cutile_launch_group_gemm_f16_nt_desc(s, &ap, &bp, &cp, &am, &bm, &cm, num_groups, o);
  }
};
struct ArgmaxBlocksF16Fn {
  static constexpr const char* name = "argmax_blocks_f16";
  template <class L, class M, class I>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, L& logits, M& block_max, I& block_idx, int32_t len) {
    auto la = input_arg(logits);
    auto mp = block_max.arg(), ip = block_idx.arg();
    return cutile_launch_argmax_blocks_f16(s, &la, &mp, &ip, len, o);
  }
};
struct LmHeadArgmaxBlocksF16Fn {
  static constexpr const char* name = "lm_head_argmax_blocks_f16";
  template <class W, class H, class M, class I>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, W& weights, H& hidden, M& block_max, I& block_idx, int32_t vocab_size) {
    auto wa = input_arg(weights), ha = input_arg(hidden);
    auto mp = block_max.arg(), ip = block_idx.arg();
    return cutile_launch_lm_head_argmax_blocks_f16(s, &wa, &ha, &mp, &ip, vocab_size, o);
  }
};
struct ArgmaxReduceBlocksToU32Fn {
  static constexpr const char* name = "argmax_reduce_blocks_to_u32";
  template <class M, class I, class O>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, M& block_max, I& block_idx, O& out, int32_t num_blocks) {
    auto ma = input_arg(block_max), ia = input_arg(block_idx);
    auto op = out.arg();
    return cutile_launch_argmax_reduce_blocks_to_u32(s, &ma, &ia, &op, num_blocks, o);
  }
};
struct EmbeddingBatchF16Fn {
  static constexpr const char* name = "embedding_batch_f16";
  template <class I, class T, class O>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, I& token_ids, T& table, O& out) {
    auto ia = input_arg(token_ids), ta = input_arg(table);
    auto op = out.arg();
    return cutile_launch_embedding_batch_f16(s, &ia, &ta, &op, o);
  }
};
struct GatherRowF16Fn {
  static constexpr const char* name = "gather_row_f16";
  template <class S, class O>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, S& src, O& out, int32_t row_idx) {
    auto sa = input_arg(src);
    auto op = out.arg();
    return cutile_launch_gather_row_f16(s, &sa, &op, row_idx, o);
  }
};
// The five sequence-layout attention kernels share one C entry point (cutile_launch_fmha_seq_f16).
template <bool Causal>
struct SeqAttentionFn {          // kv_len and query_start by value
  static constexpr const char* name = "fmha_prefill_causal";
  template <class Q, class K, class V, class O>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, Q& q, K& k, V& v, O& out, float qk_scale,
                                int32_t query_group_size, int32_t kv_len, int32_t query_start) {
    auto qa = input_arg(q), ka = input_arg(k), va = input_arg(v);
    auto op = out.arg();
    return cutile_launch_fmha_seq_f16(s, &qa, &ka, &va, &op, qk_scale, query_group_size, kv_len, query_start, nullptr, 0, Causal, o);
  }
};
template <bool Causal, bool KvLenFromPosition>
struct SeqAttentionDynposFn {    // the position in device memory
  static constexpr const char* name = "fmha_causal";
  template <class Q, class K, class V, class O, class P>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, Q& q, K& k, V& v, O& out, float qk_scale,
                                int32_t query_group_size, P& position_start) {
    auto qa = input_arg(q), ka = input_arg(k), va = input_arg(v), pa = input_arg(position_start);
    auto op = out.arg();
    return cutile_launch_fmha_seq_f16(s, &qa, &ka, &va, &op, qk_scale, query_group_size, 0, 0, &pa, KvLenFromPosition, Causal, o);
  }
};
struct GemmPersistentFn {
  static constexpr const char* name = "gemm_persistent";
  template <class Z, class X, class Yv>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, Z& z, X& x, Yv& y) {
    auto zm = z.arg();
    auto xa = input_arg(x), ya = input_arg(y);
    return cutile_launch_gemm_persistent(s, &zm, &xa, &ya, o);
  }
};
struct MappedTileIndexFn {
  static constexpr const char* name = "mapped_tile_index";
  template <class Z>
  static cutile_status_t launch(cutile_stream_t s, const cutile_launch_opts_t* o, Z& z) {
    auto zm = z.arg();
    return cutile_launch_mapped_tile_index(s, &zm, o);
  }
};
}  // namespace kernels

// saxpy(y: partition, a, x) -> (y, a, x)        cutile-examples/examples/saxpy.rs:12-17
template <class Y, class A, class X> auto saxpy(Y&& y, A&& a, X&& x) { return make_launcher<kernels::SaxpyFn>(std::forward<Y>(y), std::forward<A>(a), std::forward<X>(x)); }
// axpy(z: partition, a, x, y) -> (z, a, x, y)   three-operand form, rank 1
template <class Z, class A, class X, class Y> auto axpy(Z&& z, A&& a, X&& x, Y&& y) { return make_launcher<kernels::AxpyFn>(std::forward<Z>(z), std::forward<A>(a), std::forward<X>(x), std::forward<Y>(y)); }
// add(z: partition, x, y) -> (z, x, y)          README.md:29-38
template <class Z, class X, class Y> auto add(Z&& z, X&& x, Y&& y) { return make_launcher<kernels::AddFn>(std::forward<Z>(z), std::forward<X>(x), std::forward<Y>(y)); }
// rms_norm_f16(x, w, out: partition [1,N], eps) -> (x, w, out, eps)   cutile-kernels/src/norms.rs:22-27
template <class X, class W, class O> auto rms_norm_f16(X&& x, W&& w, O&& out, float eps) { return make_launcher<kernels::RmsNormF16Fn>(std::forward<X>(x), std::forward<W>(w), std::forward<O>(out), eps); }
// rms_norm(x, w, out: partition [1,N], eps) -> (x, w, out, eps), f32   cutile-examples/examples/rms_norm.rs:17-23
template <class X, class W, class O> auto rms_norm(X&& x, W&& w, O&& out, float eps) { return make_launcher<kernels::RmsNormF32Fn>(std::forward<X>(x), std::forward<W>(w), std::forward<O>(out), eps); }
// softmax(x, y: partition [BM,BN]) -> (x, y)    cutile-benchmarks/benches/softmax.rs:23-26
template <class X, class Y> auto softmax(X&& x, Y&& y) { return make_launcher<kernels::SoftmaxFn>(std::forward<X>(x), std::forward<Y>(y)); }
// the benchmark programs' all-f16 forms: rms_norm(x, w, out: [1,N], eps) with .generics({N, BLOCK_SIZE}); softmax(x, y: [BM,BN])
template <class X, class W, class O> auto rms_norm_all_f16(X&& x, W&& w, O&& out, float eps) { return make_launcher<kernels::RmsNormAllF16Fn>(std::forward<X>(x), std::forward<W>(w), std::forward<O>(out), eps); }
template <class X, class Y> auto softmax_all_f16(X&& x, Y&& y) { return make_launcher<kernels::SoftmaxAllF16Fn>(std::forward<X>(x), std::forward<Y>(y)); }
// relu(input_output: partition [D]) -> (input_output)                  cutile-examples/examples/async_mlp.rs:56-61
template <class IO> auto relu(IO&& io) { return make_launcher<kernels::ReluFn>(std::forward<IO>(io)); }
// dropout(p, _x, x_keep, out: partition [S]) -> (p, _x, x_keep, out)     cutile-examples/examples/dropout.rs:17-32
template <class X, class XK, class O> auto dropout(float p, X&& x, XK&& x_keep, O&& out) { return make_launcher<kernels::DropoutFn>(p, std::forward<X>(x), std::forward<XK>(x_keep), std::forward<O>(out)); }
// scale_ptr(out_ptr, in_ptr, scale, len) on raw device pointers; .grid(..) is required   cutile-examples/examples/scale_ptr.rs:26-80
inline auto scale_ptr(void* out_ptr, void* in_ptr, float scale, int32_t len) { return make_launcher<kernels::ScalePtrFn>(out_ptr, in_ptr, scale, len); }
// matvec(z: partition [BM], x, y, k) -> (z, x, y, k): z <- z + x·y       cutile-examples/examples/async_mlp.rs:38-54
template <class Z, class X, class Y> auto matvec(Z&& z, X&& x, Y&& y, int32_t k) { return make_launcher<kernels::MatvecFn>(std::forward<Z>(z), std::forward<X>(x), std::forward<Y>(y), k); }
// batch_matmul(c: partition [1,BM,BN], a, b, k) -> (c, a, b, k)          cutile-examples/examples/batch_matmul.rs:16-44
template <class Cp, class A, class B> auto batch_matmul(Cp&& c, A&& a, B&& b, int32_t k) { return make_launcher<kernels::BatchMatmulFn>(std::forward<Cp>(c), std::forward<A>(a), std::forward<B>(b), k); }
// gemm(z: partition [BM,BN], x, y, k) -> (z, x, y, k): z <- z + x·y   cutile-benchmarks/benches/gemm.rs:25-30
template <class Z, class X, class Y> auto gemm(Z&& z, X&& x, Y&& y, int32_t k) { return make_launcher<kernels::GemmFn<true>>(std::forward<Z>(z), std::forward<X>(x), std::forward<Y>(y), k); }
// gemm_zero_init: accumulator starts at 0                              cutile-examples/examples/gemm.rs:20-36
template <class Z, class X, class Y> auto gemm_zero_init(Z&& z, X&& x, Y&& y, int32_t k) { return make_launcher<kernels::GemmFn<false>>(std::forward<Z>(z), std::forward<X>(x), std::forward<Y>(y), k); }
// fmha(out: partition [1,BM,D], q, k, v, qk_scale, input_pos, query_group_size)   flash_attention_causal.rs:32-40
template <class O, class Q, class K, class V> auto fmha(O&& out, Q&& q, K&& k, V&& v, float scale, int32_t input_pos, int32_t group) { return make_launcher<kernels::FmhaFn<false>>(std::forward<O>(out), std::forward<Q>(q), std::forward<K>(k), std::forward<V>(v), scale, input_pos, group); }
template <class O, class Q, class K, class V> auto fmha_causal(O&& out, Q&& q, K&& k, V&& v, float scale, int32_t input_pos, int32_t group) { return make_launcher<kernels::FmhaFn<true>>(std::forward<O>(out), std::forward<Q>(q), std::forward<K>(k), std::forward<V>(v), scale, input_pos, group); }
// linear_tile(z: partition [BM,BN], x, y, x_scales, y_scales, alpha)   cutile-examples/examples/mxfp8.rs:35-42 (f8e4m3fn x, y) and nvfp4.rs:39-51 (f4e2m1fnx2 x, y)
template <class Z, class X, class Y, class XS, class YS> auto linear_tile(Z&& z, X&& x, Y&& y, XS&& xs, YS&& ys, float alpha) { return make_launcher<kernels::LinearTileMxfp8Fn>(std::forward<Z>(z), std::forward<X>(x), std::forward<Y>(y), std::forward<XS>(xs), std::forward<YS>(ys), alpha); }
// add_rms_norm_f16(residual, x, w, out: [1,N], residual_out: [1,N], eps)      cutile-kernels/src/norms.rs:76-83
template <class R, class X, class W, class O, class RO> auto add_rms_norm_f16(R&& residual, X&& x, W&& w, O&& out, RO&& residual_out, float eps) { return make_launcher<kernels::AddRmsNormF16Fn>(std::forward<R>(residual), std::forward<X>(x), std::forward<W>(w), std::forward<O>(out), std::forward<RO>(residual_out), eps); }
// qk_norm_f16(q, k, q_weight, k_weight, out: [1,N], eps, num_q_rows)          cutile-kernels/src/norms.rs:152-160
template <class Q, class K, class QW, class KW, class O> auto qk_norm_f16(Q&& q, K&& k, QW&& qw, KW&& kw, O&& out, float eps, int32_t num_q_rows) { return make_launcher<kernels::QkNormF16Fn>(std::forward<Q>(q), std::forward<K>(k), std::forward<QW>(qw), std::forward<KW>(kw), std::forward<O>(out), eps, num_q_rows); }
// add_2d_f16(out: [1,BLOCK], lhs, rhs) / silu_mul_2d_f16(out: [1,BLOCK], gate, up)   cutile-kernels/src/pointwise.rs:20-24, 51-55
template <class O, class A, class B> auto add_2d_f16(O&& out, A&& lhs, B&& rhs) { return make_launcher<kernels::Pointwise2dF16Fn<false>>(std::forward<O>(out), std::forward<A>(lhs), std::forward<B>(rhs)); }
template <class O, class A, class B> auto silu_mul_2d_f16(O&& out, A&& gate, B&& up) { return make_launcher<kernels::Pointwise2dF16Fn<true>>(std::forward<O>(out), std::forward<A>(gate), std::forward<B>(up)); }
// rope_seq_f16(x, inv_freq, out: [1,1,D/2], position_start)                    cutile-kernels/src/positional.rs:18-23
template <class X, class F, class O> auto rope_seq_f16(X&& x, F&& inv_freq, O&& out, int32_t position_start) { return make_launcher<kernels::RopeSeqF16Fn>(std::forward<X>(x), std::forward<F>(inv_freq), std::forward<O>(out), position_start); }
// rope_seq_dynpos_f16(x, inv_freq, position_start: [1] u32, out)               positional.rs:75-80
template <class X, class F, class P, class O> auto rope_seq_dynpos_f16(X&& x, F&& inv_freq, P&& position_start, O&& out) { return make_launcher<kernels::RopeSeqDynposF16Fn>(std::forward<X>(x), std::forward<F>(inv_freq), std::forward<P>(position_start), std::forward<O>(out)); }
// qk_rope_dynpos_f16(q, k, inv_freq, position_start, out, num_q_heads)         positional.rs:141-148
template <class Q, class K, class F, class P, class O> auto qk_rope_dynpos_f16(Q&& q, K&& k, F&& inv_freq, P&& position_start, O&& out, int32_t num_q_heads) { return make_launcher<kernels::QkRopeDynposF16Fn>(std::forward<Q>(q), std::forward<K>(k), std::forward<F>(inv_freq), std::forward<P>(position_start), std::forward<O>(out), num_q_heads); }

// kv_cache_update_seq_f16(new_k, new_v, k_cache: [1,BM_S,BLOCK], v_cache, position_start (= 0), seq_len)   cutile-kernels/src/kv_cache.rs:21-28
template <class NK, class NV, class KC, class VC> auto kv_cache_update_seq_f16(NK&& new_k, NV&& new_v, KC&& k_cache, VC&& v_cache, int32_t position_start, int32_t seq_len) { return make_launcher<kernels::KvCacheUpdateSeqF16Fn>(std::forward<NK>(new_k), std::forward<NV>(new_v), std::forward<KC>(k_cache), std::forward<VC>(v_cache), position_start, seq_len); }
// kv_cache_update_seq_dynpos_f16(new_k, new_v, k_cache: [1,MAX_SEQ,BLOCK], v_cache, position_start: [1] u32, seq_len)   kv_cache.rs:68-79
template <class NK, class NV, class KC, class VC, class P> auto kv_cache_update_seq_dynpos_f16(NK&& new_k, NV&& new_v, KC&& k_cache, VC&& v_cache, P&& position_start, int32_t seq_len) { return make_launcher<kernels::KvCacheUpdateSeqDynposF16Fn>(std::forward<NK>(new_k), std::forward<NV>(new_v), std::forward<KC>(k_cache), std::forward<VC>(v_cache), std::forward<P>(position_start), seq_len); }
// fmha_decode_gqa_split(q, k, v, att_out: [1,GROUP,D], lse_out: [1,GROUP], qk_scale, position_start: [1] u32)   cutile-kernels/src/attention.rs:737-755
template <class Q, class K, class V, class A, class L, class P> auto fmha_decode_gqa_split(Q&& q, K&& k, V&& v, A&& att_out, L&& lse_out, float qk_scale, P&& position_start) { return make_launcher<kernels::FmhaDecodeGqaSplitFn>(std::forward<Q>(q), std::forward<K>(k), std::forward<V>(v), std::forward<A>(att_out), std::forward<L>(lse_out), qk_scale, std::forward<P>(position_start)); }
// splitk_reduce_merge(att_partial, lse_partial, out: [1,GROUP,CHUNK_D])          attention.rs:917-930
template <class A, class L, class O> auto splitk_reduce_merge(A&& att_partial, L&& lse_partial, O&& out) { return make_launcher<kernels::SplitkReduceMergeFn>(std::forward<A>(att_partial), std::forward<L>(lse_partial), std::forward<O>(out)); }
// qk_norm_rope_kv_prefill_raw_f16 / qk_norm_rope_kv_decode_raw_f16 take raw device pointers (fused_transformer.rs:22-47,
// 356-372): call cutile_launch_qk_norm_rope_kv_prefill_raw_f16 / ..._decode_raw_f16 of the C ABI with
// tensor.device_ptr() values; there is no tensor argument to hand back, so they have no launcher object here.
// attention_decode_kernel_grouped (experimental/attention.rs:385-846) likewise: raw pointers with shape and stride
// arrays, cutile_launch_attention_decode_kernel_grouped_f16 of the C ABI.
// group_gemm_f16_nt_desc(a_ptrs, b_ptrs, c_ptrs, a_metas, b_metas, c_metas, num_groups); needs .grid({NUM_SM, 1, 1}) or the NUM_SM generic   cutile-kernels/src/experimental/moe.rs:73-81
template <class AP, class BP, class CP, class AM, class BM_, class CM> auto group_gemm_f16_nt_desc(AP&& a_ptrs, BP&& b_ptrs, CP&& c_ptrs, AM&& a_metas, BM_&& b_metas, CM&& c_metas, int32_t num_groups) { return make_launcher<kernels::GroupGemmF16NtDescFn>(std::forward<AP>(a_ptrs), std::forward<BP>(b_ptrs), std::forward<CP>(c_ptrs), std::forward<AM>(a_metas), std::forward<BM_>(b_metas), std::forward<CM>(c_metas), num_groups); }
// argmax_blocks_f16(logits, block_max: [1], block_idx: [1], len)                  cutile-kernels/src/argmax.rs:21-26
template <class L, class M, class I> auto argmax_blocks_f16(L&& logits, M&& block_max, I&& block_idx, int32_t len) { return make_launcher<kernels::ArgmaxBlocksF16Fn>(std::forward<L>(logits), std::forward<M>(block_max), std::forward<I>(block_idx), len); }
// lm_head_argmax_blocks_f16(weights, hidden, block_max: [1], block_idx: [1], vocab_size)   argmax.rs:88-94
template <class W, class H, class M, class I> auto lm_head_argmax_blocks_f16(W&& weights, H&& hidden, M&& block_max, I&& block_idx, int32_t vocab_size) { return make_launcher<kernels::LmHeadArgmaxBlocksF16Fn>(std::forward<W>(weights), std::forward<H>(hidden), std::forward<M>(block_max), std::forward<I>(block_idx), vocab_size); }
// argmax_reduce_blocks_to_u32(block_max, block_idx, out: [1], num_blocks)          argmax.rs:173-178
template <class M, class I, class O> auto argmax_reduce_blocks_to_u32(M&& block_max, I&& block_idx, O&& out, int32_t num_blocks) { return make_launcher<kernels::ArgmaxReduceBlocksToU32Fn>(std::forward<M>(block_max), std::forward<I>(block_idx), std::forward<O>(out), num_blocks); }
// embedding_batch_f16(token_ids, table, out: [1,BLOCK_SIZE])                       cutile-kernels/src/embeddings.rs:21-25
template <class I, class T, class O> auto embedding_batch_f16(I&& token_ids, T&& table, O&& out) { return make_launcher<kernels::EmbeddingBatchF16Fn>(std::forward<I>(token_ids), std::forward<T>(table), std::forward<O>(out)); }
// gather_row_f16(src, out: [BLOCK_SIZE], row_idx)                                  cutile-kernels/src/pointwise.rs:86-90
template <class S, class O> auto gather_row_f16(S&& src, O&& out, int32_t row_idx) { return make_launcher<kernels::GatherRowF16Fn>(std::forward<S>(src), std::forward<O>(out), row_idx); }
// flash_attn_causal_seq_f16(q, k, v, out: [BM,1,D], qk_scale, query_group_size, kv_len, query_start)   attention.rs:21-30
template <class Q, class K, class V, class O> auto flash_attn_causal_seq_f16(Q&& q, K&& k, V&& v, O&& out, float qk_scale, int32_t query_group_size, int32_t kv_len, int32_t query_start) { return make_launcher<kernels::SeqAttentionFn<true>>(std::forward<Q>(q), std::forward<K>(k), std::forward<V>(v), std::forward<O>(out), qk_scale, query_group_size, kv_len, query_start); }
// flash_attn_causal_seq_dynpos_f16(q, k, v, out: [BM,1,D], qk_scale, query_group_size, position_start: [1] u32)   attention.rs:128-136
template <class Q, class K, class V, class O, class P> auto flash_attn_causal_seq_dynpos_f16(Q&& q, K&& k, V&& v, O&& out, float qk_scale, int32_t query_group_size, P&& position_start) { return make_launcher<kernels::SeqAttentionDynposFn<true, true>>(std::forward<Q>(q), std::forward<K>(k), std::forward<V>(v), std::forward<O>(out), qk_scale, query_group_size, std::forward<P>(position_start)); }
// fmha_prefill_causal<.., CAUSAL, ..>(q, k, v, out: [BM,1,D], qk_scale, query_group_size, kv_len, query_start)   attention.rs:242-263
template <bool CAUSAL = true, class Q, class K, class V, class O> auto fmha_prefill_causal(Q&& q, K&& k, V&& v, O&& out, float qk_scale, int32_t query_group_size, int32_t kv_len, int32_t query_start) { return make_launcher<kernels::SeqAttentionFn<CAUSAL>>(std::forward<Q>(q), std::forward<K>(k), std::forward<V>(v), std::forward<O>(out), qk_scale, query_group_size, kv_len, query_start); }
// fmha_prefill_gqa<.., GROUP, M_EFF, CAUSAL, ..>(q, k, v, out: [BM,GROUP,D], qk_scale, query_group_size, kv_len, query_start)   attention.rs:408-432
template <bool CAUSAL = true, class Q, class K, class V, class O> auto fmha_prefill_gqa(Q&& q, K&& k, V&& v, O&& out, float qk_scale, int32_t query_group_size, int32_t kv_len, int32_t query_start) { return make_launcher<kernels::SeqAttentionFn<CAUSAL>>(std::forward<Q>(q), std::forward<K>(k), std::forward<V>(v), std::forward<O>(out), qk_scale, query_group_size, kv_len, query_start); }
// fmha_causal<.., CAUSAL, ..>(q, k, v, out: [BM,1,D], qk_scale (the f16 value, widened), query_group_size, position_start: [1] u32)   attention.rs:598-612
template <bool CAUSAL = true, class Q, class K, class V, class O, class P> auto fmha_causal(Q&& q, K&& k, V&& v, O&& out, float qk_scale, int32_t query_group_size, P&& position_start) { return make_launcher<kernels::SeqAttentionDynposFn<CAUSAL, false>>(std::forward<Q>(q), std::forward<K>(k), std::forward<V>(v), std::forward<O>(out), qk_scale, query_group_size, std::forward<P>(position_start)); }
// gemm_persistent(z: mapped partition [BM,BN], x, y) -> (z's partition, x, y)   cutile-examples/examples/persistent_gemm.rs:35-45
template <class Z, class X, class Y> auto gemm_persistent(Z&& z, X&& x, Y&& y) { return make_launcher<kernels::GemmPersistentFn>(std::forward<Z>(z), std::forward<X>(x), std::forward<Y>(y)); }
// write_flat_index_rank{1,2,3}(z: mapped i32 partition) -> (z's partition)      cutile/tests/gpu/mapped_partition_schedule_matrix.rs:30-76
template <class Z> auto mapped_tile_index(Z&& z) { return make_launcher<kernels::MappedTileIndexFn>(std::forward<Z>(z)); }

namespace api {
template <class T> struct is_graph_node_memcpy : std::true_type {};
}
template <class T>
struct is_graph_node<api::Memcpy<T>> : std::true_type {};

}  // namespace cutile
