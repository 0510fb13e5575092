// CPU tests of the C++ host surface on the recording stand-in for the HIP
// runtime.  They restate, case by case, the reference's host-only and
// fake-backed tests: cuda-async/tests/{execute_once,error_handling,cuda_graph}.rs,
// cutile/src/tensor.rs:2161-2202, cutile/src/bench.rs:266-291,
// cutile/src/tune.rs (FakeOracle tests), cuda-async/src/device_future.rs:325-384.
#include <unistd.h>
#include <cutile/cutile.hpp>
#include <cutile_hip_testing.h>

#include <atomic>
#include <thread>

#include "check.hpp"

using namespace cutile;

static std::shared_ptr<Stream> fresh_stream() {
  auto dev = Device::create(0).unwrap();
  return dev->new_stream().unwrap();
}
static int launches() { return cutile_testing_launch_count(); }
static std::string last_symbol() {
  cutile_testing_launch_record_t r;
  cutile_testing_get_launch(launches() - 1, &r);
  return r.symbol;
}

// An op that counts how often it executes (execute_once.rs:24 uses a boxed op the same way).
struct Counting : DeviceOp<Counting, int> {
  std::shared_ptr<std::atomic<int>> n;
  int v;
  Counting(std::shared_ptr<std::atomic<int>> n, int v) : n(std::move(n)), v(v) {}
  Result<int> execute(const ExecutionContext&) && {
    n->fetch_add(1);
    return v;
  }
};
struct Failing : DeviceOp<Failing, int> {
  Result<int> execute(const ExecutionContext&) && { return DeviceError::launch("boom"); }
};

TEST(combinators_compose_and_propagate_errors) {
  auto s = fresh_stream();
  CHECK(value(3).map([](int x) { return x + 1; }).sync_on(s).unwrap() == 4);
  int seen = 0;
  auto r = value(5).inspect([&](const int& x) { seen = x; }).then([](int x) { return value(x * 2); }).sync_on(s);
  CHECK(r.unwrap() == 10 && seen == 5);
  auto z = zip(value(1), 2.5, value(std::string("x"))).sync_on(s).unwrap();
  CHECK(std::get<0>(z) == 1 && std::get<1>(z) == 2.5 && std::get<2>(z) == "x");
  CHECK(zip(1, 2, 3).first().sync_on(s).unwrap() == 1);
  CHECK(zip(1, 2, 3).last().sync_on(s).unwrap() == 3);
  // an error short-circuits the chain: the closure after it never runs
  bool ran = false;
  auto e = Failing{}.then([&](int) { ran = true; return value(0); }).sync_on(s);
  CHECK(e.is_err() && e.error().kind == DeviceError::Kind::Launch && !ran);
  auto ez = zip(value(1), Failing{}).sync_on(s);
  CHECK(ez.is_err());
}

TEST(shared_and_unzip_execute_once) {
  auto s = fresh_stream();
  auto n = std::make_shared<std::atomic<int>>(0);
  auto sh = Counting(n, 7).shared();
  auto a = sh;  // clones share the result
  auto b = sh;
  CHECK(*std::move(a).sync_on(s).unwrap() == 7);
  CHECK(*std::move(b).sync_on(s).unwrap() == 7);
  CHECK(*std::move(sh).sync_on(s).unwrap() == 7);
  CHECK(n->load() == 1);
  // unzip: the tuple op runs once, each half takes its element
  auto m = std::make_shared<std::atomic<int>>(0);
  auto [x, y] = Counting(m, 1).map([](int v) { return std::make_tuple(v, std::string("s")); }).unzip();
  CHECK(std::move(y).sync_on(s).unwrap() == "s");
  CHECK(std::move(x).sync_on(s).unwrap() == 1);
  CHECK(m->load() == 1);
  // shared(arc): already computed
  CHECK(*shared(std::make_shared<int>(9)).sync_on(s).unwrap() == 9);
  CHECK(unwrap_arc(std::make_shared<int>(4)) == 4);
  auto two = std::make_shared<int>(4);
  auto other = two;
  CHECK_THROWS(unwrap_arc(two), "multiple owners");
  // boxed ops go into one container
  std::vector<BoxedDeviceOp<int>> ops;
  ops.push_back(value(1).boxed());
  ops.push_back(Counting(n, 2).boxed());
  int sum = 0;
  for (auto& o : ops) sum += std::move(o).sync_on(s).unwrap();
  CHECK(sum == 3);
}

TEST(execution_is_not_reentrant_on_a_thread) {
  auto s = fresh_stream();
  auto s2 = fresh_stream();
  // sync_on inside a then-closure is rejected (device_operation.rs:27-55; tests/cuda_graph.rs:130-165)
  std::optional<DeviceError> inner;
  auto r = value(1).then([&](int x) {
    auto nested = value(2).sync_on(s2);
    if (nested.is_err()) inner = nested.error();
    return value(x);
  }).sync_on(s);
  CHECK(r.is_ok() && inner && inner->message.find("non-reentrant") != std::string::npos);
  CHECK(cutile_execution_lock_held() == 0);  // released after the outer op
  CHECK(value(1).sync_on(s).is_ok());        // and usable again
}

TEST(default_policy_round_robins_over_four_streams) {
  std::vector<cutile_stream_t> seen;
  for (int i = 0; i < 9; ++i) seen.push_back(next_stream().unwrap()->raw());
  CHECK(seen[0] != seen[1] && seen[1] != seen[2] && seen[2] != seen[3]);
  CHECK(seen[4] == seen[0] && seen[5] == seen[1] && seen[8] == seen[0]);
  // contexts are per thread: another thread gets its own pool
  cutile_stream_t other = nullptr;
  std::thread([&] { other = next_stream().unwrap()->raw(); }).join();
  CHECK(other != nullptr && other != seen[0] && other != seen[1] && other != seen[2] && other != seen[3]);
  // sync() uses the policy
  CHECK(value(1).sync().unwrap() == 1);
}

TEST(explicit_policies_and_double_initialisation) {
  CHECK(init_device_contexts(0, 1).is_ok());
  auto again = init_device_contexts(0, 1);  // error_handling.rs:137-156
  CHECK(again.is_err() && again.error().message.find("Context already initialized.") != std::string::npos);
  CHECK(init_device(0, PolicyKind::SingleStream).is_ok());
  auto dup = init_device(0, PolicyKind::StreamPoolRoundRobin, 2);
  CHECK(dup.is_err() && dup.error().message.find("Device is already initialized.") != std::string::npos);
  auto a = next_stream().unwrap()->raw();
  auto b = next_stream().unwrap()->raw();
  CHECK(a == b);  // SingleStream
  // invalid device ordinal surfaces as a driver error (error_handling.rs:174-190)
  auto bad = Device::create(7);
  CHECK(bad.is_err() && bad.error().kind == DeviceError::Kind::Driver);
  set_default_device(0);
  CHECK(get_default_device() == 0);
}

struct FakeAlloc : DeviceAllocation {  // cutile/src/tensor.rs:2146-2159
  size_t len;
  explicit FakeAlloc(size_t l) : len(l) {}
  void* device_ptr() const override { return (void*)16; }
  size_t len_bytes() const override { return len; }
  int device_id() const override { return 0; }
};

TEST(tensor_extent_validation_vectors) {
  // tensor.rs:2161-2202
  CHECK(addressable_bytes<float>({4}, {1}) == 16);
  CHECK(addressable_bytes<float>({4}, {10}) == 31 * 4);
  CHECK(addressable_bytes<float>({0}, {1}) == 0);
  auto ok = Tensor<float>::from_foreign(std::make_shared<FakeAlloc>(124), {4}, {10});
  CHECK(ok.size() == 4);
  CHECK_THROWS(Tensor<float>::from_foreign(std::make_shared<FakeAlloc>(16), {4}, {10}), "addressable extent");
  CHECK_THROWS(Tensor<float>::from_foreign(std::make_shared<FakeAlloc>(16), {INT32_MAX, INT32_MAX}, {INT32_MAX, INT32_MAX}),
               "addressable extent overflowed");
  // prod(shape) * sizeof(T) must equal the storage size (tensor.rs:739-752)
  CHECK_THROWS(Tensor<float>::from_raw_parts((void*)16, 12, 0, {4}, {1}), "storage size");
}

TEST(meta_tensors_have_metadata_but_no_pointer) {
  auto m = Tensor<float>::from_meta({128, 256});
  CHECK(m.is_meta() && m.size() == 128 * 256 && m.strides() == std::vector<int32_t>({256, 1}));
  CHECK(m.spec().base_ptr_div == 16 && m.spec().shape_div[0] == 16);
  CHECK_THROWS(m.device_pointer(), "meta tensor");
}

TEST(tensor_views_reshape_reinterpret_partition) {
  auto s = fresh_stream();
  auto t = api::arange<float>(1024).sync_on(s).unwrap();
  CHECK(t.shape() == std::vector<int32_t>({1024}) && t.is_contiguous() && t.num_bytes() == 4096);
  // views / slices: offsets accumulate (host-api reference: tensor[110..120])
  auto inner = t.slice({{100, 200}}).unwrap().slice({{10, 20}}).unwrap();
  CHECK(inner.offset_bytes() == 110 * 4 && inner.shape()[0] == 10);
  auto mat = t.view({32, 32}).unwrap();
  auto block = mat.slice({{1, 3}, {2, 6}}).unwrap();
  CHECK(block.offset_bytes() == (32 + 2) * 4 && block.shape() == std::vector<int32_t>({2, 4}) && block.strides() == std::vector<int32_t>({32, 1}));
  CHECK((char*)block.arg().ptr - (char*)t.device_pointer() == (32 + 2) * 4);
  CHECK(t.view({33, 31}).is_err() && t.slice({{0, 2000}}).is_err());
  // reshape consumes; reshape_shared and reinterpret share the allocation
  auto r = std::move(t).reshape({4, 256}).unwrap();
  CHECK(r.strides() == std::vector<int32_t>({256, 1}));
  CHECK(std::move(r).reshape({5, 5}).is_err());
  auto arc = std::make_shared<Tensor<uint32_t>>(api::arange<uint32_t>(4).sync_on(s).unwrap());
  auto fl = Tensor<uint32_t>::reinterpret<float>(arc, {4}).unwrap();
  CHECK(fl->device_pointer() == arc->device_pointer() && fl->shape()[0] == 4);
  CHECK(Tensor<uint32_t>::reinterpret<double>(arc, {4}).is_err());  // byte size must match
  auto two = Tensor<uint32_t>::reshape_shared(arc, {2, 2}).unwrap();
  // partition needs unique storage: the allocation is shared by three handles now
  CHECK(try_partition(arc, {2}).is_err());
  auto solo = api::zeros<float>({128, 256}).sync_on(s).unwrap();
  auto p = std::move(solo).partition({32, 64});
  auto g = p.grid().unwrap();
  CHECK(g[0] == 4 && g[1] == 4 && g[2] == 1);  // tensor.rs:440-442
  auto back = std::move(p).unpartition();
  CHECK(back.size() == 128 * 256);
  auto one = std::make_shared<Tensor<float>>(std::move(back));
  CHECK(try_partition(std::move(one), {128, 256}).is_ok());
}

TEST(transfers_round_trip) {
  auto s = fresh_stream();
  auto host = std::make_shared<std::vector<float>>(std::vector<float>{1, 2, 3, 4, 5, 6});
  auto t = api::copy_host_vec_to_device(host).sync_on(s).unwrap();
  auto d = api::dup(t).sync_on(s).unwrap();
  CHECK(d.device_pointer() != t.device_pointer());
  CHECK(api::to_host_vec(d).sync_on(s).unwrap() == *host);
  auto dst = api::zeros<float>({6}).sync_on(s).unwrap();
  CHECK(api::memcpy(dst, t).sync_on(s).is_ok());
  CHECK(api::to_host_vec(dst).sync_on(s).unwrap() == *host);
  auto small = api::zeros<float>({3}).sync_on(s).unwrap();
  CHECK_THROWS(api::memcpy(small, t), "same number of elements");
  // op-level helpers: reshape / partition / to_host_vec on an op's output
  auto v = api::to_host_vec_op(reshape_op(api::copy_host_vec_to_device(host), {2, 3})).sync_on(s).unwrap();
  CHECK(v == *host);
  // owned storage is released when the tensor goes away
  uint64_t before = cutile_testing_bytes_allocated();
  { auto tmp = api::zeros<float>({1024}).sync_on(s).unwrap(); CHECK(cutile_testing_bytes_allocated() == before + 4096); }
  CHECK(cutile_testing_bytes_allocated() == before);
}

TEST(launchers_hand_arguments_back_in_the_form_given) {
  auto s = fresh_stream();
  cutile_testing_clear_log();
  auto x = std::make_shared<Tensor<float>>(api::arange<float>(32).sync_on(s).unwrap());
  auto x2 = Tensor<float>::reshape_shared(x, {4, 8}).unwrap();
  x.reset();
  int before = launches();
  // owned partition + Arc input: cutile-examples/examples/saxpy.rs:27-45
  auto y = reshape_op(api::arange<float>(32), {4, 8}).sync_on(s).unwrap().partition({2, 2});
  auto [y_out, a_out, x_out] = saxpy(std::move(y), 2.0f, x2).sync_on(s).unwrap();
  CHECK(launches() == before + 2);  // arange for y + the saxpy itself
  CHECK(last_symbol() == "saxpy_entry__f32_r2_flat");
  CHECK(a_out == 2.0f && x_out.get() == x2.get());
  Tensor<float> y_back = std::move(y_out).unpartition();
  CHECK(y_back.shape() == std::vector<int32_t>({4, 8}));
  // borrowed input and in-place partition: nothing changes hands
  Tensor<float> w = api::ones<float>({4, 8}).sync_on(s).unwrap();
  auto res = saxpy(y_back.partition_mut({2, 2}), 1.0f, &w).sync_on(s).unwrap();
  CHECK(std::get<2>(res) == &w && &std::get<0>(res).tensor() == &y_back);
  // arguments may themselves be ops; views are passed as pointer + offset
  auto view = w.slice({{0, 2}}).unwrap();
  auto r2 = saxpy(partition_op(api::zeros<float>({2, 8}), {2, 8}), 3.0f, view).sync_on(s);
  CHECK(r2.is_ok());
  // a launch-time violation is reported before any GPU work
  int n0 = launches();
  auto bad = rms_norm_f16(api::zeros<f16>({4, 64}), api::zeros<f16>({32}), partition_op(api::zeros<f16>({4, 64}), {1, 64}), 1e-6f).sync_on(s);
  CHECK(bad.is_err() && bad.error().kind == DeviceError::Kind::Launch);
  CHECK(launches() == n0 + 3);  // the three fills ran, the kernel did not
  // a tile shape without a matrix-core kernel runs on the any-layout kernel ...
  auto odd_tile = gemm(partition_op(api::zeros<bf16>({64, 64}), {48, 48}), api::zeros<bf16>({64, 64}), api::zeros<bf16>({64, 64}), 64).sync_on(s);
  CHECK(odd_tile.is_ok() && last_symbol() == "gemm_entry__bf16_generic");
  // ... and a key nothing was built for is a kernel-cache error that names what exists
  auto nokernel = fmha(partition_op(api::zeros<bf16>({2, 96, 32}), {1, 48, 32}), api::zeros<bf16>({1, 2, 96, 32}), api::zeros<bf16>({1, 2, 96, 32}),
                       api::zeros<bf16>({1, 2, 96, 32}), 0.125f, 0, 1).sync_on(s);
  CHECK(nokernel.is_err() && nokernel.error().kind == DeviceError::Kind::KernelCache);
  CHECK(nokernel.error().message.find("available:") != std::string::npos);
  // builder methods reach the launcher
  auto g = gemm(partition_op(api::zeros<bf16>({256, 256}), {128, 128}), api::zeros<bf16>({256, 64}), api::zeros<bf16>({64, 256}), 64)
               .generics({"bf16", "128", "128", "64"}).variant("bf16_128x128x64_w2x2").sync_on(s);
  CHECK(g.is_ok() && last_symbol() == "gemm_entry__bf16_128x128x64_w2x2");
  auto wrong = gemm(partition_op(api::zeros<bf16>({256, 256}), {128, 128}), api::zeros<bf16>({256, 64}), api::zeros<bf16>({64, 256}), 64)
                   .grid(1, 1, 1).sync_on(s);
  CHECK(wrong.is_err() && wrong.error().message.find("does not match the inferred partition grid") != std::string::npos);
}

// ---- cache-key identity: cutile/tests/warmup.rs, case by case -------------------------------------------------
static TileFunctionKeyBuilder default_key() {
  return TileFunctionKey::builder("m", "f").source_hash("hash").gpu_name("gfx950").compiler_version("0.0.1").toolchain_fingerprint(
      "AMD clang version 20.0.0");
}
TEST(tile_function_key_distinguishes_everything_that_selects_a_kernel) {
  // cache_key_deterministic
  auto k1 = TileFunctionKey::builder("mod", "fn").generics({"f32"}).source_hash("abc123").gpu_name("gfx950").compiler_version("0.0.1-alpha")
                .toolchain_fingerprint("AMD clang version 20.0.0").build();
  auto k2 = k1;
  CHECK(k1 == k2 && k1.display_hash() == k2.display_hash());
  // different source hash / gpu name / device id / compiler version / toolchain fingerprint / generics
  CHECK(default_key().source_hash("hash_v1").build() != default_key().source_hash("hash_v2").build());
  CHECK(default_key().gpu_name("gfx942").build() != default_key().gpu_name("gfx950").build());
  CHECK(default_key().device_id(0).build() != default_key().device_id(1).build());
  CHECK(default_key().compiler_version("0.0.1").build() != default_key().compiler_version("0.0.2").build());
  CHECK(default_key().toolchain_fingerprint("AMD clang version 19.0.0").build() != default_key().toolchain_fingerprint("AMD clang version 20.0.0").build());
  // the stat-style fallback fingerprint (embedded NULs) must not collide with a version string
  CHECK(default_key().toolchain_fingerprint(std::string("stat\0/opt/rocm/bin/hipcc\094855128\0170000000", 44)).build() !=
        default_key().toolchain_fingerprint("AMD clang version 20.0.0").build());
  CHECK(default_key().generics({"f32"}).build() != default_key().generics({"f16"}).build());
  // cache_key_different_spec_args
  SpecializationBits aligned, misaligned;
  aligned.shape_div = {DivHint::from_value(16), DivHint::from_value(16)};
  aligned.stride_div = {DivHint::from_value(16), DivHint::from_value(16)};
  aligned.stride_one = {false, true};
  aligned.base_ptr_div = DivHint::from_ptr(16);
  misaligned = aligned;
  misaligned.shape_div = {DivHint::from_value(4), DivHint::from_value(4)};
  misaligned.stride_div = {DivHint::from_value(4), DivHint::from_value(4)};
  misaligned.base_ptr_div = DivHint::from_ptr(4);
  CHECK(DivHint::from_value(16).divisor == 16 && DivHint::from_value(48).divisor == 16 && DivHint::from_value(12).divisor == 4 &&
        DivHint::from_value(7).divisor == 1 && DivHint::from_ptr(0x7f0000001008ull).divisor == 8 && DivHint::from_value(64).with_max(8).divisor == 8);
  CHECK(default_key().spec_args({{"x", aligned}}).build() != default_key().spec_args({{"x", misaligned}}).build());
  // cache_key_different_compile_options
  CHECK(default_key().compile_options(CompileOptions().max_divisibility(8)).build() != default_key().compile_options(CompileOptions().max_divisibility(16)).build());
  CHECK(default_key().compile_options(CompileOptions().occupancy(2)).build() != default_key().compile_options(CompileOptions().occupancy(4)).build());
  CHECK(default_key().compile_options(CompileOptions().num_worker_warps_per_cta(4)).build() !=
        default_key().compile_options(CompileOptions().num_worker_warps_per_cta(8)).build());
  CHECK(default_key().compile_options(CompileOptions().occupancy(2)).build() != default_key().build());
  // cache_key_no_field_boundary_ambiguity: also in the digest's input
  auto ka = default_key().gpu_name("sm_9").compiler_version("0").build(), kb = default_key().gpu_name("sm_90").compiler_version("").build();
  CHECK(ka != kb && ka.canonical() != kb.canonical());
  // a constant grid is part of the key, a plain grid is not there at all
  CHECK(default_key().grid(4, 1, 1).build() != default_key().build() && default_key().grid(4, 1, 1).build() != default_key().grid(8, 1, 1).build());
}

TEST(launcher_compile_specialize_and_cache_keys) {
  // .compile() / .compile_on() / .specialize() / .l1_cache_key() / .l2_cache_key() / .const_grid() / .compile_options() / _apply
  // (cutile-macro/src/_module.rs:852-923, kernel_launcher_generator.rs:1036-1044)
  auto s = fresh_stream();
  auto z = [&] { return partition_op(api::zeros<bf16>({256, 256}), {128, 128}); };
  auto x = api::zeros<bf16>({256, 64}).sync_on(s).unwrap();
  auto y = api::zeros<bf16>({64, 256}).sync_on(s).unwrap();
  // specialize: the identity, nothing loaded, nothing launched
  uint64_t loads0 = cutile_module_load_count();
  int n0 = launches();
  auto spec = gemm(z(), &x, &y, 64).generics({"bf16", "128", "128", "64"}).specialize_on(s).unwrap();
  CHECK(launches() == n0 + 1);                                   // the fill of z ran; the kernel did not
  CHECK(spec.l1_cache_key().function_name() == "gemm" && spec.variant() == "bf16_128x128x64_d2x2" && spec.symbol() == "gemm_entry__bf16_128x128x64_d2x2");
  CHECK(spec.l1_cache_key().function_generics == std::vector<std::string>({"bf16", "128", "128", "64"}));
  CHECK(spec.l1_cache_key().spec_args.size() == 3 && spec.l1_cache_key().scalar_hints.size() == 1 && spec.l1_cache_key().scalar_hints[0].second.divisor == 16);
  CHECK(spec.l1_cache_key().gpu_name().find("gfx") == 0 && !spec.l1_cache_key().source_hash().empty() && !spec.l1_cache_key().grid);
  CHECK(spec.l2_cache_key().find("gemm:bf16_128x128x64_d2x2:") == 0);
  // compile: the code object is loaded now ...
  uint64_t loads1 = cutile_module_load_count();
  int n1 = launches();
  CHECK(gemm(z(), &x, &y, 64).compile_on(s).is_ok());
  CHECK(launches() == n1 + 1 && cutile_module_load_count() >= loads1);
  uint64_t loads2 = cutile_module_load_count();
  // ... so the first launch after it loads nothing
  CHECK(gemm(z(), &x, &y, 64).sync_on(s).is_ok() && last_symbol() == "gemm_entry__bf16_128x128x64_d2x2");
  CHECK(cutile_module_load_count() == loads2 && launches() == n1 + 3);
  (void)loads0;
  // compile reports what a launch would: validation still runs
  auto bad = gemm(z(), &x, &y, 64).generics({"bf16", "64", "128", "64"}).compile_on(s);
  CHECK(bad.is_err() && bad.error().message.find("generic BM") != std::string::npos);
  int32_t mode = -1;
  CHECK(cutile_get_launch_mode(&mode) == CUTILE_SUCCESS && mode == 0);        // the mode never leaks out of a call
  // keys: equal for equal launches whatever the extents, different for a misaligned view / options / const grid
  auto key = [&](auto launcher) { return std::move(launcher).l1_cache_key_on(s).unwrap(); };
  auto base = key(gemm(z(), &x, &y, 64));
  CHECK(base == key(gemm(z(), &x, &y, 64)));
  auto x_big = api::zeros<bf16>({512, 64}).sync_on(s).unwrap();
  auto z_big = [&] { return partition_op(api::zeros<bf16>({512, 256}), {128, 128}); };
  CHECK(base == key(gemm(z_big(), &x_big, &y, 64)));                          // extents are not part of the key
  CHECK(base != key(gemm(z(), &x, &y, 64).compile_options(CompileOptions().occupancy(2))));
  CHECK(base != key(gemm(z(), &x, &y, 64).const_grid(2, 2, 1)));
  CHECK(base == key(gemm(z(), &x, &y, 64).grid(2, 2, 1)));                    // a plain grid is a launch parameter only
  CHECK(key(gemm(z(), &x, &y, 64).const_grid(2, 2, 1)) == key(gemm(z(), &x, &y, 64).const_grid(2, 2, 1)));
  auto wide = api::zeros<bf16>({256, 72}).sync_on(s).unwrap();
  auto x_view = wide.slice({{0, 256}, {8, 72}}).unwrap();                    // same shape as x, row stride 72, base 16 bytes in
  auto misaligned = key(gemm(z(), x_view, &y, 64));
  CHECK(base != misaligned && misaligned.spec_args[1].second.stride_div[0].divisor == 8);
  CHECK(key(gemm(z(), &x, &y, 64).compile_options(CompileOptions().max_divisibility(4))).spec_args[1].second.stride_div[0].divisor == 4);
  // l2 key names the resolved kernel; a launch that resolves to another variant has another key
  auto l2a = gemm(z(), &x, &y, 64).l2_cache_key_on(s).unwrap();
  auto l2b = gemm(z(), &x, &y, 64).variant("bf16_128x128x64_w2x2").l2_cache_key_on(s).unwrap();
  CHECK(l2a != l2b && l2b.find("gemm:bf16_128x128x64_w2x2:") == 0);
  // default-stream forms
  CHECK(gemm(z(), &x, &y, 64).compile().is_ok() && gemm(z(), &x, &y, 64).l1_cache_key().unwrap() == base);
  CHECK(gemm(z(), &x, &y, 64).get_launch_grid() == (std::array<uint32_t, 3>{0, 0, 0}) &&
        gemm(z(), &x, &y, 64).const_grid(2, 2, 1).get_launch_grid() == (std::array<uint32_t, 3>{2, 2, 1}));
  // _apply: a launcher over a tuple of materialised arguments
  auto yv = api::ones<float>({32}).sync_on(s).unwrap();
  auto xv = std::make_shared<Tensor<float>>(api::ones<float>({32}).sync_on(s).unwrap());
  auto out = apply_launcher<kernels::SaxpyFn>(std::make_tuple(std::move(yv).partition({8}), 2.0f, xv)).sync_on(s).unwrap();
  CHECK(last_symbol() == "saxpy_entry__f32_r1_flat" && std::get<2>(out).get() == xv.get());
}

TEST(mapped_partitions_validate_and_hand_the_inner_partition_back) {
  auto s = fresh_stream();
  cutile_testing_clear_log();
  // cutile/src/tensor.rs:2203-2345: the launch grid is (num_tile_blocks, 1, 1) when the map can traverse the partition
  auto z = api::zeros<float>({8, 12}).sync_on(s).unwrap();     // logical grid (2, 3) with [4, 4] tiles
  auto grid_of = [&](std::vector<int32_t> map, uint32_t n) { return z.partition_mut({4, 4}).map(std::move(map), n).grid(); };
  CHECK(grid_of({4, 1}, 3).unwrap() == (std::array<uint32_t, 3>{3, 1, 1}));
  CHECK(grid_of({4, 1}, 7).error().message.find("num_tile_blocks cannot exceed the streamed logical tile count") != std::string::npos);
  CHECK(grid_of({1, OWNED}, 2).unwrap()[0] == 2 && grid_of({1, OWNED}, 3).is_err());
  CHECK(grid_of({OWNED, OWNED}, 1).error().message.find("at least one streamed (non-OWNED) map axis") != std::string::npos);
  CHECK(grid_of({OWNED, 1}, 3).unwrap()[0] == 3);
  CHECK(grid_of({4, 1}, 0).error().message.find("num_tile_blocks > 0") != std::string::npos);
  CHECK(grid_of({1}, 2).error().message.find("map rank must match the logical partition grid rank") != std::string::npos);
  CHECK(grid_of({1, 1, 1, 1}, 2).error().message.find("rank-1 through rank-3 map shape") != std::string::npos);
  CHECK_THROWS(z.partition_mut({4, 4}).prefix().map({1, 1}, 2), "cannot be mapped");   // tensor.rs:319-323
  // the schedule as a host-visible map: bands of two tile rows, column by column
  auto m = z.partition_mut({4, 4}).map({2, 1}, 2);
  CHECK(m.index(0).unwrap() == (std::array<uint32_t, 3>{0, 0, 0}) && m.index(1).unwrap() == (std::array<uint32_t, 3>{1, 0, 0}) &&
        m.index(2).unwrap() == (std::array<uint32_t, 3>{0, 1, 0}) && m.index(5).unwrap() == (std::array<uint32_t, 3>{1, 2, 0}));
  CHECK(m.index(6).is_err());
  // iter_indices_within (cutile/src/_core.rs:912-930): the schedule over the range's lengths, shifted by its starts
  auto sub = m.indices_within({{0, -1}, {1, 2}}).unwrap();
  CHECK(sub.size() == 4 && sub[0] == (std::array<uint32_t, 3>{0, 1, 0}) && sub[1] == (std::array<uint32_t, 3>{1, 1, 0}) &&
        sub[2] == (std::array<uint32_t, 3>{0, 2, 0}) && sub[3] == (std::array<uint32_t, 3>{1, 2, 0}));
  CHECK(m.indices_within({{1, 0}, {0, -1}}).unwrap().empty());
  CHECK(m.indices_within({{-1, 2}, {0, -1}}).error().message.find("is negative") != std::string::npos);   // partition_index_schedules.rs:553
  CHECK(m.indices_within({{0, -1}}).is_err());
  // persistent_gemm.rs:96-108: the launcher takes the mapped partition and returns the partition
  auto x = api::zeros<float>({64, 32}).sync_on(s).unwrap();
  auto y = api::zeros<float>({32, 64}).sync_on(s).unwrap();
  auto out = api::zeros<float>({64, 64}).sync_on(s).unwrap().partition({16, 16}).map({4, 1}, 4);
  auto [zp, xb, yb] = gemm_persistent(std::move(out), &x, &y).generics({"f32", "16", "16", "8", "4", "1"}).sync_on(s).unwrap();
  CHECK(last_symbol() == "gemm_persistent_entry__f32_generic");
  CHECK(xb == &x && yb == &y);
  Tensor<float> z_back = std::move(zp).unpartition();
  CHECK(z_back.shape() == std::vector<int32_t>({64, 64}));
  auto bad = gemm_persistent(z_back.partition_mut({16, 16}).map({4, 1}, 4), &x, &y).generics({"f32", "16", "16", "8", "2", "1"}).sync_on(s);
  CHECK(bad.is_err() && bad.error().message.find("MAP_SHAPE") != std::string::npos);
  auto short_y = api::zeros<float>({16, 64}).sync_on(s).unwrap();
  auto ties = gemm_persistent(z_back.partition_mut({16, 16}).map({4, 1}, 4), &x, &short_y).generics({"f32", "16", "16", "8", "4", "1"}).sync_on(s);
  CHECK(ties.is_err() && ties.error().message.find("ceil(dim(x, 1)/BK) <= ceil(dim(y, 0)/BK)") != std::string::npos);
}

TEST(graph_capture_replay_and_failure_matrix) {
  auto s = fresh_stream();
  Tensor<float> out = api::zeros<float>({1024}).sync_on(s).unwrap();
  Tensor<float> w = api::ones<float>({1024}).sync_on(s).unwrap();
  Tensor<float> staging = api::zeros<float>({1024}).sync_on(s).unwrap();
  cutile_testing_clear_log();
  // scope: two launches recorded, none executed eagerly twice (cuda_graphs.rs example shape)
  auto graph = HipGraph<Unit>::scope(s, [&](Scope& sc) -> Result<Unit> {
    CUTILE_TRY(sc.record(saxpy(out.partition_mut({128}), 2.0f, &w)));
    CUTILE_TRY(sc.record(saxpy(out.partition_mut({64}), 1.0f, &w)));
    CUTILE_TRY(sc.record(api::memcpy(staging, out)));
    return ok();
  }).unwrap();
  CHECK(launches() == 2);
  cutile_testing_launch_record_t rec;
  cutile_testing_get_launch(0, &rec);
  CHECK(rec.in_capture == 1 && rec.from_graph_replay == 0);
  CHECK(graph.launch().sync_on(s).is_ok());
  CHECK(graph.launch().sync_on(s).is_ok());
  CHECK(launches() == 6);  // each replay re-issues both kernels
  cutile_testing_get_launch(5, &rec);
  CHECK(rec.from_graph_replay == 1 && std::string(rec.symbol) == "saxpy_entry__f32_r1_flat");
  CHECK(cutile_execution_lock_held() == 0);
  // update runs on the graph's stream without a sync
  CHECK(graph.update(api::memcpy(staging, w)).is_ok());
  // graph_on keeps the op's output from the capture pass
  auto g2 = saxpy(partition_op(api::zeros<float>({256}), {128}), 1.0f, api::ones<float>({256})).graph_on(s);
  CHECK(g2.is_err());  // allocation inside a capture is refused by the runtime (hipErrorStreamCaptureUnsupported)
  auto g3 = value(41).map([](int v) { return v + 1; }).graph_on(s).unwrap();
  CHECK(*g3.take_output() == 42 && !g3.take_output());
  // failure matrix (cuda_graph.rs:81-104): op fails -> its error, capture still ended
  auto f1 = Failing{}.graph_on(s);
  CHECK(f1.is_err() && f1.error().message == "boom");
  CHECK(value(1).sync_on(s).is_ok());  // the stream is usable: capture was closed
  cutile_testing_inject_failure("hipStreamEndCapture", 901, 1);
  auto f2 = value(1).graph_on(s);
  CHECK(f2.is_err() && f2.error().kind == DeviceError::Kind::Driver && f2.error().code == 901);
  cutile_testing_inject_failure("hipGraphInstantiateWithFlags", 2, 1);
  CHECK(value(1).graph_on(s).is_err());
  cutile_testing_inject_failure("hipGraphUpload", 2, 1);
  CHECK(value(1).graph_on(s).is_err());
  // a body that throws still ends the capture and releases the lock (cuda_graph.rs:400-505)
  bool threw = false;
  try {
    (void)HipGraph<Unit>::scope(s, [&](Scope&) -> Result<Unit> { throw std::runtime_error("body panicked"); });
  } catch (const std::runtime_error&) { threw = true; }
  CHECK(threw && cutile_execution_lock_held() == 0 && value(1).sync_on(s).is_ok());
  // nested execution inside a scope is rejected
  auto nested = HipGraph<Unit>::scope(s, [&](Scope&) -> Result<Unit> {
    auto r = value(1).sync_on(s);
    return r.is_err() ? Result<Unit>(r.error()) : ok();
  });
  CHECK(nested.is_err() && nested.error().message.find("non-reentrant") != std::string::npos);
}

TEST(device_future_states) {
  auto s = fresh_stream();
  // failed(): first poll yields the error, a second poll is a bug (device_future.rs:88-97,312-316)
  auto f = DeviceFuture<Value<int>>::failed(DeviceError::scheduling("no stream"));
  CHECK(f.state() == DeviceFutureState::Failed);
  auto r = f.poll([] {});
  CHECK(r && r->is_err() && r->error().kind == DeviceError::Kind::Scheduling && f.state() == DeviceFutureState::Complete);
  CHECK_THROWS(f.poll([] {}), "Poll called after completion.");
  // a scheduled future: Idle -> (Executing ->) Complete, result delivered once
  auto fut = value(5).map([](int v) { return v * 3; }).schedule_on(s);
  CHECK(fut.state() == DeviceFutureState::Idle);
  CHECK(fut.block_on().unwrap() == 15 && fut.state() == DeviceFutureState::Complete);
  // the op's error comes out of the first poll
  auto bad = Failing{}.schedule_on(s);
  auto br = bad.poll([] {});
  CHECK(br && br->is_err() && bad.state() == DeviceFutureState::Complete);
  // wait() = into_future().block_on() on the policy's stream
  CHECK(value(2).wait().unwrap() == 2);
  CHECK(cutile_execution_lock_held() == 0);
}

TEST(completion_goes_through_the_reactor_when_not_spun) {
  // CUTILE_ASYNC_SPIN_BUDGET_US=0 is set by main(): every future registers for a notification
  auto s = fresh_stream();
  uint64_t before = cutile_reactor_registrations();
  std::atomic<int> wakes{0};
  auto fut = value(1).schedule_on(s);
  auto first = fut.poll([&] { wakes.fetch_add(1); });
  CHECK(!first && fut.state() == DeviceFutureState::Executing);
  for (int i = 0; i < 2000 && wakes.load() == 0; ++i) std::this_thread::sleep_for(std::chrono::milliseconds(1));
  CHECK(wakes.load() == 1 && cutile_reactor_registrations() == before + 1);
  auto second = fut.poll([] {});
  CHECK(second && second->unwrap() == 1);
  // many in flight at once, from several threads
  std::vector<std::thread> ts;
  std::atomic<int> done{0};
  for (int t = 0; t < 4; ++t)
    ts.emplace_back([&] {
      auto st = Device::create(0).unwrap()->new_stream().unwrap();
      for (int i = 0; i < 200; ++i)
        if (value(i).schedule_on(st).block_on().unwrap() == i) done.fetch_add(1);
    });
  for (auto& t : ts) t.join();
  CHECK(done.load() == 800 && cutile_reactor_armed() == 0);
  // the raw registration API reports exhaustion instead of blocking: hold the stream in capture so flags never fire
  CHECK(cutile_stream_begin_capture(s->raw()) == CUTILE_SUCCESS);
  int ok_regs = 0, exhausted = 0;
  static std::atomic<int> fired{0};
  for (int i = 0; i < 1100; ++i) {
    cutile_status_t st = cutile_reactor_register(s->raw(), [](void*) { fired.fetch_add(1); }, nullptr);
    if (st == CUTILE_SUCCESS) ++ok_regs; else if (st == CUTILE_ERR_OUT_OF_SLOTS) ++exhausted;
  }
  CHECK(ok_regs == 1024 && exhausted == 76);
  // completion_register falls back to a host callback when the reactor is full (device_future.rs:142-153)
  CHECK(cutile_completion_register(s->raw(), [](void*) { fired.fetch_add(1000000); }, nullptr) == CUTILE_SUCCESS);
  cutile_graph_t g = nullptr;
  CHECK(cutile_stream_end_capture(s->raw(), &g) == CUTILE_SUCCESS);
  cutile_graph_exec_t ge = nullptr;
  CHECK(cutile_graph_instantiate(g, &ge) == CUTILE_SUCCESS && cutile_graph_launch(ge, s->raw()) == CUTILE_SUCCESS);
  for (int i = 0; i < 2000 && fired.load() < 1001024; ++i) std::this_thread::sleep_for(std::chrono::milliseconds(1));
  CHECK(fired.load() == 1001024 && cutile_reactor_armed() == 0);
}

TEST(bench_quantiles) {
  // cutile/src/bench.rs:266-291
  bench::Measurement r({4.0f, 1.0f, 3.0f, 2.0f});
  CHECK(r.min_ms() == 1.0f && r.median_ms() == 2.5f && r.quantile_ms(0.0f) == 1.0f && r.quantile_ms(1.0f) == 4.0f);
  CHECK(r.quantile_ms(-1.0f) == 1.0f && r.quantile_ms(2.0f) == 4.0f && std::fabs(r.mean_ms() - 2.5f) < 1e-6f);
  bench::Measurement one({7.0f});
  CHECK(one.median_ms() == 7.0f && one.quantile_ms(0.25f) == 7.0f);
  bench::Measurement out({1.0f, 1.0f, 1.0f, 1.0f, 100.0f});
  CHECK(out.median_ms() == 1.0f && out.mean_ms() > 20.0f);
  // do_bench on the recording runtime: warm-up at least once, reps within bounds, the closure sees the stream
  auto s = fresh_stream();
  int calls = 0;
  bench::BenchOptions o;
  o.warmup = std::chrono::milliseconds(0);
  o.rep = std::chrono::milliseconds(1);
  o.min_reps = 3;
  o.max_reps = 3;
  auto m = bench::do_bench(s, o, [&](const std::shared_ptr<Stream>& st) -> Result<Unit> { CHECK(st.get() == s.get()); ++calls; return ok(); }).unwrap();
  CHECK(m.reps() == 3 && calls == 1 + 1 + 3);
}

struct FakeOracle : tune::Oracle {  // cutile/src/tune.rs:1037-1069
  std::vector<tune::Config> cfgs;
  std::map<std::string, float> ms;
  std::vector<std::string> measured;
  size_t budget = SIZE_MAX;    // measurements allowed before the budget reads zero
  const std::vector<tune::Config>& configs() const override { return cfgs; }
  std::optional<std::chrono::nanoseconds> budget_remaining() const override {
    if (budget == SIZE_MAX) return std::nullopt;
    return std::chrono::nanoseconds(measured.size() >= budget ? 0 : 1000);
  }
  tune::Trial measure(size_t i) override {
    measured.push_back(cfgs[i].id);
    auto it = ms.find(cfgs[i].id);
    if (it == ms.end()) return tune::Trial::invalid(cfgs[i].id, "gate failed");
    return tune::Trial::ok(cfgs[i].id, it->second, it->second, 3);
  }
};

static tune::Config bn_splits(int64_t bn, int64_t splits) { return tune::Config::make({{"BN", bn}, {"SPLITS", splits}}); }

TEST(autotuner_search_semantics) {
  using tune::Config;
  // tune.rs:1072-1080, 1424-1435, 1635-1644: ids are stable, sorted by key, and cannot alias
  CHECK(Config::make({{"SPLITS", 8}, {"BN", 64}}).id == "BN=64,SPLITS=8" && bn_splits(64, 8).id == "BN=64,SPLITS=8");
  CHECK(*bn_splits(64, 8).integer("BN") == 64 && !bn_splits(64, 8).integer("missing"));
  CHECK(Config::make({{"A", 1}}).id != Config::make({{"A", "1"}}).id && Config::make({{"A", "1"}}).id == "A=\"1\"");
  CHECK(Config::make({{"x", "1,y=2"}}).id != Config::make({{"x", "1"}, {"y", 2}}).id);
  CHECK(Config::make({{"A=1,B", 2}}).id != Config::make({{"A", 1}, {"B", 2}}).id);
  CHECK(Config::make({{"\"A\"", 1}}).id != Config::make({{"A", 1}}).id);
  auto a = bn_splits(32, 2), b = bn_splits(64, 4), c = bn_splits(128, 8);
  CHECK(tune::space_hash({a, b, c}) == tune::space_hash({c, a, b}) && tune::space_hash({a, b}) != tune::space_hash({a, b, c}));
  // FNV-1a over the sorted ids, each closed by a zero byte: no ids -> the offset basis; "a" -> two rounds by hand
  CHECK(tune::space_hash({}) == "cbf29ce484222325");
  {
    uint64_t h = 0xcbf29ce484222325ull;
    h = (h ^ 'x') * 0x100000001b3ull;
    h = (h ^ '=') * 0x100000001b3ull;
    h = (h ^ '1') * 0x100000001b3ull;
    h = (h ^ 0) * 0x100000001b3ull;
    char buf[17];
    snprintf(buf, sizeof(buf), "%016llx", (unsigned long long)h);
    CHECK(tune::space_hash({Config::make({{"x", 1}})}) == buf);
  }
  // tune.rs:1082-1112: every candidate once, the best median wins, an invalid one is data and never wins
  FakeOracle o;
  o.cfgs = {a, b, c};
  o.ms = {{a.id, 32.0f}, {b.id, 64.0f}, {c.id, 128.0f}};
  auto trials = tune::GridSearch{}.search(o);
  CHECK(o.measured.size() == 3 && trials.size() == 3 && *tune::best_config(o.cfgs, trials)->integer("BN") == 32);
  FakeOracle inv;
  inv.cfgs = {a, b};
  inv.ms = {{b.id, 1.0f}};
  auto ti = tune::GridSearch{}.search(inv);
  CHECK(ti.size() == 2 && !ti[0].measured && ti[0].invalid_reason == "gate failed" && *tune::best_config(inv.cfgs, ti)->integer("BN") == 64);
  // tune.rs:1114-1136, 1437-1479: resume keeps measured known trials, retries invalid ones, drops stale configs
  FakeOracle o2;
  o2.cfgs = {a, b, c};
  o2.ms = {{a.id, 9.0f}, {b.id, 9.0f}, {c.id, 9.0f}};
  auto t2 = tune::GridSearch{}.resume({tune::Trial::ok(b.id, 0.5f, 0.5f, 3)}).search(o2);
  CHECK(o2.measured.size() == 2 && t2.size() == 3 && *tune::best_config(o2.cfgs, t2)->integer("BN") == 64);
  FakeOracle o4;
  o4.cfgs = {b};
  o4.ms = {{b.id, 1.0f}};
  auto t4 = tune::GridSearch{}.resume({tune::Trial::ok("BN=16,SPLITS=2", 0.1f, 0.1f, 3)}).search(o4);
  CHECK(t4.size() == 1 && *tune::best_config(o4.cfgs, t4)->integer("BN") == 64);
  FakeOracle o5;
  o5.cfgs = {b};
  o5.ms = {{b.id, 1.0f}};
  auto t5 = tune::GridSearch{}.resume({tune::Trial::invalid(b.id, "transient")}).search(o5);
  CHECK(o5.measured.size() == 1 && t5.size() == 1 && *t5[0].median() == 1.0f);
  // tune.rs:1138-1149: a zero budget measures nothing
  FakeOracle o3;
  o3.cfgs = {a, b, c};
  o3.ms = o2.ms;
  o3.budget = 0;
  CHECK(tune::GridSearch{}.search(o3).empty());
  // tune.rs:1500-1522: NaN never wins
  CHECK(*tune::best_config({b, c}, {tune::Trial::ok(b.id, NAN, NAN, 3), tune::Trial::ok(c.id, 2.0f, 2.0f, 3)})->integer("BN") == 128);
  // tune.rs:1481-1498: prune composes with configs in either order
  auto keep = [](const Config& cfg) { return *cfg.integer("BN") != 32; };
  CHECK(tune::Autotuner("t").prune(keep).configs({a, b}).pruned_configs().size() == 1);
  CHECK(tune::Autotuner("t").configs({a, b}).prune(keep).pruned_configs()[0].id == b.id);
}

TEST(autotuner_runoff_verdicts) {   // tune.rs:1533-1632
  auto a = bn_splits(32, 2), b = bn_splits(64, 4);
  auto silent = tune::TrialLog::open(std::nullopt, "t", "s").unwrap();
  auto meas = [](std::vector<float> t) { return bench::Measurement(std::move(t)); };
  for (bool b_failed : {false, true}) {
    std::vector<tune::Trial> trials;
    tune::RunoffError err{b_failed ? tune::RunoffError::Kind::SetupB : tune::RunoffError::Kind::SetupA, DeviceError::tensor("boom")};
    auto winner = tune::runoff_verdict(a, b, err, &trials, &silent);
    CHECK(winner.id == (b_failed ? a.id : b.id) && trials.size() == 1 && trials[0].config_id == (b_failed ? b.id : a.id));
    CHECK(!trials[0].measured && trials[0].invalid_reason.find("runoff setup failed") != std::string::npos);
  }
  std::vector<tune::Trial> none;
  CHECK(tune::runoff_verdict(a, b, tune::RunoffError{tune::RunoffError::Kind::Bench, DeviceError::tensor("stream died")}, &none, &silent).id == a.id && none.empty());
  std::vector<tune::Trial> scratch;
  CHECK(tune::runoff_verdict(a, b, std::make_pair(meas({2.0f, 2.0f, 2.0f}), meas({NAN, NAN})), &scratch, &silent).id == a.id);
  CHECK(tune::runoff_verdict(a, b, std::make_pair(meas({NAN}), meas({3.0f})), &scratch, &silent).id == b.id);
  std::vector<tune::Trial> real;
  CHECK(tune::runoff_verdict(a, b, std::make_pair(meas({1.0f, 2.0f, 3.0f}), meas({4.0f, 5.0f, 6.0f})), &real, &silent).id == a.id);
  CHECK(real.size() == 2 && real[0].measured && real[0].median_ms == 2.0f && real[0].min_ms == 1.0f && real[0].reps == 3);
}

TEST(trial_log_roundtrips_resumes_and_refuses_foreign_logs) {   // tune.rs:1364-1421, 1646-1663
  std::string path = "/tmp/cutile_tune_log_" + std::to_string(getpid());
  remove(path.c_str());
  {
    auto log = tune::TrialLog::open(path, "t", "s").unwrap();
    log.append(tune::Trial::ok("BN=64", 1.5f, 1.4f, 5));
    log.append(tune::Trial::invalid("BN=128", "launch check"));
  }
  {
    std::ifstream in(path);
    std::string l1, l2, l3;
    std::getline(in, l1); std::getline(in, l2); std::getline(in, l3);
    CHECK(l1 == "{\"log_schema\":1,\"tuner\":\"t\",\"space\":\"s\"}");
    CHECK(l2 == "{\"config_id\":\"BN=64\",\"state\":{\"Measured\":{\"median_ms\":1.5,\"min_ms\":1.4,\"reps\":5}}}");
    CHECK(l3 == "{\"config_id\":\"BN=128\",\"state\":{\"Invalid\":{\"reason\":\"launch check\"}}}");
  }
  auto again = tune::TrialLog::open(path, "t", "s").unwrap();
  CHECK(again.existing_trials().size() == 2 && *again.existing_trials()[0].median() == 1.5f && !again.existing_trials()[1].median());
  CHECK(tune::TrialLog::open(path, "other", "s").error().message.find("belongs to tuner") != std::string::npos);
  CHECK(tune::TrialLog::open(path, "t", "different").error().message.find("belongs to tuner") != std::string::npos);
  { std::ofstream torn(path, std::ios::app); torn << "{\"config_id\":\"torn"; }      // a crash mid-write
  { auto log = tune::TrialLog::open(path, "t", "s").unwrap(); log.append(tune::Trial::ok("BN=256", 2.0f, 2.0f, 3)); }
  CHECK(tune::TrialLog::open(path, "t", "s").unwrap().existing_trials().size() == 3);   // torn line dropped, new record intact
  { std::ofstream junk(path, std::ios::trunc); junk << "not json\n"; }
  CHECK(tune::TrialLog::open(path, "t", "s").error().message.find("no valid header") != std::string::npos);
  { std::ofstream ws(path, std::ios::trunc); ws << "\n"; }                               // whitespace only: fresh
  { auto log = tune::TrialLog::open(path, "t", "s").unwrap(); log.append(tune::Trial::invalid("BN=1,SPLITS=1", "x")); }
  CHECK(tune::TrialLog::open(path, "t", "s").unwrap().existing_trials().size() == 1);
  remove(path.c_str());
}

TEST(json_reader_refuses_deep_nesting_and_malformed_numbers) {
  CHECK(json::parse("{\"a\": [1, 2.5, -3e2, {\"b\": null}]}").has_value());
  CHECK(json::parse("[1, 2.5e-3, -0.5, 10]")->items[1].as_double() == 2.5e-3);
  for (const char* bad : {"1-2", "--", "-", "1e", "1.2.3", "[1, 2-]", "{\"a\": +1}", "1e+", "12.", "99999999999999999999"})
    CHECK(!json::parse(bad).has_value());
  std::string deep(100000, '[');      // would recurse 100000 frames without the cap
  CHECK(!json::parse(deep).has_value());
  std::string ok_depth = std::string(60, '[') + "1" + std::string(60, ']');
  CHECK(json::parse(ok_depth).has_value());
  std::string too_deep = std::string(70, '[') + "1" + std::string(70, ']');
  CHECK(!json::parse(too_deep).has_value());
}

TEST(tuning_records_roundtrip_and_refuse_stale_provenance) {   // tune.rs:1151-1362
  using tune::Record;
  using tune::RecordEntry;
  auto ws = [] { return tune::Workspace{"fmha_decode", "abc123", "sm_120", "release 13.3, V13.3.36", std::nullopt}; };
  std::string path = "/tmp/cutile_record_" + std::to_string(getpid()) + ".json";
  auto decline = [](const RecordEntry&) -> Result<std::optional<std::string>> { return std::optional<std::string>(); };
  auto err_of = [&](const tune::Workspace& w, const Record::VerifyKey& v) { return Record::load_verified(path, w, v).error().message; };
  {
    Record a(ws());
    a.cutile_version = cutile_library_version();
    a.insert({"tg<=512", bn_splits(64, 8), 1.25f, 12, std::string(64, 'f')});
    CHECK(a.save(path).is_ok());
    auto [loaded, warnings] = Record::load_verified(path, ws(), [](const RecordEntry& e) -> Result<std::optional<std::string>> { return e.l2_key; }).unwrap();
    CHECK(warnings.empty() && *loaded.get("tg<=512")->config.integer("BN") == 64 && loaded.get("tg<=512")->samples == 12 && loaded.get("tg<=512")->median_ms == 1.25f);
    // recomputed key differs => refused; toolchain drift => the verifier is not even consulted, one warning
    CHECK(err_of(ws(), [](const RecordEntry&) -> Result<std::optional<std::string>> { return std::optional<std::string>(std::string(64, 'b')); })
              .find("l2 key for bucket") != std::string::npos);
    auto drifted = ws();
    drifted.tileiras_fingerprint = "release 13.4, V13.4.1";
    bool called = false;
    auto [rec2, warn2] = Record::load_verified(path, drifted, [&](const RecordEntry&) -> Result<std::optional<std::string>> {
      called = true;
      return std::optional<std::string>(std::string(64, 'b'));
    }).unwrap();
    CHECK(!called && warn2.size() == 1 && warn2[0].find("different tileiras") != std::string::npos && warn2[0].find("skipped") != std::string::npos);
  }
  {
    CHECK(Record(ws()).save(path).is_ok());
    auto other = ws(); other.source_hash = "different";
    CHECK(err_of(other, decline).find("source_hash mismatch") != std::string::npos && err_of(other, decline).find("re-tune") != std::string::npos);
    other = ws(); other.arch = "sm_100";
    CHECK(err_of(other, decline).find("arch mismatch") != std::string::npos);
    other = ws(); other.kernel = "other_kernel";
    CHECK(err_of(other, decline).find("kernel mismatch") != std::string::npos);
    // a record without space_hash where the workspace has one: a warning
    auto expecting = ws(); expecting.space_hash = tune::space_hash({bn_splits(64, 8)});
    auto [r3, w3] = Record::load_verified(path, expecting, decline).unwrap();
    CHECK(w3.size() == 1 && w3[0].find("no space_hash") != std::string::npos);
  }
  {
    auto with_space = ws(); with_space.space_hash = tune::space_hash({bn_splits(64, 8), bn_splits(128, 8)});
    CHECK(Record(with_space).save(path).is_ok());
    auto other = ws(); other.space_hash = tune::space_hash({bn_splits(64, 8)});
    CHECK(err_of(other, decline).find("space_hash mismatch") != std::string::npos);
    CHECK(Record::load_verified(path, ws(), decline).is_ok());       // loader without an expectation: accepted
    Record dup(ws());
    for (int i = 0; i < 2; ++i) dup.entries.push_back({"b", bn_splits(64, 8), 1.0f, 3, std::nullopt});
    CHECK(dup.save(path).is_ok());
    CHECK(err_of(ws(), decline).find("duplicate entries for bucket") != std::string::npos);
  }
  {
    Record a(ws());
    for (auto [bn, ms] : {std::make_pair(64, 2.0f), std::make_pair(128, 1.0f)}) a.insert({"b", bn_splits(bn, 4), ms, 3, std::nullopt});
    CHECK(a.entries.size() == 1 && *a.get("b")->config.integer("BN") == 128);     // one winner per bucket
    Record s(ws());
    s.schema = tune::kRecordSchema + 1;
    CHECK(s.save(path).is_ok());
    CHECK(err_of(ws(), decline).find("schema mismatch") != std::string::npos);
    Record edited(ws());
    auto config = bn_splits(64, 8);
    config.id = "BN=128,SPLITS=8";                                              // hand-edited: id and params disagree
    edited.insert({"b", config, 1.0f, 3, std::nullopt});
    CHECK(edited.save(path).is_ok());
    CHECK(err_of(ws(), decline).find("config id for bucket") != std::string::npos);
    Record old(ws());
    old.cutile_version = "0.0.0-elsewhere";
    CHECK(old.save(path).is_ok());
    auto [r5, w5] = Record::load_verified(path, ws(), decline).unwrap();
    CHECK(w5.size() == 1 && w5[0].find("produced by cutile 0.0.0-elsewhere") != std::string::npos);
  }
  // this build's provenance: fingerprints come from the kernel table
  auto live = tune::Workspace::of_kernel("gemm").unwrap();
  CHECK(live.arch == "gfx950" && live.source_hash.size() == 16 && !live.tileiras_fingerprint.empty());
  auto k1 = tune::variant_key("gemm", "bf16_256x256x64_d4x2").unwrap(), k2 = tune::variant_key("gemm", "bf16_256x256x64_d2x4").unwrap();
  CHECK(k1 && k2 && *k1 != *k2 && *k1 != live.source_hash);
  CHECK(tune::variant_key("gemm", "no_such_variant").is_err() && tune::Workspace::of_kernel("no_such_kernel").is_err());
  CHECK(tune::Workspace::of_kernel("rms_norm_f16").unwrap().source_hash != live.source_hash);   // another code object
  remove(path.c_str());
}

TEST(autotuner_end_to_end_on_the_recording_runtime) {
  using tune::Config;
  auto a = Config::make({{"bm", 128}, {"bn", 128}}), b = Config::make({{"bm", 256}, {"bn", 256}}), c = Config::make({{"bm", 64}, {"bn", 64}});
  // candidates that fail to set up are recorded as invalid; the log makes the second run resume
  auto s = fresh_stream();
  bench::BenchOptions bo;
  bo.warmup = std::chrono::milliseconds(0);
  bo.rep = std::chrono::milliseconds(1);
  bo.min_reps = 2;
  bo.max_reps = 2;
  bo.clear_l2 = false;
  std::string log = "/tmp/cutile_tune_test_" + std::to_string(getpid()) + ".jsonl";
  remove(log.c_str());
  int setups = 0;
  auto run = [&] {
    return tune::Autotuner("unit").configs({a, b, c}).bench_options(bo).log(log)
        .prune([](const Config& cfg) { return *cfg.integer("bm") >= 128; })
        .run(s, [&](const std::shared_ptr<Stream>&, const Config& cfg) -> Result<bench::BenchFn> {
          ++setups;
          if (*cfg.integer("bm") == 256) return DeviceError::launch("tile too large");
          return bench::BenchFn([](const std::shared_ptr<Stream>&) { return ok(); });
        }).unwrap();
  };
  auto out = run();
  CHECK(out.best && out.best->id == a.id && out.trials.size() == 2 && setups == 2);   // one measurable candidate: no runoff
  auto out2 = run();  // resumed from the log: the measured candidate is not measured again, the invalid one is retried
  CHECK(out2.best->id == a.id && setups == 3);
  // the same log under another candidate set is refused, not overwritten
  auto foreign = tune::Autotuner("unit").configs({a}).bench_options(bo).log(log)
                     .run(s, [&](const std::shared_ptr<Stream>&, const Config&) -> Result<bench::BenchFn> { return DeviceError::launch("unused"); });
  CHECK(foreign.is_err() && foreign.error().message.find("belongs to tuner") != std::string::npos);
  remove(log.c_str());
  auto variants = tune::variant_configs("gemm", "256x256");
  CHECK(variants.size() >= 3 && variants[0].id.rfind("variant=\"", 0) == 0);
}

int main(int argc, char** argv) {
  setenv("CUTILE_ASYNC_SPIN_BUDGET_US", "0", 1);
  if (cutile_testing_use_fake_hip(1) != CUTILE_SUCCESS) return 2;
  return run_all_tests(argc, argv);
}
