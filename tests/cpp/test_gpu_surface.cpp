// GPU tests of the C++ host surface: the reference's runnable examples, end to end
// through Tensor / Partition / DeviceOp / graph / future on a real MI355X, with
// the known answers those examples assert (cutile-examples/examples/saxpy.rs:47-53,
// softmax.rs:55-60, mxfp8.rs:129-135, cuda_graphs.rs:333-344,
// cutile/tests/gpu/add_basic.rs:29-43, cutile/tests/slice_non_divisible.rs:459-500).
#include <unistd.h>
#include <cutile/cutile.hpp>

#include <atomic>
#include <cmath>
#include <thread>

#include "check.hpp"

using namespace cutile;

static std::shared_ptr<Stream> new_stream() { return Device::create(0).unwrap()->new_stream().unwrap(); }

TEST(device_is_gfx950) {
  auto dev = Device::create(0).unwrap();
  CHECK(dev->arch().unwrap().find("gfx950") != std::string::npos);
  CHECK(dev->props().unwrap().wavefront_size == 64 && dev->l2_cache_size_bytes().unwrap() > 0);
  CHECK(Device::device_count().unwrap() >= 1 && dev->name().is_ok());
}

TEST(saxpy_example) {
  auto stream = new_stream();
  auto input = std::make_shared<Tensor<float>>(api::arange<float>(32).sync_on(stream).unwrap());
  auto x = std::make_shared<Tensor<float>>(std::move(api::dup(*input).sync_on(stream).unwrap()).reshape({4, 8}).unwrap());
  auto y = std::move(api::dup(*input).sync_on(stream).unwrap()).reshape({4, 8}).unwrap().partition({2, 2});
  auto y_host = api::to_host_vec_op(unpartition_op(saxpy(std::move(y), 2.0f, x).first())).sync_on(stream).unwrap();
  auto in_host = api::to_host_vec(input).sync_on(stream).unwrap();
  for (size_t i = 0; i < in_host.size(); ++i) CHECK(y_host[i] == 2.0f * in_host[i] + in_host[i]);
}

TEST(add_with_lazy_arguments) {
  auto z = add(partition_op(api::zeros<float>({256}), {64}), api::ones<float>({256}), api::ones<float>({256}));
  auto host = api::to_host_vec_op(unpartition_op(std::move(z).first())).sync().unwrap();  // default policy stream
  for (float v : host) CHECK(v == 2.0f);
}

TEST(softmax_example_rows_sum_to_one) {
  auto stream = new_stream();
  auto x = std::make_shared<Tensor<float>>(reshape_op(api::arange<float>(32), {4, 8}).sync_on(stream).unwrap());
  auto y = partition_op(api::zeros<float>({4, 8}), {2, 8});
  auto [xo, yo] = softmax(x, std::move(y)).sync_on(stream).unwrap();
  auto host = api::to_host_vec(std::move(yo).unpartition()).sync_on(stream).unwrap();
  for (int r = 0; r < 4; ++r) {
    float sum = 0;
    for (int c = 0; c < 8; ++c) sum += host[r * 8 + c];
    CHECK(std::fabs(sum - 1.0f) < 1e-4f);
  }
  CHECK(xo.get() == x.get());
}

TEST(rms_norm_constant_rows) {
  auto stream = new_stream();
  auto x = api::full<f16>(3.0, {16, 1024}).sync_on(stream).unwrap();
  auto w = api::full<f16>(0.5, {1024}).sync_on(stream).unwrap();
  auto out = api::zeros<f16>({16, 1024}).sync_on(stream).unwrap();
  CHECK(rms_norm_f16(&x, &w, out.partition_mut({1, 1024}), 0.0f).generics({"1024", "512"}).sync_on(stream).is_ok());
  for (f16 v : api::to_host_vec(out).sync_on(stream).unwrap()) CHECK(f32_from_f16(v) == 0.5f);  // x == c -> out = w
}

TEST(all_f16_benchmark_forms_closed_forms) {
  // Constant rows make the f16 chain checkable by hand (values from exact rational arithmetic rounded step by step,
  // tests/test_oracle.py): x = 1.7 (f16 1.7002), w = 0.5, N = 2048, BLOCK_SIZE 512 gives 0x37FF (0.49976) with the
  // square root rounded toward minus infinity and 0x3800 (0.5) with it rounded to nearest; x = 6 overflows the f16
  // sum of squares (36 * 2048 > 65504): inf -> 1 / inf = 0 -> every output is 0.
  auto stream = new_stream();
  auto w = api::full<f16>(0.5, {2048}).sync_on(stream).unwrap();
  auto out = api::zeros<f16>({16, 2048}).sync_on(stream).unwrap();
  auto x = api::full<f16>(1.7, {16, 2048}).sync_on(stream).unwrap();
  CHECK(rms_norm_all_f16(&x, &w, out.partition_mut({1, 2048}), 1e-5f).generics({"2048", "512"}).sync_on(stream).is_ok());
  for (f16 v : api::to_host_vec(out).sync_on(stream).unwrap()) CHECK(v.bits == 0x37FF);
  auto big = api::full<f16>(6.0, {16, 2048}).sync_on(stream).unwrap();
  CHECK(rms_norm_all_f16(&big, &w, out.partition_mut({1, 2048}), 1e-5f).generics({"2048", "512"}).sync_on(stream).is_ok());
  for (f16 v : api::to_host_vec(out).sync_on(stream).unwrap()) CHECK(v.bits == 0);
  // BLOCK_SIZE is part of the arithmetic: leaving it out is an error, not a default
  CHECK(rms_norm_all_f16(&x, &w, out.partition_mut({1, 2048}), 1e-5f).sync_on(stream).is_err());
  // softmax of a constant row: exp(0) = 1, the tree of ones is exact, every output is 1 / BN
  auto y = api::zeros<f16>({16, 2048}).sync_on(stream).unwrap();
  CHECK(softmax_all_f16(&x, y.partition_mut({1, 512})).sync_on(stream).is_ok());
  for (f16 v : api::to_host_vec(y).sync_on(stream).unwrap()) CHECK(f32_from_f16(v) == 1.0f / 512.0f);
}

TEST(transformer_block_kernels_closed_forms) {
  auto stream = new_stream();
  // add_rms_norm: residual = 1, x = 2 -> combined = 3 everywhere; out = w, residual_out = 3
  auto res = api::full<f16>(1.0, {8, 512}).sync_on(stream).unwrap();
  auto x = api::full<f16>(2.0, {8, 512}).sync_on(stream).unwrap();
  auto w = api::full<f16>(0.25, {512}).sync_on(stream).unwrap();
  auto out = api::zeros<f16>({8, 512}).sync_on(stream).unwrap();
  auto res_out = api::zeros<f16>({8, 512}).sync_on(stream).unwrap();
  CHECK(add_rms_norm_f16(&res, &x, &w, out.partition_mut({1, 512}), res_out.partition_mut({1, 512}), 0.0f).sync_on(stream).is_ok());
  for (f16 v : api::to_host_vec(out).sync_on(stream).unwrap()) CHECK(f32_from_f16(v) == 0.25f);
  for (f16 v : api::to_host_vec(res_out).sync_on(stream).unwrap()) CHECK(f32_from_f16(v) == 3.0f);
  // qk_norm: q rows take q_weight, k rows k_weight
  auto q = api::full<f16>(-2.0, {6, 128}).sync_on(stream).unwrap();
  auto k = api::full<f16>(5.0, {2, 128}).sync_on(stream).unwrap();
  auto qw = api::full<f16>(1.0, {128}).sync_on(stream).unwrap();
  auto kw = api::full<f16>(2.0, {128}).sync_on(stream).unwrap();
  auto qk = api::zeros<f16>({8, 128}).sync_on(stream).unwrap();
  CHECK(qk_norm_f16(&q, &k, &qw, &kw, qk.partition_mut({1, 128}), 0.0f, 6).sync_on(stream).is_ok());
  auto qk_host = api::to_host_vec(qk).sync_on(stream).unwrap();
  for (int i = 0; i < 8 * 128; ++i) CHECK(f32_from_f16(qk_host[i]) == (i < 6 * 128 ? -1.0f : 2.0f));
  // silu_mul: gate = 0 -> 0; add_2d: 2 + 2 = 4
  auto gate = api::zeros<f16>({4, 256}).sync_on(stream).unwrap();
  auto act = api::full<f16>(7.0, {4, 256}).sync_on(stream).unwrap();
  auto up = api::full<f16>(2.0, {4, 256}).sync_on(stream).unwrap();
  CHECK(silu_mul_2d_f16(act.partition_mut({1, 64}), &gate, &up).sync_on(stream).is_ok());
  for (f16 v : api::to_host_vec(act).sync_on(stream).unwrap()) CHECK(f32_from_f16(v) == 0.0f);
  CHECK(add_2d_f16(act.partition_mut({1, 64}), &up, &up).generics({"64"}).sync_on(stream).is_ok());
  for (f16 v : api::to_host_vec(act).sync_on(stream).unwrap()) CHECK(f32_from_f16(v) == 4.0f);
  // rope at position 0 is the identity, whichever way the position arrives
  auto ramp = std::make_shared<Tensor<float>>(api::arange<float>(3 * 2 * 16).sync_on(stream).unwrap());
  auto xr = reshape_op(api::convert<f16>(ramp), {3, 2, 16}).sync_on(stream).unwrap();
  auto inv_freq = api::full<float>(0.5, {8}).sync_on(stream).unwrap();
  auto rot = api::zeros<f16>({1, 2, 16}).sync_on(stream).unwrap();
  CHECK(rope_seq_f16(&xr, &inv_freq, rot.partition_mut({1, 1, 8}), 0).sync_on(stream).is_ok());
  auto rot_host = api::to_host_vec(rot).sync_on(stream).unwrap();
  for (int i = 0; i < 32; ++i) CHECK(f32_from_f16(rot_host[i]) == (float)i);
  auto pos = api::zeros<uint32_t>({1}).sync_on(stream).unwrap();
  CHECK(rope_seq_dynpos_f16(&xr, &inv_freq, &pos, rot.partition_mut({1, 1, 8})).sync_on(stream).is_ok());
  CHECK(qk_rope_dynpos_f16(&xr, &xr, &inv_freq, &pos, rot.partition_mut({1, 1, 8}), 1).sync_on(stream).is_ok());
  rot_host = api::to_host_vec(rot).sync_on(stream).unwrap();
  for (int i = 0; i < 16; ++i) CHECK(f32_from_f16(rot_host[16 + i]) == (float)i);   // head 1 of out = head 0 of k
}

TEST(decode_kernels_closed_forms) {
  auto stream = new_stream();
  const int heads = 4, group = 4, d = 128, max_seq = 256, splits = 4;
  // cache update: three new rows of 3.0 land at positions 9..11 of a cache of 1.0
  auto new_k = api::full<f16>(3.0, {3, heads, d}).sync_on(stream).unwrap();
  auto new_v = api::full<f16>(-3.0, {3, heads, d}).sync_on(stream).unwrap();
  auto k_cache = api::full<f16>(1.0, {heads, max_seq, d}).sync_on(stream).unwrap();
  auto v_cache = api::full<f16>(1.0, {heads, max_seq, d}).sync_on(stream).unwrap();
  auto pos = api::full<uint32_t>(9, {1}).sync_on(stream).unwrap();
  CHECK(kv_cache_update_seq_dynpos_f16(&new_k, &new_v, k_cache.partition_mut({1, max_seq, d}), v_cache.partition_mut({1, max_seq, d}), &pos, 3)
            .generics({"128", "128", "256"}).sync_on(stream).is_ok());
  auto kh = api::to_host_vec(k_cache).sync_on(stream).unwrap();
  auto vh = api::to_host_vec(v_cache).sync_on(stream).unwrap();
  for (int h = 0; h < heads; ++h)
    for (int r = 0; r < max_seq; ++r) {
      const bool fresh = r >= 9 && r < 12;
      CHECK(f32_from_f16(kh[((size_t)h * max_seq + r) * d + 5]) == (fresh ? 3.0f : 1.0f));
      CHECK(f32_from_f16(vh[((size_t)h * max_seq + r) * d + 77]) == (fresh ? -3.0f : 1.0f));
    }
  // the prefill form writes rows 0..seq_len and refuses another offset
  CHECK(kv_cache_update_seq_f16(&new_k, &new_v, k_cache.partition_mut({1, 16, 64}), v_cache.partition_mut({1, 16, 64}), 0, 2).sync_on(stream).is_ok());
  CHECK(!kv_cache_update_seq_f16(&new_k, &new_v, k_cache.partition_mut({1, 16, 64}), v_cache.partition_mut({1, 16, 64}), 5, 2).sync_on(stream).is_ok());
  kh = api::to_host_vec(k_cache).sync_on(stream).unwrap();
  CHECK(f32_from_f16(kh[0]) == 3.0f && f32_from_f16(kh[d]) == 3.0f && f32_from_f16(kh[2 * d]) == 1.0f);
  // decode: every value row is 2.0 -> softmax weights sum to one -> every output is 2.0, whatever the scores
  auto q = api::full<f16>(0.5, {heads, group, d}).sync_on(stream).unwrap();
  auto vals = api::full<f16>(2.0, {heads, max_seq, d}).sync_on(stream).unwrap();
  auto att = api::zeros<f16>({heads, splits * group, d}).sync_on(stream).unwrap();
  auto lse = api::zeros<float>({heads, splits * group}).sync_on(stream).unwrap();
  auto out = api::zeros<f16>({heads, group, d}).sync_on(stream).unwrap();
  auto at = api::full<uint32_t>(199, {1}).sync_on(stream).unwrap();
  CHECK(fmha_decode_gqa_split(&q, &k_cache, &vals, att.partition_mut({1, group, d}), lse.partition_mut({1, group}), 0.0884f, &at)
            .generics({"4", "64", "128", "4"}).sync_on(stream).is_ok());
  CHECK(splitk_reduce_merge(&att, &lse, out.partition_mut({1, group, d})).sync_on(stream).is_ok());
  for (f16 v : api::to_host_vec(out).sync_on(stream).unwrap()) CHECK(f32_from_f16(v) == 2.0f);
  // GROUP = 3 has no precompiled variant: an error that names what exists, not a wrong answer
  auto q3 = api::zeros<f16>({heads, 3, d}).sync_on(stream).unwrap();
  auto att3 = api::zeros<f16>({heads, 3, d}).sync_on(stream).unwrap();
  auto lse3 = api::zeros<float>({heads, 3}).sync_on(stream).unwrap();
  auto r = fmha_decode_gqa_split(&q3, &k_cache, &vals, att3.partition_mut({1, 3, d}), lse3.partition_mut({1, 3}), 0.1f, &at).sync_on(stream);
  CHECK(!r.is_ok());
}

TEST(sequence_attention_launchers_closed_forms) {
  // every value row is 2.0: the weights sum to one, so each of the five kernels returns 2.0 whatever the scores;
  // with no key in range (kv_len = 0) the production kernels return zeros
  auto stream = new_stream();
  const int q_len = 40, q_heads = 8, kv_heads = 2, d = 128, max_seq = 96, group = q_heads / kv_heads;
  auto q = api::full<f16>(0.25, {q_len, q_heads, d}).sync_on(stream).unwrap();
  auto k = api::full<f16>(0.5, {kv_heads, max_seq, d}).sync_on(stream).unwrap();
  auto v = api::full<f16>(2.0, {kv_heads, max_seq, d}).sync_on(stream).unwrap();
  auto pos = api::full<uint32_t>(50, {1}).sync_on(stream).unwrap();
  auto all_equal = [&](Tensor<f16>& t, float want) {
    for (f16 x : api::to_host_vec(t).sync_on(stream).unwrap())
      if (f32_from_f16(x) != want) return false;
    return true;
  };
  auto out = api::zeros<f16>({q_len, q_heads, d}).sync_on(stream).unwrap();
  {
    auto [q_, k_, v_, o_, scale, g, kv_len, start] =
        flash_attn_causal_seq_f16(&q, &k, &v, out.partition_mut({16, 1, d}), 0.0884f, group, 90, 50).generics({"16", "32", "128"}).sync_on(stream).unwrap();
    CHECK(g == group && kv_len == 90 && start == 50 && scale == 0.0884f);      // arguments come back in signature order
  }
  CHECK(all_equal(out, 2.0f));
  CHECK(fmha_prefill_causal<false>(&q, &k, &v, out.partition_mut({16, 1, d}), 0.0884f, group, 0, 0).sync_on(stream).is_ok());
  CHECK(all_equal(out, 0.0f));
  CHECK(fmha_prefill_gqa(&q, &k, &v, out.partition_mut({8, group, d}), 0.0884f, group, 96, 56).sync_on(stream).is_ok());
  CHECK(all_equal(out, 2.0f));
  auto q1 = api::full<f16>(0.25, {1, q_heads, d}).sync_on(stream).unwrap();
  auto o1 = api::zeros<f16>({1, q_heads, d}).sync_on(stream).unwrap();
  CHECK(flash_attn_causal_seq_dynpos_f16(&q1, &k, &v, o1.partition_mut({1, 1, d}), 0.0884f, group, &pos).sync_on(stream).is_ok());
  CHECK(all_equal(o1, 2.0f));
  CHECK(api::full<f16>(0.0, {1, q_heads, d}).sync_on(stream).is_ok());
  CHECK(fmha_causal(&q1, &k, &v, o1.partition_mut({1, 1, d}), 0.0884f, group, &pos).sync_on(stream).is_ok());
  CHECK(all_equal(o1, 2.0f));
  // the heads must group as the tensors say; nothing is launched otherwise
  CHECK(!fmha_prefill_causal(&q, &k, &v, out.partition_mut({16, 1, d}), 0.0884f, 2, 96, 0).sync_on(stream).is_ok());
}

TEST(greedy_sampling_and_gathers_closed_forms) {
  // logits = arange: the largest valid index wins; constant weights and hidden: every logit is K / 2, the first row wins
  auto stream = new_stream();
  const int n = 2000, nb = 2;                          // f16 holds every integer up to 2048
  auto logits = api::arange<f16>(n).sync_on(stream).unwrap();
  auto bm = api::zeros<float>({nb}).sync_on(stream).unwrap();
  auto bi = api::zeros<uint32_t>({nb}).sync_on(stream).unwrap();
  auto tok = api::zeros<uint32_t>({1}).sync_on(stream).unwrap();
  CHECK(argmax_blocks_f16(&logits, bm.partition_mut({1}), bi.partition_mut({1}), 1500).generics({"1024"}).sync_on(stream).is_ok());
  CHECK(argmax_reduce_blocks_to_u32(&bm, &bi, tok.partition_mut({1}), nb).sync_on(stream).is_ok());
  auto bih = api::to_host_vec(bi).sync_on(stream).unwrap();
  auto bmh = api::to_host_vec(bm).sync_on(stream).unwrap();
  CHECK(bih[0] == 1023 && bih[1] == 1499 && bmh[0] == 1023.0f && bmh[1] == 1499.0f);
  CHECK(api::to_host_vec(tok).sync_on(stream).unwrap()[0] == 1499);
  const int vocab = 256, k = 64;
  auto table = api::full<f16>(0.5, {vocab, k}).sync_on(stream).unwrap();
  auto hidden = api::full<f16>(1.0, {1, k}).sync_on(stream).unwrap();
  auto bm2 = api::zeros<float>({4}).sync_on(stream).unwrap();
  auto bi2 = api::zeros<uint32_t>({4}).sync_on(stream).unwrap();
  CHECK(lm_head_argmax_blocks_f16(&table, &hidden, bm2.partition_mut({1}), bi2.partition_mut({1}), 200).generics({"64"}).sync_on(stream).is_ok());
  auto bm2h = api::to_host_vec(bm2).sync_on(stream).unwrap();
  auto bi2h = api::to_host_vec(bi2).sync_on(stream).unwrap();
  for (int b = 0; b < 3; ++b) CHECK(bm2h[b] == 32.0f && bi2h[b] == (uint32_t)(b * 64));     // all equal: the first row of the block
  CHECK(bm2h[3] == 32.0f && bi2h[3] == 192);                                              // rows 192 .. 199 are valid
  // embedding rows and a gathered row are copies
  auto ids = api::full<uint32_t>(7, {5}).sync_on(stream).unwrap();
  auto emb = api::zeros<f16>({5, k}).sync_on(stream).unwrap();
  CHECK(embedding_batch_f16(&ids, &table, emb.partition_mut({1, 32})).generics({"64", "32"}).sync_on(stream).is_ok());
  for (f16 x : api::to_host_vec(emb).sync_on(stream).unwrap()) CHECK(f32_from_f16(x) == 0.5f);
  auto row = api::zeros<f16>({k}).sync_on(stream).unwrap();
  CHECK(gather_row_f16(&table, row.partition_mut({16}), 3).sync_on(stream).is_ok());
  for (f16 x : api::to_host_vec(row).sync_on(stream).unwrap()) CHECK(f32_from_f16(x) == 0.5f);
  CHECK(!gather_row_f16(&table, row.partition_mut({16}), -1).sync_on(stream).is_ok());
}

TEST(persistent_gemm_example) {
  // cutile-examples/examples/persistent_gemm.rs:61-126 as written: f32, 16x16x8 tiles, M = N = 64, K = 32, map [4, 1], 4 tile blocks
  auto stream = new_stream();
  const int M = 64, N = 64, K = 32;
  auto xh = std::make_shared<std::vector<float>>(M * K), yh = std::make_shared<std::vector<float>>(K * N);
  for (int r = 0; r < M; ++r)
    for (int c = 0; c < K; ++c) (*xh)[r * K + c] = ((float)(r % 7) - 3.0f) * 0.25f + (float)(c % 5) * 0.125f;
  for (int r = 0; r < K; ++r)
    for (int c = 0; c < N; ++c) (*yh)[r * N + c] = ((float)(r % 3) + 1.0f) * 0.2f - (float)(c % 11) * 0.05f;
  auto z = api::full<float>(-333.25, {M, N}).sync_on(stream).unwrap().partition({16, 16}).map({4, 1}, 4);
  auto x = std::make_shared<Tensor<float>>(reshape_op(api::copy_host_vec_to_device(xh), {M, K}).sync_on(stream).unwrap());
  auto y = std::make_shared<Tensor<float>>(reshape_op(api::copy_host_vec_to_device(yh), {K, N}).sync_on(stream).unwrap());
  auto [zp, x_, y_] = gemm_persistent(std::move(z), x, y).generics({"f32", "16", "16", "8", "4", "1"}).sync_on(stream).unwrap();
  auto zh = api::to_host_vec(std::move(zp).unpartition()).sync_on(stream).unwrap();
  float max_err = 0.0f;
  for (int i = 0; i < M; ++i)
    for (int j = 0; j < N; ++j) {
      float ref = 0.0f;
      for (int t = 0; t < K; ++t) ref += (*xh)[i * K + t] * (*yh)[t * N + j];   // cpu_gemm, persistent_gemm.rs:140-152
      max_err = std::max(max_err, std::fabs(zh[i * N + j] - ref));
    }
  CHECK(max_err < 1e-3f);
  // the coverage kernel of the reference's schedule tests: every tile holds its own index, none keeps the fill
  auto idx = api::full<int32_t>(-0x5EAD, {24, 40}).sync_on(stream).unwrap().partition({8, 8}).map({3, 2}, 5);
  auto [ip] = mapped_tile_index(std::move(idx)).sync_on(stream).unwrap();
  auto ih = api::to_host_vec(std::move(ip).unpartition()).sync_on(stream).unwrap();
  for (int r = 0; r < 24; ++r)
    for (int c = 0; c < 40; ++c) CHECK(ih[r * 40 + c] == (r / 8) * 5 + c / 8);
}

TEST(gemm_ones_non_divisible) {
  auto stream = new_stream();
  const int m = 200, n = 264, k = 128;
  auto x = api::ones<bf16>({m, k}).sync_on(stream).unwrap();
  auto y = api::ones<bf16>({k, n}).sync_on(stream).unwrap();
  auto z = api::zeros<bf16>({m, n}).sync_on(stream).unwrap();
  CHECK(gemm(z.partition_mut({128, 128}), &x, &y, k).sync_on(stream).is_ok());
  for (bf16 v : api::to_host_vec(z).sync_on(stream).unwrap()) CHECK(f32_from_bf16(v) == (float)k);
}

TEST(fmha_uniform_values) {
  auto stream = new_stream();
  const int b = 1, h = 2, s = 256, d = 64;
  // V == 1 -> every output is 1 whatever the scores; Q, K random
  auto to_bf16 = [&](Tensor<float> t) {
    auto arc = std::make_shared<Tensor<float>>(std::move(t));
    return std::move(api::convert<bf16>(arc).sync_on(stream).unwrap()).reshape({b, h, s, d}).unwrap();
  };
  auto q = to_bf16(api::randn(0.0f, 1.0f, {b * h * s * d}, 7).sync_on(stream).unwrap());
  auto k = to_bf16(api::randn(0.0f, 1.0f, {b * h * s * d}, 11).sync_on(stream).unwrap());
  auto v = api::ones<bf16>({b, h, s, d}).sync_on(stream).unwrap();
  auto out = api::zeros<bf16>({b * h, s, d}).sync_on(stream).unwrap();
  CHECK(fmha_causal(out.partition_mut({1, 64, d}), &q, &k, &v, 1.0f / std::sqrt((float)d), 0, 1).sync_on(stream).is_ok());
  for (bf16 o : api::to_host_vec(out).sync_on(stream).unwrap()) CHECK(std::fabs(f32_from_bf16(o) - 1.0f) < 1e-2f);
}

TEST(mxfp8_example_all_ones) {
  auto stream = new_stream();
  const int M = 16, N = 16, K = 128;
  auto bytes = [&](uint8_t v, int n, std::vector<int32_t> shape) {
    auto host = std::make_shared<std::vector<uint8_t>>(n, v);
    return std::make_shared<Tensor<uint8_t>>(std::move(api::copy_host_vec_to_device(host).sync_on(stream).unwrap()).reshape(std::move(shape)).unwrap());
  };
  auto x = Tensor<uint8_t>::reinterpret<f8e4m3fn>(bytes(0x38, M * K, {M, K}), {M, K}).unwrap();
  auto y = Tensor<uint8_t>::reinterpret<f8e4m3fn>(bytes(0x38, N * K, {N, K}), {N, K}).unwrap();
  auto xs = Tensor<uint8_t>::reinterpret<f8e8m0fnu>(bytes(0x7F, M * K / 32, {M, K / 32}), {M, K / 32}).unwrap();
  auto ys = Tensor<uint8_t>::reinterpret<f8e8m0fnu>(bytes(0x7F, N * K / 32, {N, K / 32}), {N, K / 32}).unwrap();
  auto z = partition_op(api::zeros<float>({M, N}), {16, 16});
  auto res = linear_tile(std::move(z), x, y, xs, ys, 1.0f).generics({"16", "16", "64", "2"}).sync_on(stream).unwrap();
  auto host = api::to_host_vec(std::move(std::get<0>(res)).unpartition()).sync_on(stream).unwrap();
  for (float v : host) CHECK(std::fabs(v - (float)K) <= 1e-3f);
}

TEST(nvfp4_example_all_ones) {
  // cutile-examples/examples/nvfp4.rs:96-160: packed ones (nibble 0x2), scales 1.0 (0x38), 16x16x64 tiles -> z = K
  auto stream = new_stream();
  const int M = 16, N = 16, K = 128;
  auto bytes = [&](uint8_t v, int n, std::vector<int32_t> shape) {
    auto host = std::make_shared<std::vector<uint8_t>>(n, v);
    return std::make_shared<Tensor<uint8_t>>(std::move(api::copy_host_vec_to_device(host).sync_on(stream).unwrap()).reshape(std::move(shape)).unwrap());
  };
  const uint8_t one = f4e2m1fnx2_one().bits;
  CHECK(one == 0x22 && f4e2m1fnx2::from_nibbles(0x7, 0x1).low() == 0x7 && f4e2m1fnx2::from_nibbles(0x7, 0x1).high() == 0x1);
  auto x = Tensor<uint8_t>::reinterpret<f4e2m1fnx2>(bytes(one, M * K / 2, {M, K / 2}), {M, K / 2}).unwrap();
  auto y = Tensor<uint8_t>::reinterpret<f4e2m1fnx2>(bytes(one, N * K / 2, {N, K / 2}), {N, K / 2}).unwrap();
  auto xs = Tensor<uint8_t>::reinterpret<f8e4m3fn>(bytes(0x38, M * K / 16, {M, K / 16}), {M, K / 16}).unwrap();
  auto ys = Tensor<uint8_t>::reinterpret<f8e4m3fn>(bytes(0x38, N * K / 16, {N, K / 16}), {N, K / 16}).unwrap();
  auto z = partition_op(api::zeros<float>({M, N}), {16, 16});
  auto res = linear_tile(std::move(z), x, y, xs, ys, 1.0f).generics({"16", "16", "64", "32", "4"}).sync_on(stream).unwrap();
  auto host = api::to_host_vec(std::move(std::get<0>(res)).unpartition()).sync_on(stream).unwrap();
  for (float v : host) CHECK(v == (float)K);
}

TEST(eye_and_eye_rect) {
  // cutile/tests/arange.rs:106-186: eye(4), eye(32), eye_rect(16, 32), eye_rect(32, 16), plus sizes off the 16 x 16 tiles
  auto stream = new_stream();
  const std::pair<size_t, size_t> cases[] = {{4, 4}, {32, 32}, {16, 32}, {32, 16}, {3, 5}, {100, 37}};
  for (auto [rows, cols] : cases) {
    auto m = (rows == cols ? api::eye(rows) : api::eye_rect(rows, cols)).sync_on(stream).unwrap();
    CHECK(m.shape() == (std::vector<int32_t>{(int32_t)rows, (int32_t)cols}));
    auto host = api::to_host_vec(m).sync_on(stream).unwrap();
    CHECK(host.size() == rows * cols);
    bool ok = true;
    for (size_t r = 0; r < rows; ++r)
      for (size_t c = 0; c < cols; ++c) ok = ok && host[r * cols + c] == (r == c ? 1.0f : 0.0f);
    CHECK(ok);
  }
}

TEST(example_programs_batch_matmul_scale_ptr_dropout_mlp) {
  auto stream = new_stream();
  {  // cutile-examples/examples/batch_matmul.rs:49-76: ones [4,128,64] x ones [4,64,256], tiles (64, 64, 32) -> every output K
    const int batch = 4, m = 128, n = 256, k = 64;
    auto a = std::make_shared<Tensor<float>>(api::ones<float>({batch, m, k}).sync_on(stream).unwrap());
    auto b = std::make_shared<Tensor<float>>(api::ones<float>({batch, k, n}).sync_on(stream).unwrap());
    auto c = api::zeros<float>({batch, m, n}).sync_on(stream).unwrap().partition({1, 64, 64});
    auto res = batch_matmul(std::move(c), a, b, k).generics({"f32", "64", "64", "32", "64"}).sync_on(stream).unwrap();
    auto host = api::to_host_vec(std::move(std::get<0>(res)).unpartition()).sync_on(stream).unwrap();
    CHECK(host.size() == (size_t)batch * m * n);
    for (float v : host) CHECK(v == (float)k);
  }
  {  // cutile-examples/examples/scale_ptr.rs:86-110: arange(1024) * 3 through raw pointers, 4 tile blocks
    const int len = 1024;
    auto input = api::arange<float>(len).sync_on(stream).unwrap();
    auto output = api::zeros<float>({len}).sync_on(stream).unwrap();
    CHECK(scale_ptr(output.device_pointer(), input.device_pointer(), 3.0f, len).grid(4, 1, 1).sync_on(stream).is_ok());
    auto in_host = api::to_host_vec(input).sync_on(stream).unwrap();
    auto out_host = api::to_host_vec(output).sync_on(stream).unwrap();
    for (int i = 0; i < len; ++i) CHECK(out_host[i] == in_host[i] * 3.0f);
    // no partition to infer a grid from
    auto err = scale_ptr(output.device_pointer(), input.device_pointer(), 3.0f, len).sync_on(stream);
    CHECK(err.is_err() && err.error().message.find("Launch grid required.") != std::string::npos);
  }
  {  // cutile-examples/examples/dropout.rs:39-50: m = 16, tiles of 4, p = 0.4, seeded inputs; (p, x, x_keep, out) come back
    const float p = 0.4f;
    auto x = std::make_shared<Tensor<float>>(api::randn(0.0f, 1.0f, {16}, 123).sync_on(stream).unwrap());
    auto x_keep = std::make_shared<Tensor<float>>(api::rand<float>({16}, 123).sync_on(stream).unwrap());
    auto out = api::zeros<float>({16}).sync_on(stream).unwrap().partition({4});
    auto res = dropout(p, x, x_keep, std::move(out)).sync_on(stream).unwrap();
    auto host = api::to_host_vec(std::move(std::get<3>(res)).unpartition()).sync_on(stream).unwrap();
    auto keep = api::to_host_vec(x_keep).sync_on(stream).unwrap();
    for (int i = 0; i < 16; ++i) CHECK(host[i] == (keep[i] > p ? keep[i] : 0.0f) / (1.0f - p));
  }
  {  // cutile-examples/examples/async_mlp.rs:124-137: gemm(data, w0) -> matvec(., w1) -> relu, dim 16, tiles of 4, lazily chained
    const int dim = 16, bd = 4;
    auto data = std::make_shared<Tensor<float>>(api::randn(0.0f, 1.0f, {dim, dim}, 1).sync_on(stream).unwrap());
    auto w0 = std::make_shared<Tensor<float>>(api::randn(0.0f, 1.0f, {dim, dim}, 2).sync_on(stream).unwrap());
    auto w1 = std::make_shared<Tensor<float>>(api::randn(0.0f, 1.0f, {dim}, 3).sync_on(stream).unwrap());
    auto out0 = gemm(partition_op(api::zeros<float>({dim, dim}), {bd, bd}), data, w0, dim).generics({"f32", "4", "4", "4"}).first();
    auto out1 = matvec(partition_op(api::zeros<float>({dim}), {bd}), unpartition_op(std::move(out0)), w1, dim).generics({"4", "4", "16"}).first();
    auto out = api::to_host_vec_op(unpartition_op(relu(std::move(out1)).first())).sync_on(stream).unwrap();
    auto d = api::to_host_vec(data).sync_on(stream).unwrap(), a = api::to_host_vec(w0).sync_on(stream).unwrap(), v = api::to_host_vec(w1).sync_on(stream).unwrap();
    for (int r = 0; r < dim; ++r) {
      double acc = 0;
      for (int c = 0; c < dim; ++c) {
        double h = 0;
        for (int kk = 0; kk < dim; ++kk) h += (double)d[r * dim + kk] * a[kk * dim + c];
        acc += h * v[c];
      }
      CHECK(std::fabs(out[r] - std::max(acc, 0.0)) < 1e-3);
    }
  }
}

TEST(random_constructors_draw_on_the_device) {
  // api::randn / rand / randn_f16 (cutile/src/api.rs:683-735): distribution, seed determinism, shapes
  auto stream = new_stream();
  const int n = 1 << 20;
  auto a = api::to_host_vec(api::randn(1.0f, 2.0f, {n}, 42).sync_on(stream).unwrap()).sync_on(stream).unwrap();
  auto b = api::to_host_vec(api::randn(1.0f, 2.0f, {n}, 42).sync_on(stream).unwrap()).sync_on(stream).unwrap();
  auto c = api::to_host_vec(api::randn(1.0f, 2.0f, {n}, 43).sync_on(stream).unwrap()).sync_on(stream).unwrap();
  CHECK(a == b);
  CHECK(a != c);
  double mean = 0, var = 0;
  for (float v : a) mean += v;
  mean /= n;
  for (float v : a) var += (v - mean) * (v - mean);
  var /= n;
  CHECK(std::fabs(mean - 1.0) < 1e-2 && std::fabs(std::sqrt(var) - 2.0) < 1e-2);
  auto u_t = api::rand<double>({64, 32}, 5).sync_on(stream).unwrap();
  CHECK((u_t.shape() == std::vector<int32_t>{64, 32}));
  auto u = api::to_host_vec(u_t).sync_on(stream).unwrap();
  double umean = 0;
  for (double v : u) {
    CHECK(v >= 0.0 && v < 1.0);
    umean += v;
  }
  CHECK(std::fabs(umean / u.size() - 0.5) < 0.03);
  auto h_t = api::randn_f16(0.0f, 1.0f, {128, 256}, 9).sync_on(stream).unwrap();
  CHECK((h_t.shape() == std::vector<int32_t>{128, 256}));
  auto h = api::to_host_vec(h_t).sync_on(stream).unwrap();
  auto f = api::to_host_vec(api::randn(0.0f, 1.0f, {128 * 256}, 9).sync_on(stream).unwrap()).sync_on(stream).unwrap();
  for (size_t i = 0; i < h.size(); ++i) CHECK(std::fabs(f32_from_f16(h[i]) - f[i]) <= std::fabs(f[i]) * 0.001f + 1e-7f);   // the f32 draw, rounded
  // without a seed the generator's default seed is used: still a valid draw
  auto d = api::to_host_vec(api::rand<float>({1000}).sync_on(stream).unwrap()).sync_on(stream).unwrap();
  for (float v : d) CHECK(v >= 0.0f && v < 1.0f);
}

TEST(graph_replay_matches_eager) {
  auto stream = new_stream();
  const int n = 1 << 16;
  auto w = api::randn(0.0f, 1.0f, {n}, 3).sync_on(stream).unwrap();
  auto input = api::zeros<float>({n}).sync_on(stream).unwrap();
  auto acc = api::zeros<float>({n}).sync_on(stream).unwrap();
  // graph: acc <- input; acc <- 2*w + acc; acc <- 0.5*w + acc
  auto graph = HipGraph<Unit>::scope(stream, [&](Scope& s) -> Result<Unit> {
    CUTILE_TRY(s.record(api::memcpy(acc, input)));
    CUTILE_TRY(s.record(saxpy(acc.partition_mut({1024}), 2.0f, &w)));
    CUTILE_TRY(s.record(saxpy(acc.partition_mut({1024}), 0.5f, &w)));
    return ok();
  }).unwrap();
  auto wh = api::to_host_vec(w).sync_on(stream).unwrap();
  for (int rep = 0; rep < 4; ++rep) {  // several replays with eager work and syncs in between
    auto fresh = api::full<float>((double)rep, {n}).sync_on(stream).unwrap();
    CHECK(graph.update(api::memcpy(input, fresh)).is_ok());
    CHECK(graph.launch().sync_on(stream).is_ok());
    auto got = api::to_host_vec(acc).sync_on(stream).unwrap();
    for (int i = 0; i < n; i += 97) {
      float eager = std::fmaf(0.5f, wh[i], std::fmaf(2.0f, wh[i], (float)rep));
      CHECK(got[i] == eager);
    }
  }
  // graph_on keeps the captured op's output; launching it again recomputes in place
  auto y = api::zeros<float>({n}).sync_on(stream).unwrap();
  auto g2 = saxpy(y.partition_mut({1024}), 1.0f, &w).graph_on(stream).unwrap();
  CHECK(g2.take_output().has_value());
  CHECK(g2.launch().sync_on(stream).is_ok());
  auto yh = api::to_host_vec(y).sync_on(stream).unwrap();
  for (int i = 0; i < n; i += 101) CHECK(yh[i] == wh[i]);  // one replay after a capture pass that does not execute
}

TEST(futures_complete_through_the_reactor) {
  // CUTILE_ASYNC_SPIN_BUDGET_US=0 (set in main) forces the notification path
  auto stream = new_stream();
  const int n = 1 << 20;
  auto w = api::ones<float>({n}).sync_on(stream).unwrap();
  auto y = api::zeros<float>({n}).sync_on(stream).unwrap();
  uint64_t before = cutile_reactor_registrations();
  for (int i = 0; i < 50; ++i) CHECK(saxpy(y.partition_mut({1024}), 1.0f, &w).schedule_on(stream).block_on().is_ok());
  CHECK(cutile_reactor_registrations() == before + 50 && cutile_reactor_armed() == 0);
  auto host = api::to_host_vec(y).sync_on(stream).unwrap();
  CHECK(host[0] == 50.0f && host[n - 1] == 50.0f);
  // wait() on the default policy, from several threads at once
  std::atomic<int> okc{0};
  std::vector<std::thread> ts;
  for (int t = 0; t < 4; ++t)
    ts.emplace_back([&] {
      for (int i = 0; i < 25; ++i)
        if (api::to_host_vec_op(api::full<float>(3.0, {4096})).wait().unwrap()[4095] == 3.0f) okc.fetch_add(1);
    });
  for (auto& t : ts) t.join();
  CHECK(okc.load() == 100);
}

TEST(memory_pool_and_streams) {
  auto dev = Device::create(0).unwrap();
  auto pool = dev->new_mem_pool().unwrap();
  CHECK(pool->set_release_threshold(64u << 20).is_ok());
  CHECK(cutile_set_device_pool(0, pool->raw()) == CUTILE_SUCCESS);
  auto stream = dev->new_stream().unwrap();
  {
    auto t = api::zeros<float>({1 << 20}).sync_on(stream).unwrap();  // allocated from the thread's pool
    auto st = pool->mem_stats().unwrap();
    CHECK(st.used_current >= (4u << 20) && st.used_high >= st.used_current);
  }
  CHECK(cutile_set_device_pool(0, nullptr) == CUTILE_SUCCESS);
  CHECK(stream->query().is_ok() && stream->synchronize().is_ok());
}

TEST(do_bench_and_autotune_pick_a_variant) {
  auto stream = new_stream();
  const int rows = 4096, n = 8192;
  auto x = api::full<f16>(1.0, {rows, n}).sync_on(stream).unwrap();
  auto w = api::ones<f16>({n}).sync_on(stream).unwrap();
  auto out = api::zeros<f16>({rows, n}).sync_on(stream).unwrap();
  bench::BenchOptions bo;
  bo.warmup = std::chrono::milliseconds(5);
  bo.rep = std::chrono::milliseconds(20);
  auto m = bench::do_bench(stream, bo, [&](const std::shared_ptr<Stream>& s) -> Result<Unit> {
    auto r = rms_norm_f16(&x, &w, out.partition_mut({1, n}), 1e-6f).async_on(s);
    return r.is_err() ? Result<Unit>(r.error()) : ok();
  }).unwrap();
  CHECK(m.reps() >= 5 && m.median_ms() > 0.005f && m.median_ms() < 5.0f && m.min_ms() <= m.median_ms());
  auto tuned = tune::Autotuner("rms_norm_f16_8192").configs(tune::variant_configs("rms_norm_f16")).bench_options(bo)
                   .run(stream, [&](const std::shared_ptr<Stream>&, const tune::Config& c) -> Result<bench::BenchFn> {
                     std::string v = *c.str("variant");
                     // probe once: variants that cannot hold an 8192-wide row are invalid candidates
                     auto probe = rms_norm_f16(&x, &w, out.partition_mut({1, n}), 1e-6f).variant(v).sync_on(stream);
                     if (probe.is_err()) return probe.error();
                     return bench::BenchFn([&, v](const std::shared_ptr<Stream>& s) -> Result<Unit> {
                       auto r = rms_norm_f16(&x, &w, out.partition_mut({1, n}), 1e-6f).variant(v).async_on(s);
                       return r.is_err() ? Result<Unit>(r.error()) : ok();
                     });
                   }).unwrap();
  CHECK(tuned.best.has_value());
  int invalid = 0;
  for (auto& t : tuned.trials) invalid += !t.measured;
  CHECK(invalid >= 4);  // w1v1..w1v8 cannot hold the row
  std::string best = *tuned.best->str("variant");
  CHECK(best != "generic");
  // the winner goes into a provenance-checked record and comes back verified (tune.rs:762-1016)
  auto space = tune::space_hash(tune::variant_configs("rms_norm_f16"));
  auto ws = tune::Workspace::of_kernel("rms_norm_f16", space).unwrap();
  tune::Record record(ws);
  float best_ms = INFINITY;
  size_t best_reps = 0;
  for (auto& t : tuned.trials)
    if (t.measured && t.config_id == tuned.best->id && t.median_ms < best_ms) { best_ms = t.median_ms; best_reps = t.reps; }
  record.insert({"n<=8192", *tuned.best, best_ms, best_reps, tune::variant_key("rms_norm_f16", best).unwrap()});
  std::string record_path = "/tmp/cutile_rms_norm_record_" + std::to_string(getpid()) + ".json";
  CHECK(record.save(record_path).is_ok());
  auto [loaded, warnings] = tune::Record::load_verified(record_path, ws, [](const tune::RecordEntry& e) {
    return tune::variant_key("rms_norm_f16", *e.config.str("variant"));
  }).unwrap();
  CHECK(warnings.empty() && *loaded.get("n<=8192")->config.str("variant") == best);
  auto other = tune::Workspace::of_kernel("softmax", space).unwrap();       // another kernel's workspace refuses it
  CHECK(tune::Record::load_verified(record_path, other, [](const tune::RecordEntry&) -> Result<std::optional<std::string>> { return std::optional<std::string>(); }).is_err());
  remove(record_path.c_str());
  best = *loaded.get("n<=8192")->config.str("variant");
  CHECK(cutile_kernel_set_preferred_variant("rms_norm_f16", best.c_str()) == CUTILE_SUCCESS);
  CHECK(rms_norm_f16(&x, &w, out.partition_mut({1, n}), 1e-6f).sync_on(stream).is_ok());
  CHECK(cutile_kernel_set_preferred_variant("rms_norm_f16", nullptr) == CUTILE_SUCCESS);
  printf("     autotune picked rms_norm_f16 variant %s\n", best.c_str());
}

int main(int argc, char** argv) {
  setenv("CUTILE_ASYNC_SPIN_BUDGET_US", "0", 1);
  return run_all_tests(argc, argv);
}
