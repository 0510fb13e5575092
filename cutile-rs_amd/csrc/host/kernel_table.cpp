// Part B of the C ABI: the table of precompiled gfx950 kernels (see kernel_table.h).
#include "kernel_table.h"
#include "toolchain.h"   // written by the build: CUTILE_TOOLCHAIN_FINGERPRINT

#include <array>
#include <atomic>
#include <cstring>
#include <deque>
#include <map>
#include <mutex>
#include <string>
#include <unordered_map>

// Code objects, embedded by embed.S (one ELF image per kernel source file).
extern "C" {
extern const unsigned char cutile_img_elementwise_start[], cutile_img_elementwise_end[];
extern const unsigned char cutile_img_rowwise_start[], cutile_img_rowwise_end[];
extern const unsigned char cutile_img_gemm_start[], cutile_img_gemm_end[];
extern const unsigned char cutile_img_fmha_start[], cutile_img_fmha_end[];
extern const unsigned char cutile_img_mxgemm_start[], cutile_img_mxgemm_end[];
extern const unsigned char cutile_img_nvfp4_start[], cutile_img_nvfp4_end[];
extern const unsigned char cutile_img_rng_start[], cutile_img_rng_end[];
}

namespace cutile {
namespace {

std::atomic<uint64_t> g_module_loads{0};
std::mutex g_pref_mutex;
std::map<std::string, std::string> g_preferred;
// winners of tuning records: "function|bucket" -> variant
std::map<std::string, std::string> g_bucket_preferred;

struct ImageRef {
  const unsigned char* start;
  const unsigned char* end;
};
ImageRef image_ref(Image img) {
  switch (img) {
    case IMG_ELEMENTWISE: return {cutile_img_elementwise_start, cutile_img_elementwise_end};
    case IMG_ROWWISE: return {cutile_img_rowwise_start, cutile_img_rowwise_end};
    case IMG_GEMM: return {cutile_img_gemm_start, cutile_img_gemm_end};
    case IMG_FMHA: return {cutile_img_fmha_start, cutile_img_fmha_end};
    case IMG_MXGEMM: return {cutile_img_mxgemm_start, cutile_img_mxgemm_end};
    case IMG_NVFP4: return {cutile_img_nvfp4_start, cutile_img_nvfp4_end};
    case IMG_RNG: return {cutile_img_rng_start, cutile_img_rng_end};
    default: return {nullptr, nullptr};
  }
}

std::vector<KernelEntry> build_table() {
  std::vector<KernelEntry> t;
  auto add = [&](const char* fn, const char* variant, const char* symbol, Image img, uint32_t threads,
                 uint32_t lds, int bm, int bn, int bk, int extra, const char* dtype, int64_t capacity,
                 int rank) {
    t.push_back(KernelEntry{fn, variant, symbol, img, {threads, 1, 1}, lds, {bm, bn, bk, extra}, dtype,
                            capacity, rank});
  };
  // ---- elementwise / creation (256 threads, no LDS) ----
#define EW(fn, dtype, suffix, rank) \
  add(fn, dtype "_" suffix, fn "_entry__" dtype "_" suffix, IMG_ELEMENTWISE, 256, 0, 0, 0, 0, 0, dtype, 0, rank)
  {
    EW("saxpy", "f32", "r1_flat", 1); EW("saxpy", "f32", "r2_flat", 2);
    EW("saxpy", "f32", "r1_tiled", 1); EW("saxpy", "f32", "r2_tiled", 2);
    EW("saxpy", "f16", "r1_flat", 1); EW("saxpy", "f16", "r2_flat", 2);
    EW("saxpy", "f16", "r1_tiled", 1); EW("saxpy", "f16", "r2_tiled", 2);
    EW("saxpy", "f64", "r1_flat", 1); EW("saxpy", "f64", "r2_flat", 2);
    EW("saxpy", "f64", "r1_tiled", 1); EW("saxpy", "f64", "r2_tiled", 2);
    EW("axpy", "f32", "r1_flat", 1); EW("axpy", "f32", "r1_tiled", 1);
    EW("axpy", "f16", "r1_flat", 1); EW("axpy", "f16", "r1_tiled", 1);
    EW("axpy", "f64", "r1_flat", 1); EW("axpy", "f64", "r1_tiled", 1);
    EW("add", "f32", "r1_flat", 1); EW("add", "f32", "r1_tiled", 1); EW("add", "f32", "r2_tiled", 2);
    EW("add", "f16", "r1_flat", 1); EW("add", "f16", "r1_tiled", 1); EW("add", "f16", "r2_tiled", 2);
    EW("add", "bf16", "r1_flat", 1); EW("add", "bf16", "r1_tiled", 1); EW("add", "bf16", "r2_tiled", 2);
    EW("add", "f32", "r2_flat", 2); EW("add", "f16", "r2_flat", 2); EW("add", "bf16", "r2_flat", 2);
    EW("silu_mul_2d_f16", "f16", "r2_flat", 2); EW("silu_mul_2d_f16", "f16", "r2_tiled", 2);
  }
  add("rope", "f16", "rope_entry__f16", IMG_ELEMENTWISE, 256, 0, 0, 0, 0, 0, "f16", 0, 3);
  add("kv_cache_update", "f16", "kv_cache_update_entry__f16", IMG_ELEMENTWISE, 256, 0, 0, 0, 0, 0, "f16", 0, 3);
  // greedy sampling and row gathers (cutile-kernels/src/argmax.rs, embeddings.rs, pointwise.rs:86-99)
  add("argmax_blocks", "f16", "argmax_blocks_entry__f16", IMG_ELEMENTWISE, 256, 0, 0, 0, 0, 0, "f16", 0, 1);
  add("lm_head_argmax_blocks", "f16", "lm_head_argmax_blocks_entry__f16", IMG_ELEMENTWISE, 256, 0, 64, 0, 0, 0, "f16", 0, 2);
  add("argmax_reduce_blocks", "u32", "argmax_reduce_blocks_entry__u32", IMG_ELEMENTWISE, 256, 0, 0, 0, 0, 0, "u32", 0, 1);
  add("embedding_batch", "f16", "embedding_batch_entry__f16", IMG_ELEMENTWISE, 256, 0, 0, 0, 0, 0, "f16", 0, 2);
  add("gather_row", "f16", "gather_row_entry__f16", IMG_ELEMENTWISE, 256, 0, 0, 0, 0, 0, "f16", 0, 2);
  add("qk_norm_rope_kv", "f16", "qk_norm_rope_kv_entry__f16", IMG_ELEMENTWISE, 256, 0, 0, 0, 0, 0, "f16", 0, 3);
  add("kvbm_copy", "f16", "kvbm_copy_entry__f16", IMG_ELEMENTWISE, 256, 0, 0, 0, 0, 0, "f16", 0, 3);
#undef EW
  static const char* kCreationTypes[] = {"f32", "f64", "f16", "bf16", "i32", "i64", "u8", "u16", "u32"};
  static std::deque<std::string> names;  // keeps generated strings alive at stable addresses
  auto keep = [&](std::string s) -> const char* {
    names.push_back(std::move(s));
    return names.back().c_str();
  };
  for (const char* ty : kCreationTypes) {
    add("full", ty, keep(std::string("full_entry__") + ty), IMG_ELEMENTWISE, 256, 0, 0, 0, 0, 0, ty, 0, 1);
    add("arange", ty, keep(std::string("arange_entry__") + ty), IMG_ELEMENTWISE, 256, 0, 0, 0, 0, 0, ty, 0, 1);
  }
  // random fills behind cutile_rng_* (Philox4x32-10)
  add("rng_fill", "f32", "rng_fill_entry__f32", IMG_RNG, 256, 0, 0, 0, 0, 0, "f32", 0, 1);
  add("rng_fill", "f64", "rng_fill_entry__f64", IMG_RNG, 256, 0, 0, 0, 0, 0, "f64", 0, 1);
  add("linspace", "f32", "linspace_entry__f32", IMG_ELEMENTWISE, 256, 0, 0, 0, 0, 0, "f32", 0, 1);
  add("eye", "f32", "eye_entry__f32", IMG_ELEMENTWISE, 256, 0, 0, 0, 0, 0, "f32", 0, 2);
  // the example programs' small kernels (cutile-examples/examples/async_mlp.rs, dropout.rs, scale_ptr.rs)
  add("relu", "f32", "relu_entry__f32", IMG_ELEMENTWISE, 256, 0, 0, 0, 0, 0, "f32", 0, 1);
  add("dropout", "f32", "dropout_entry__f32", IMG_ELEMENTWISE, 256, 0, 0, 0, 0, 0, "f32", 0, 1);
  add("scale_ptr", "f32", "scale_ptr_entry__f32", IMG_ELEMENTWISE, 256, 0, 0, 0, 0, 0, "f32", 0, 1);
  add("matvec", "f32", "matvec_entry__f32", IMG_ELEMENTWISE, 256, 0, 0, 0, 0, 0, "f32", 0, 2);
  // the benchmark programs' all-f16 arithmetic (one wavefront per row; v = tile lanes per lane, c = 512-wide chunks)
  for (int v : {1, 2, 4, 8, 16})
    add("rms_norm_all_f16", keep("v" + std::to_string(v)), keep("rms_norm_all_f16_entry__v" + std::to_string(v)), IMG_ROWWISE, 256, 0, 0, 0, 0,
        0, "f16", 0, 2);
  for (auto cv : {std::pair<int, int>{1, 1}, {1, 2}, {1, 4}, {1, 8}, {2, 8}, {4, 8}, {8, 8}, {16, 8}, {32, 8}})
    add("softmax_all_f16", keep("c" + std::to_string(cv.first) + "v" + std::to_string(cv.second)),
        keep("softmax_all_f16_entry__c" + std::to_string(cv.first) + "v" + std::to_string(cv.second)), IMG_ROWWISE, 256, 0, 0, 0, 0, 0, "f16", 0, 2);
  static const char* kConvertTypes[] = {"f32", "f64", "f16", "bf16", "i32", "i64"};
  for (const char* s : kConvertTypes)
    for (const char* d : kConvertTypes)
      add("convert", keep(std::string(s) + "_" + d), keep(std::string("convert_entry__") + s + "_" + d),
          IMG_ELEMENTWISE, 256, 0, 0, 0, 0, 0, s, 0, 1);

  // ---- row-wise (256 threads; capacity = elements of one segment held in registers;
  //      tile[2] = 16-byte vectors per lane, tile[3] = wavefronts per segment) ----
  struct RowVariant { int wpr, vpl; };
  static const RowVariant kRow[] = {{1, 1}, {1, 2}, {1, 4}, {1, 8}, {1, 16}, {2, 2}, {2, 4}, {2, 8},
                                    {4, 1}, {4, 2}, {4, 4}, {4, 8}, {4, 16}};
  for (auto rv : kRow) {
    std::string v = "w" + std::to_string(rv.wpr) + "v" + std::to_string(rv.vpl);
    add("rms_norm_f16", keep(v), keep("rms_norm_f16_entry__" + v), IMG_ROWWISE, 256, 0, 0, 0, rv.vpl, rv.wpr, "f16",
        (int64_t)rv.wpr * 64 * rv.vpl * 8, 2);
    add("softmax", keep("f16_" + v), keep("softmax_entry__f16_" + v), IMG_ROWWISE, 256, 0, 0, 0, rv.vpl, rv.wpr, "f16",
        (int64_t)rv.wpr * 64 * rv.vpl * 8, 2);
    add("softmax", keep("f32_" + v), keep("softmax_entry__f32_" + v), IMG_ROWWISE, 256, 0, 0, 0, rv.vpl, rv.wpr, "f32",
        (int64_t)rv.wpr * 64 * rv.vpl * 4, 2);
  }
  // short rows: LPR lanes per row, 4 passes of 256 / LPR rows per workgroup (tile[1] rows in all); capacity LPR * 8
  for (const char* fn : {"rms_norm_f16", "qk_norm_f16"})
    for (int lpr : {8, 16, 32}) {
      std::string v = "s" + std::to_string(lpr);
      add(fn, keep(v), keep(std::string(fn) + "_entry__" + v), IMG_ROWWISE, 256, 0, 0, 4 * 256 / lpr, 1, 1, "f16", (int64_t)lpr * 8, 2);
    }
  // the fused row norms of the transformer block share the register-resident row machinery
  static const RowVariant kFusedRow[] = {{1, 1}, {1, 2}, {1, 4}, {1, 8}, {2, 2}, {2, 4}, {2, 8}, {4, 1}, {4, 2}, {4, 4}, {4, 8}};
  for (const char* fn : {"add_rms_norm_f16", "qk_norm_f16"}) {
    for (auto rv : kFusedRow) {
      std::string v = "w" + std::to_string(rv.wpr) + "v" + std::to_string(rv.vpl);
      add(fn, keep(v), keep(std::string(fn) + "_entry__" + v), IMG_ROWWISE, 256, 0, 0, 0, rv.vpl, rv.wpr, "f16",
          (int64_t)rv.wpr * 64 * rv.vpl * 8, 2);
    }
    add(fn, "generic", keep(std::string(fn) + "_entry__generic"), IMG_ROWWISE, 256, 0, 0, 0, 0, 0, "f16", 0, 2);
  }
  add("rms_norm_f16", "generic", "rms_norm_f16_entry__generic", IMG_ROWWISE, 256, 0, 0, 0, 0, 0, "f16", 0, 2);
  add("rms_norm", "f32", "rms_norm_entry__f32", IMG_ROWWISE, 256, 0, 0, 0, 0, 0, "f32", 0, 2);   // the f32 example form
  add("softmax", "f16_generic", "softmax_entry__f16_generic", IMG_ROWWISE, 256, 0, 0, 0, 0, 0, "f16", 0, 2);
  add("softmax", "f32_generic", "softmax_entry__f32_generic", IMG_ROWWISE, 256, 0, 0, 0, 0, 0, "f32", 0, 2);

  // ---- bf16 GEMM: LDS = 2 stages x (BM*BK + BK*BN) x 2 bytes ----
  auto gemm = [&](const char* dtype, int bm, int bn, int bk, int wvm, int wvn, const char* kind = "w") {
    std::string v = std::string(dtype) + "_" + std::to_string(bm) + "x" + std::to_string(bn) + "x" +
                    std::to_string(bk) + "_" + kind + std::to_string(wvm) + "x" + std::to_string(wvn);
    // "r" = ring of three x stages and two y stages, the others hold two stages of each
    const uint32_t lds = kind[0] == 'r' || kind[0] == 'q' || kind[0] == 'p' ? (uint32_t)((3 * bm * bk + 2 * bk * bn) * 2) : (uint32_t)(2 * (bm * bk + bk * bn) * 2);
    add("gemm", keep(v), keep("gemm_entry__" + v), IMG_GEMM, (uint32_t)(wvm * wvn * 64), lds, bm, bn, bk, 0, dtype, 0, 2);
  };
  // first entry of a tile shape = default variant; "d" = global->LDS direct, pipelined
  gemm("bf16", 256, 256, 64, 4, 2, "d");
  gemm("bf16", 256, 256, 64, 2, 4, "d");
  gemm("bf16", 128, 128, 64, 2, 2, "d");
  gemm("bf16", 256, 256, 64, 4, 2, "r");
  gemm("bf16", 256, 256, 64, 2, 4, "r");
  gemm("bf16", 128, 128, 64, 2, 2, "r");
  gemm("bf16", 256, 256, 64, 2, 4, "q");   // "q" = the ring on v_mfma_f32_16x16x32
  gemm("bf16", 128, 128, 64, 2, 2, "q");   // 80 KiB of stages: two workgroups per compute unit
  gemm("bf16", 256, 256, 64, 2, 4, "p");   // "p" = the same tile body, one workgroup per compute unit walking its tiles
  // "s" = the same ring streaming over the output tiles a workgroup walks (one workgroup per compute unit, whole
  // tiles only).  A family of four kernels: the variant itself reads z as the initial accumulator and moves z past
  // the caches; "+cached" moves z through them, "+new" starts from zero.  The launcher picks the member; only the
  // family name is a variant a caller, a pin or a tuning record can name.
  auto stream_family = [&](const char* fn, const char* dtype, std::initializer_list<const char*> members) {
    const std::string v = std::string(dtype) + "_256x256x64_s2x4";
    for (const char* m : members) {
      std::string sym = std::string(fn) + "_entry__" + v;
      for (const char* c = m; *c; ++c) sym += *c == '+' ? '_' : *c;
      add(fn, keep(v + m), keep(sym), IMG_GEMM, 512, (uint32_t)((3 * 256 * 64 + 2 * 64 * 256) * 2), 256, 256, 64, 0, dtype, 0, 2);
    }
  };
  stream_family("gemm", "bf16", {"", "+cached", "+new", "+new+cached"});
  gemm("bf16", 256, 256, 64, 4, 2);
  gemm("bf16", 256, 256, 64, 2, 4);
  gemm("bf16", 256, 256, 64, 2, 2);
  gemm("bf16", 256, 128, 64, 2, 2);
  gemm("bf16", 128, 256, 64, 2, 2);
  gemm("bf16", 128, 128, 64, 2, 2);
  gemm("bf16", 64, 128, 64, 2, 2);
  gemm("f16", 256, 256, 64, 4, 2, "d");
  gemm("f16", 128, 128, 64, 2, 2, "d");
  gemm("f16", 256, 256, 64, 4, 2, "r");
  gemm("f16", 256, 256, 64, 2, 4, "r");
  gemm("f16", 256, 256, 64, 2, 4, "q");
  gemm("f16", 128, 128, 64, 2, 2, "q");
  gemm("f16", 256, 256, 64, 2, 4, "p");
  stream_family("gemm", "f16", {"", "+cached", "+new", "+new+cached"});
  gemm("bf16f32", 128, 128, 64, 2, 2);
  gemm("bf16f32", 256, 256, 64, 2, 2);
  // any tile shape, strides and extents (tile = 0: not tied to a partition shape); 64x64 outputs per workgroup
  for (const char* dt : {"bf16", "bf16f32", "f16", "f32"})
    add("gemm", keep(std::string(dt) + "_generic"), keep(std::string("gemm_entry__") + dt + "_generic"), IMG_GEMM, 256,
        (uint32_t)((64 * 17 + 16 * 65) * 4), 0, 0, 0, 0, dt, 0, 2);

  // batched GEMM (cutile-examples/examples/batch_matmul.rs): the pipelined bodies with the batch on a grid axis
  for (const char* kind : {"q", "r"})          // rings of three a stages and two b stages (q: on v_mfma_f32_16x16x32, any K; r: whole K tiles only)
    for (const char* dt : {"bf16", "f16"}) {
      std::string v = std::string(dt) + "_256x256x64_" + kind + "2x4";
      add("batch_matmul", keep(v), keep("batch_matmul_entry__" + v), IMG_GEMM, 512, (uint32_t)((3 * 256 * 64 + 2 * 64 * 256) * 2), 256, 256, 64, 0, dt, 0, 3);
    }
  for (auto t : {std::array<int, 4>{256, 256, 2, 4}, std::array<int, 4>{128, 128, 2, 2}}) {
    std::string v = "bf16_" + std::to_string(t[0]) + "x" + std::to_string(t[1]) + "x64_d" + std::to_string(t[2]) + "x" + std::to_string(t[3]);
    add("batch_matmul", keep(v), keep("batch_matmul_entry__" + v), IMG_GEMM, (uint32_t)(t[2] * t[3] * 64),
        (uint32_t)(2 * (t[0] * 64 + 64 * t[1]) * 2), t[0], t[1], 64, 0, "bf16", 0, 3);
  }
  for (auto t : {std::array<int, 4>{256, 256, 4, 2}, std::array<int, 4>{128, 128, 2, 2}}) {
    std::string v = "f16_" + std::to_string(t[0]) + "x" + std::to_string(t[1]) + "x64_d" + std::to_string(t[2]) + "x" + std::to_string(t[3]);
    add("batch_matmul", keep(v), keep("batch_matmul_entry__" + v), IMG_GEMM, (uint32_t)(t[2] * t[3] * 64),
        (uint32_t)(2 * (t[0] * 64 + 64 * t[1]) * 2), t[0], t[1], 64, 0, "f16", 0, 3);
  }
  for (const char* dt : {"bf16", "f16", "f32"})
    add("batch_matmul", keep(std::string(dt) + "_generic"), keep(std::string("batch_matmul_entry__") + dt + "_generic"), IMG_GEMM, 256,
        (uint32_t)((64 * 17 + 16 * 65) * 4), 0, 0, 0, 0, dt, 0, 3);

  // ---- NVFP4 GEMM: operands expanded to f16 on the way into LDS; LDS = 2 stages x (BM + BN) rows of 128 bytes ----
  // first (the default for 256 x 256 tiles) the forms on v_mfma_f32_16x16x32_f16 ("q"): +9 % at the power limit
  for (auto t : {std::array<int, 2>{2, 4}, std::array<int, 2>{4, 2}})
    for (const char* dt : {"f32", "bf16"}) {
      std::string v = std::string(dt) + "_256x256x64_q" + std::to_string(t[0]) + "x" + std::to_string(t[1]);
      add("linear_tile_nvfp4", keep(v), keep("linear_tile_nvfp4_entry__" + v), IMG_NVFP4, 512, (uint32_t)(2 * 512 * 128), 256, 256, 64, 0, dt, 0, 2);
    }
  for (auto t : {std::array<int, 4>{256, 256, 4, 2}, std::array<int, 4>{256, 256, 2, 4}, std::array<int, 4>{128, 128, 2, 2},
                 std::array<int, 4>{64, 64, 1, 1}, std::array<int, 4>{32, 32, 1, 1}})
    for (const char* dt : {"f32", "bf16"}) {
      if (dt[0] == 'b' && t[0] < 128) continue;
      std::string v = std::string(dt) + "_" + std::to_string(t[0]) + "x" + std::to_string(t[1]) + "x64_w" + std::to_string(t[2]) + "x" + std::to_string(t[3]);
      add("linear_tile_nvfp4", keep(v), keep("linear_tile_nvfp4_entry__" + v), IMG_NVFP4, (uint32_t)(t[2] * t[3] * 64),
          (uint32_t)(2 * (t[0] + t[1]) * 128), t[0], t[1], 64, 0, dt, 0, 2);
    }
  // ---- persistent GEMM over a mapped partition: the pipelined bodies in a stream-item loop ----
  // first the ring on v_mfma_f32_16x16x32
  for (const char* dt : {"bf16", "f16"}) {
    std::string v = std::string(dt) + "_256x256x64_q2x4";
    add("gemm_persistent", keep(v), keep("gemm_persistent_entry__" + v), IMG_GEMM, 512, (uint32_t)((3 * 256 * 64 + 2 * 64 * 256) * 2), 256, 256, 64, 0, dt, 0, 2);
  }
  for (const char* dt : {"bf16", "f16"}) stream_family("gemm_persistent", dt, {"", "+cached"});   // from zero accumulators always
  // 2 x 4 wavefronts first at 256 x 256: the item loop around the tile body costs the 4 x 2 form ten spilled registers (-2 %)
  for (auto t : {std::array<int, 4>{256, 256, 2, 4}, std::array<int, 4>{256, 256, 4, 2}, std::array<int, 4>{128, 128, 2, 2}}) {
    std::string v = "bf16_" + std::to_string(t[0]) + "x" + std::to_string(t[1]) + "x64_d" + std::to_string(t[2]) + "x" + std::to_string(t[3]);
    add("gemm_persistent", keep(v), keep("gemm_persistent_entry__" + v), IMG_GEMM, (uint32_t)(t[2] * t[3] * 64),
        (uint32_t)(2 * (t[0] * 64 + 64 * t[1]) * 2), t[0], t[1], 64, 0, "bf16", 0, 2);
  }
  // grouped GEMM over descriptor tables: first the ring on v_mfma_f32_16x16x32 (it masks a ragged last K tile itself)
  add("group_gemm_nt_desc", "f16_256x256x64_q2x4", "group_gemm_nt_desc_entry__f16_256x256x64_q2x4", IMG_GEMM, 512,
      (uint32_t)((3 * 256 * 64 + 2 * 64 * 256) * 2), 256, 256, 64, 0, "f16", 0, 2);
  // f16: persistent and grouped (descriptor-table) forms of the pipelined bodies
  for (auto t : {std::array<int, 4>{256, 256, 4, 2}, std::array<int, 4>{128, 128, 2, 2}}) {
    std::string v = "f16_" + std::to_string(t[0]) + "x" + std::to_string(t[1]) + "x64_d" + std::to_string(t[2]) + "x" + std::to_string(t[3]);
    add("gemm_persistent", keep(v), keep("gemm_persistent_entry__" + v), IMG_GEMM, (uint32_t)(t[2] * t[3] * 64),
        (uint32_t)(2 * (t[0] * 64 + 64 * t[1]) * 2), t[0], t[1], 64, 0, "f16", 0, 2);
    // the grouped form keeps the group descriptors live across the tile loop: 2 x 4 wavefronts at 256 x 256 (no spills)
    std::string gv = t[0] == 256 ? std::string("f16_256x256x64_d2x4") : v;
    add("group_gemm_nt_desc", keep(gv), keep("group_gemm_nt_desc_entry__" + gv), IMG_GEMM, (uint32_t)(t[2] * t[3] * 64),
        (uint32_t)(2 * (t[0] * 64 + 64 * t[1]) * 2), t[0], t[1], 64, 0, "f16", 0, 2);
  }
  for (const char* dt : {"bf16", "f16", "f32"})
    add("gemm_persistent", keep(std::string(dt) + "_generic"), keep(std::string("gemm_persistent_entry__") + dt + "_generic"),
        IMG_GEMM, 256, (uint32_t)((64 * 17 + 16 * 65) * 4), 0, 0, 0, 0, dt, 0, 2);
  for (int r = 1; r <= 3; ++r)
    add("mapped_tile_index", keep("i32_r" + std::to_string(r)), keep("mapped_tile_index_entry__i32_r" + std::to_string(r)),
        IMG_ELEMENTWISE, 256, 0, 0, 0, 0, 0, "i32", 0, r);
  add("mapped_shared_cache_update", "f32", "mapped_shared_cache_update_entry__f32", IMG_ELEMENTWISE, 256, 0, 0, 0, 0, 0, "f32", 0, 3);
  for (int r = 1; r <= 3; ++r)
    add("mapped_tile_index_within", keep("i32_r" + std::to_string(r)),
        keep("mapped_tile_index_within_entry__i32_r" + std::to_string(r)), IMG_ELEMENTWISE, 256, 0, 0, 0, 0, 0, "i32", 0, r);

  // ---- FMHA: LDS = 2 stages x (K tile + V tile) ----
  // "_pp": the two wavefronts of a SIMD run half a tile apart (BM = 256 only)
  auto fmha = [&](const char* dtype, int bm, int bn, int d, const char* suffix = "") {
    std::string v = std::string(dtype) + "_" + std::to_string(bm) + "x" + std::to_string(bn) + "x" + std::to_string(d) + suffix;
    add("fmha", keep(v), keep("fmha_entry__" + v), IMG_FMHA, (uint32_t)(bm / 32 * 64),
        (uint32_t)(2 * 2 * bn * d * 2), bm, bn, d, 0, dtype, 0, 3);
  };
  fmha("bf16", 256, 64, 128, "_pp");
  fmha("f16", 256, 64, 128, "_pp");
  fmha("bf16", 128, 64, 128);
  fmha("bf16", 128, 128, 128);
  fmha("bf16", 256, 64, 128);
  fmha("bf16", 128, 64, 64);
  fmha("bf16", 64, 64, 64);
  fmha("bf16", 64, 32, 32);
  fmha("bf16", 32, 32, 32);
  fmha("f16", 128, 64, 128);
  fmha("f16", 128, 64, 64);
  fmha("f16", 32, 32, 32);
  fmha("bf16", 128, 32, 256);
  fmha("f16", 128, 32, 256);
  // the same kernels with the query position read from device memory (sequence-layout callers)
  for (auto t : {std::array<int, 3>{128, 64, 128}, std::array<int, 3>{128, 64, 64}, std::array<int, 3>{32, 32, 32},
                 std::array<int, 3>{128, 32, 256}}) {
    std::string v = "f16_" + std::to_string(t[0]) + "x" + std::to_string(t[1]) + "x" + std::to_string(t[2]);
    add("fmha_seq", keep(v), keep("fmha_seq_entry__" + v), IMG_FMHA, (uint32_t)(t[0] / 32 * 64),
        (uint32_t)(2 * 2 * t[1] * t[2] * 2), t[0], t[1], t[2], 0, "f16", 0, 3);
  }

  // ---- decode attention: one workgroup per (KV head, split); tile = (GROUP, 0, D) ----
  for (int d : {64, 128, 256})
    for (int grp : {1, 2, 4, 8}) {
      std::string v = "f16_g" + std::to_string(grp) + "_d" + std::to_string(d);
      add("fmha_decode_gqa_split", keep(v), keep("fmha_decode_gqa_split_entry__" + v), IMG_FMHA, 256,
          (uint32_t)(4 * grp * (d + 2) * 4), grp, 0, d, 0, "f16", 0, 3);
    }
  // the same on the matrix cores (heads are the N dimension of a 16x16x32 MFMA, columns beyond GROUP are zero); LDS = 4 wavefronts x 2 stages x 32 V rows
  for (int d : {64, 128, 256})
    for (int grp : {1, 2, 4, 8, 16}) {
      std::string v = "f16_g" + std::to_string(grp) + "_d" + std::to_string(d) + "_mfma";
      add("fmha_decode_gqa_split", keep(v), keep("fmha_decode_gqa_split_entry__" + v), IMG_FMHA, 256, (uint32_t)(4 * 2 * 32 * d * 2), grp,
          0, d, 0, "f16", 0, 3);
    }
  // the batched-layout form of the matrix-core kernel: one workgroup per (batch, KV head, split)
  for (int d : {64, 128, 256})
    for (int grp : {1, 2, 4, 8, 16}) {
      std::string v = "f16_g" + std::to_string(grp) + "_d" + std::to_string(d);
      add("attention_decode_kernel_grouped", keep(v), keep("attention_decode_grouped_entry__" + v), IMG_FMHA, 256,
          (uint32_t)(4 * 2 * 32 * d * 2), grp, 0, d, 0, "f16", 0, 3);
    }
  add("splitk_reduce_merge", "f16", "splitk_reduce_merge_entry__f16", IMG_FMHA, 256, 0, 0, 0, 0, 0, "f16", 0, 3);

  // ---- MXFP8 GEMM: LDS = 2 stages x (BM + BN) x 128 bytes ----
  // "d", "e" = global->LDS direct, pipelined; scales staged in blocks of four K tiles (16 bytes per row, two blocks)
  auto mx = [&](const char* out, int bm, int bn, int wvm, int wvn, const char* kind = "w") {
    std::string v = std::string("mxfp8_") + out + "_" + std::to_string(bm) + "x" + std::to_string(bn) + "x128_" + kind +
                    std::to_string(wvm) + "x" + std::to_string(wvn);
    add("linear_tile", keep(v), keep("linear_tile_entry__" + v), IMG_MXGEMM, (uint32_t)(wvm * wvn * 64),
        (uint32_t)(2 * (bm + bn) * (128 + (kind[0] == 'd' || kind[0] == 'e' ? 16 : 0))), bm, bn, 128, 0, out, 0, 2);
  };
  mx("bf16", 256, 256, 4, 2, "d");
  mx("bf16", 256, 256, 2, 4, "d");
  mx("f32", 256, 256, 2, 4, "d");
  mx("bf16", 256, 256, 4, 2, "e");   // "e" = the direct pipeline on v_mfma_scale_f32_16x16x128_f8f6f4
  mx("f32", 256, 256, 4, 2, "e");
  mx("bf16", 256, 256, 2, 2);
  mx("bf16", 256, 256, 2, 4);
  mx("bf16", 128, 128, 2, 2);
  mx("f32", 256, 256, 2, 2);
  mx("f32", 128, 128, 2, 2);
  mx("f32", 32, 32, 1, 1);
  mx("f32", 64, 64, 1, 1);
  return t;
}

}  // namespace

const std::vector<KernelEntry>& kernel_table() {
  static const std::vector<KernelEntry> table = build_table();
  return table;
}

// (function, variant) -> entry.  Every launch looks its kernel up at least once, so the table is indexed once
// (the first entry of a key wins, as a scan in table order would find it).
const KernelEntry* find_entry(const char* function, const std::string& variant) {
  static const std::unordered_map<std::string, const KernelEntry*> index = [] {
    std::unordered_map<std::string, const KernelEntry*> m;
    for (const auto& e : kernel_table()) m.emplace(std::string(e.function) + '|' + e.variant, &e);
    return m;
  }();
  std::string key;
  key.reserve(strlen(function) + 1 + variant.size());
  key.append(function).push_back('|');
  key.append(variant);
  auto it = index.find(key);
  return it == index.end() ? nullptr : it->second;
}

std::string list_variants(const char* function) {
  std::string s;
  for (const auto& e : kernel_table())
    if (strcmp(e.function, function) == 0) {
      if (!s.empty()) s += ", ";
      s += e.variant;
    }
  return s;
}

std::string preferred_variant(const char* function) {
  std::lock_guard<std::mutex> lock(g_pref_mutex);
  auto it = g_preferred.find(function);
  return it == g_preferred.end() ? std::string() : it->second;
}

std::string preferred_variant_for(const char* function, const std::string& bucket) {
  if (bucket.empty()) return std::string();
  std::lock_guard<std::mutex> lock(g_pref_mutex);
  auto it = g_bucket_preferred.find(std::string(function) + "|" + bucket);
  return it == g_bucket_preferred.end() ? std::string() : it->second;
}

void clear_bucket_preferences() {
  std::lock_guard<std::mutex> lock(g_pref_mutex);
  g_bucket_preferred.clear();
}

void count_module_load() { g_module_loads.fetch_add(1, std::memory_order_relaxed); }

cutile_status_t load_entry(cutile_device_t device, const KernelEntry* entry, hipFunction_t* fn) {
  CUTILE_REQUIRE(device && entry && fn, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  // The device mutex makes the load single-flight: concurrent first launches of
  // one kernel load its code object once (tile_kernel.rs:371-399,705-733).
  std::lock_guard<std::mutex> lock(device->mutex);
  auto fit = device->functions.find(entry->symbol);
  if (fit != device->functions.end()) {
    *fn = fit->second;
    return CUTILE_SUCCESS;
  }
  CUTILE_API_OR_RETURN(api);
  cutile_module* mod = nullptr;
  auto mit = device->table_modules.find((int)entry->image);
  if (mit == device->table_modules.end()) {
    ImageRef img = image_ref(entry->image);
    CUTILE_REQUIRE(img.start && img.end > img.start, CUTILE_ERR_KERNEL_NOT_FOUND,
                   "no code object embedded for kernel %s", entry->symbol);
    CUTILE_HIP_OR_RETURN(api, hipSetDevice(device->ordinal));
    hipModule_t m = nullptr;
    CUTILE_HIP_OR_RETURN(api, hipModuleLoadData(&m, img.start));
    mod = new cutile_module();
    mod->device = device;
    mod->handle = m;
    device->table_modules[(int)entry->image] = mod;
    count_module_load();
  } else {
    mod = mit->second;
  }
  hipFunction_t f = nullptr;
  CUTILE_HIP_OR_RETURN(api, hipModuleGetFunction(&f, mod->handle, entry->symbol));
  device->functions[entry->symbol] = f;
  *fn = f;
  return CUTILE_SUCCESS;
}

}  // namespace cutile

using namespace cutile;

extern "C" {

uint64_t cutile_module_load_count(void) { return g_module_loads.load(std::memory_order_relaxed); }

int32_t cutile_kernel_list(const char** names, int32_t cap) {
  static std::vector<std::string> labels = [] {
    std::vector<std::string> v;
    for (const auto& e : kernel_table()) v.push_back(std::string(e.function) + ":" + e.variant);
    return v;
  }();
  for (int32_t i = 0; i < cap && i < (int32_t)labels.size(); ++i) names[i] = labels[i].c_str();
  return (int32_t)labels.size();
}

cutile_status_t cutile_kernel_set_preferred_variant(const char* function, const char* variant) {
  CUTILE_REQUIRE(function, CUTILE_ERR_INVALID_ARGUMENT, "function is null");
  std::lock_guard<std::mutex> lock(g_pref_mutex);
  if (!variant) {
    g_preferred.erase(function);
    return CUTILE_SUCCESS;
  }
  CUTILE_REQUIRE(find_entry(function, variant) != nullptr, CUTILE_ERR_KERNEL_NOT_FOUND,
                 "no variant '%s' of kernel '%s'; available: %s", variant, function,
                 list_variants(function).c_str());
  g_preferred[function] = variant;
  return CUTILE_SUCCESS;
}

cutile_status_t cutile_kernel_set_preferred_variant_for(const char* function, const char* bucket, const char* variant) {
  CUTILE_REQUIRE(function && bucket && *bucket, CUTILE_ERR_INVALID_ARGUMENT, "function or bucket is null");
  std::lock_guard<std::mutex> lock(g_pref_mutex);
  const std::string key = std::string(function) + "|" + bucket;
  if (!variant) {
    g_bucket_preferred.erase(key);
    return CUTILE_SUCCESS;
  }
  CUTILE_REQUIRE(find_entry(function, variant) != nullptr, CUTILE_ERR_KERNEL_NOT_FOUND,
                 "no variant '%s' of kernel '%s'; available: %s", variant, function, list_variants(function).c_str());
  g_bucket_preferred[key] = variant;
  return CUTILE_SUCCESS;
}

const char* cutile_library_version(void) { return "0.1.0"; }
const char* cutile_toolchain_fingerprint(void) { return CUTILE_TOOLCHAIN_FINGERPRINT; }
const char* cutile_target_arch(void) { return "gfx950"; }

cutile_status_t cutile_kernel_fingerprint(const char* function, const char* variant, char out[17]) {
  CUTILE_REQUIRE(function && out, CUTILE_ERR_INVALID_ARGUMENT, "null argument");
  const KernelEntry* entry = nullptr;
  for (const auto& e : kernel_table())
    if (strcmp(e.function, function) == 0 && (!variant || strcmp(e.variant, variant) == 0)) { entry = &e; break; }
  CUTILE_REQUIRE(entry, CUTILE_ERR_KERNEL_NOT_FOUND, "no kernel '%s'%s%s; available: %s", function, variant ? " variant " : "",
                 variant ? variant : "", list_variants(function).c_str());
  uint64_t h = 0xcbf29ce484222325ull;   // FNV-1a
  auto mix = [&](const unsigned char* p, size_t n) { for (size_t i = 0; i < n; ++i) { h ^= p[i]; h *= 0x100000001b3ull; } };
  const ImageRef img = image_ref(entry->image);
  mix(img.start, (size_t)(img.end - img.start));
  mix((const unsigned char*)function, strlen(function) + 1);
  if (variant) mix((const unsigned char*)entry->symbol, strlen(entry->symbol) + 1);
  snprintf(out, 17, "%016llx", (unsigned long long)h);
  return CUTILE_SUCCESS;
}

}  // extern "C"
