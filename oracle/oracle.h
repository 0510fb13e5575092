/*
 * CPU oracle for the tile-kernel path.  TEST INFRASTRUCTURE ONLY: nothing in the
 * shipped library links, loads or calls this; it is the checker the GPU kernels
 * are compared against, and the CPU baseline that is timed next to them.
 *
 * Every function restates, from the reference's text, either a naive CPU
 * reference the reference's own tests/examples use, or (where the reference has
 * none) the arithmetic of the kernel body itself.  The reference is Rust and
 * cannot be built in this image, so there is no compiled-reference cross-check;
 * each function lists what pins it instead.
 *
 *   orc_saxpy_f32        cutile-examples/examples/saxpy.rs:47-53 (answer = a*x+y),
 *                        evaluated with one fused multiply-add.  Pinned by the
 *                        reference vectors arange(32), a = 2 (exact either way).
 *   orc_add_f32          cutile/tests/gpu/add_basic.rs:29-43.
 *   orc_rms_norm_f16     cutile-kernels/src/norms.rs:28-60 (kernel body; the
 *                        reference has no CPU reference).  Pinned by closed forms
 *                        and an independent float64 evaluation: parity unpinned
 *                        by reference tests.
 *   orc_softmax_*        cutile-examples/examples/softmax.rs:11-24 (kernel body),
 *                        row sums = 1 (softmax.rs:55-60).  Pinned by closed forms
 *                        and scipy.special.softmax: parity unpinned by reference
 *                        tests beyond the row-sum property.
 *   orc_cpu_gemm_f32     cutile-examples/examples/persistent_gemm.rs:140-152.
 *   orc_gemm_bf16        the same loop over bf16-decoded inputs, bf16 (RNE) store.
 *   orc_fmha_ref_cpu     cutile-examples/examples/flash_attention_causal.rs:140-210.
 *   orc_mx_*             cutile-examples/examples/mxfp8.rs:25-64 (layout, formula),
 *                        cuda-core/src/dtype.rs:225-227 (0x38 = 1.0, 0x7F = 2^0);
 *                        codecs pinned against torch.float8_e4m3fn /
 *                        float8_e8m0fnu over all 256 codes.  The quantiser is not
 *                        in the reference (OCP MX v1.0 rule): parity unpinned.
 *   orc_add_rms_norm_f16, orc_qk_norm_f16      cutile-kernels/src/norms.rs (kernel bodies);
 *   orc_add_f16, orc_silu_mul_f16              cutile-kernels/src/pointwise.rs;
 *   orc_rope_seq_f16                           cutile-kernels/src/positional.rs:13-64;
 *   orc_kv_cache_update_f16                    cutile-kernels/src/kv_cache.rs:15-49, 58-97;
 *   orc_fmha_decode_gqa_split, orc_splitk_reduce_merge
 *                                              cutile-kernels/src/attention.rs:737-902, 917-1013.
 *                        The reference only compiles these kernels in its tests
 *                        (cutile-kernels/tests/smoke.rs), so they are pinned by the
 *                        mathematics: reduction to orc_rms_norm_f16, float64
 *                        definitions, scipy expit, complex rotation, float64 softmax
 *                        attention for any number of splits, per-split log-sum-exp,
 *                        merge closed forms, exact-copy checks: parity unpinned by
 *                        reference tests.
 *   orc_attention_decode_grouped_f16          cutile-kernels/src/experimental/attention.rs:385-846.
 *                        Only compiled by the reference's tests; pinned per split against
 *                        float64 softmax attention and log-sum-exp over the split's keys, by the
 *                        lse-weighted merge against attention over all keys, by poisoned keys
 *                        beyond s_kv, empty splits and a one-key split: parity unpinned by
 *                        reference tests.
 *   kvbm_stacked_to_contiguous / kvbm_contiguous_to_stacked (numpy, Python wrapper)
 *                        cutile-kernels/src/experimental/kvbm.rs:112-400: a transpose by the
 *                        reference's index maps; pinned element by element against the layouts'
 *                        definitions ([tokens, heads, head_dim] etc.) and by the round trip.
 *   orc_rms_norm_f32_example
 *                        cutile-examples/examples/rms_norm.rs:17-61 (the example only prints).
 *                        Pinned by float64 (the scale is the largest f32 not above the exact
 *                        square root), x = c -> out = sign(c) w, and agreement with
 *                        orc_rms_norm_f16 on f16-representable inputs up to the rounding mode:
 *                        parity unpinned by reference tests.
 *   orc_qk_norm_rope_kv_f16
 *                        cutile-kernels/src/experimental/fused_transformer.rs (kernel bodies).
 *                        Pinned by orc_rms_norm_f16 at position 0 (no rotation), by
 *                        orc_qk_norm_f16 -> orc_rope_seq_f16 -> orc_kv_cache_update_f16 (equal
 *                        up to the f16 rounding between the separate kernels), by a float64
 *                        evaluation, the norm-preserving rotation and exact copies of v;
 *                        the reference only compiles these kernels: parity unpinned by
 *                        reference tests.
 *   orc_argmax_blocks_f16, orc_lm_head_argmax_blocks_f16, orc_argmax_reduce_blocks_to_u32
 *                        cutile-kernels/src/argmax.rs (kernel bodies).  Pinned by numpy.argmax
 *                        (first index of the maximum) block by block and through the
 *                        composition blocks -> reduce = argmax of the whole vector, and by a
 *                        float64 matrix-vector product; the reference only compiles these
 *                        kernels: parity unpinned by reference tests.  embedding_batch_f16
 *                        and gather_row_f16 (embeddings.rs:21-41, pointwise.rs:86-99) are
 *                        numpy indexing in the Python wrapper.
 *   orc_attention_seq_ref
 *                        the five sequence-layout attention kernels of
 *                        cutile-kernels/src/attention.rs:21-726 (kernel bodies).  Pinned by
 *                        orc_fmha_ref_cpu (pinned above) where the two coincide (kv_len =
 *                        q_len, permuted layout), a float64 evaluation with an explicit mask,
 *                        row 0 = V[0], zero queries = mean of the visible V rows, empty key
 *                        range = 0.
 *                        The reference only compiles these kernels: parity unpinned by
 *                        reference tests.
 *   orc_nvfp4_*          cutile-examples/examples/nvfp4.rs:24-78 (layout, formula),
 *                        cuda-core/src/dtype.rs:60-99 (low nibble first), :228 (0x2 = 1.0).
 *                        Pinned by the reference's all-ones known answer (z = K), the
 *                        e2m1 value table, torch.float8_e4m3fn scales and a float64
 *                        evaluation of the dequantised product.  The quantiser is not in
 *                        the reference: parity unpinned.
 */
#ifndef CUTILE_ORACLE_H
#define CUTILE_ORACLE_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

int orc_num_threads(void);
void orc_set_num_threads(int n);

/* ---- scalar codecs ---------------------------------------------------- */
uint16_t orc_f32_to_f16(float f);   /* round-to-nearest-even, IEEE binary16 */
float orc_f16_to_f32(uint16_t h);
uint16_t orc_f32_to_bf16(float f);  /* round-to-nearest-even */
float orc_bf16_to_f32(uint16_t h);
float orc_e4m3fn_to_f32(uint8_t b); /* OCP e4m3fn: bias 7, no inf, S.1111.111 = NaN */
uint8_t orc_f32_to_e4m3fn(float f); /* RNE, saturating to +-448, NaN -> 0x7F */
float orc_e8m0_to_f32(uint8_t b);   /* 2^(b-127), 0xFF = NaN */

void orc_f32_to_f16_n(const float* src, uint16_t* dst, size_t n);
void orc_f16_to_f32_n(const uint16_t* src, float* dst, size_t n);
void orc_f32_to_bf16_n(const float* src, uint16_t* dst, size_t n);
void orc_bf16_to_f32_n(const uint16_t* src, float* dst, size_t n);

/* ---- seeded host inputs (SplitMix64 counter stream; same bytes feed the
 *      oracle and the GPU) ------------------------------------------------ */
void orc_fill_uniform_f32(float* dst, size_t n, uint64_t seed, float lo, float hi);
void orc_fill_normal_f32(float* dst, size_t n, uint64_t seed, float mean, float std);

/* ---- K1: saxpy / add --------------------------------------------------- */
void orc_saxpy_f32(size_t n, float a, const float* x, const float* y, float* z);
void orc_add_f32(size_t n, const float* x, const float* y, float* z);

/* ---- K2: RMSNorm (f16 IO, f32 math) ----------------------------------- */
/* block: chunk width of the kernel body's [1,BLOCK] accumulator tile; lane l
 * accumulates columns l, l+block, ... in order, lanes are then summed in
 * ascending order. */
void orc_rms_norm_f16(const uint16_t* x, const uint16_t* w, uint16_t* out, int64_t rows,
                      int64_t n, float eps, int64_t block);
/* independent float64 evaluation of the same formula (pins the f32 one) */
void orc_rms_norm_f16_f64(const uint16_t* x, const uint16_t* w, uint16_t* out, int64_t rows,
                          int64_t n, double eps);

/* ---- transformer-block kernels (f16 IO, f32 math) ----------------------- */
/* add_rms_norm_f16: cutile-kernels/src/norms.rs:68-136 */
void orc_add_rms_norm_f16(const uint16_t* residual, const uint16_t* x, const uint16_t* w,
                          uint16_t* out, uint16_t* residual_out, int64_t rows, int64_t n, float eps,
                          int64_t block);
/* qk_norm_f16: norms.rs:143-216; out has q_rows + k_rows rows */
void orc_qk_norm_f16(const uint16_t* q, const uint16_t* k, const uint16_t* qw, const uint16_t* kw,
                     uint16_t* out, int64_t q_rows, int64_t k_rows, int64_t n, float eps,
                     int64_t block);
/* add_2d_f16 / silu_mul_2d_f16: cutile-kernels/src/pointwise.rs:15-40, 46-78 */
void orc_add_f16(size_t n, const uint16_t* lhs, const uint16_t* rhs, uint16_t* out);
void orc_silu_mul_f16(size_t n, const uint16_t* gate, const uint16_t* up, uint16_t* out);
/* rope_seq_f16 (and its dynpos / qk forms): cutile-kernels/src/positional.rs:13-64 */
void orc_rope_seq_f16(const uint16_t* x, const float* inv_freq, uint16_t* out, int64_t seq,
                      int64_t heads, int64_t d, int32_t position_start);

/* kv_cache_update_seq(_dynpos)_f16: cutile-kernels/src/kv_cache.rs:15-49, 58-97 */
void orc_kv_cache_update_f16(const uint16_t* new_k, const uint16_t* new_v, uint16_t* k_cache,
                             uint16_t* v_cache, int64_t heads, int64_t d, int64_t max_seq,
                             int64_t position_start, int64_t seq_len);
/* the f32 example form of RMSNorm: cutile-examples/examples/rms_norm.rs:17-61 */
void orc_rms_norm_f32_example(const float* x, const float* w, float* out, int64_t rows, int64_t n, float eps,
                              int64_t block);
/* fused Q/K norm + RoPE + KV-cache update: cutile-kernels/src/experimental/fused_transformer.rs:22-345, 356-625 */
void orc_qk_norm_rope_kv_f16(const uint16_t* q, const uint16_t* k, const uint16_t* v, const uint16_t* qw,
                             const uint16_t* kw, const float* inv_freq, uint16_t* q_out, uint16_t* k_cache,
                             uint16_t* v_cache, float eps, int64_t position_start, int64_t seq_len, int64_t nq,
                             int64_t nkv, int64_t d, int64_t max_seq);
/* greedy sampling: cutile-kernels/src/argmax.rs:21-71, 88-158, 173-213 */
void orc_argmax_blocks_f16(const uint16_t* logits, int64_t n, int64_t block_size, int64_t len, float* block_max,
                           uint32_t* block_idx, int64_t num_blocks);
void orc_lm_head_argmax_blocks_f16(const uint16_t* weights, const uint16_t* hidden, int64_t rows, int64_t k,
                                   int64_t vocab_size, float* block_max, uint32_t* block_idx, int64_t num_blocks);
uint32_t orc_argmax_reduce_blocks_to_u32(const float* block_max, const uint32_t* block_idx, int64_t n,
                                         int64_t block_size, int64_t num_blocks);
/* the five sequence-layout attention kernels: cutile-kernels/src/attention.rs:21-726 */
void orc_attention_seq_ref(const float* q, const float* k, const float* v, float* out, int64_t q_len,
                           int64_t q_heads, int64_t kv_heads, int64_t max_seq, int64_t dsz, float qk_scale,
                           int64_t query_group_size, int64_t kv_len, int64_t query_start, int causal);
/* fmha_decode_gqa_split / splitk_reduce_merge: cutile-kernels/src/attention.rs:737-902, 917-1013 */
void orc_fmha_decode_gqa_split(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                               uint16_t* att_out, float* lse_out, int64_t kv_heads, int64_t group,
                               int64_t d, int64_t max_seq, int64_t bn, int64_t splits,
                               float qk_scale, int64_t input_pos);
void orc_attention_decode_grouped_f16(const uint16_t* q, const uint16_t* k, const uint16_t* v, uint16_t* att, float* lse,
                                      int64_t batch, int64_t heads, int64_t group, int64_t d, int64_t s_max,
                                      int64_t splits, int64_t tile_n, int64_t kv_len_per_split, float softmax_scale,
                                      int64_t s_kv);
void orc_splitk_reduce_merge(const uint16_t* att, const float* lse, uint16_t* out, int64_t kv_heads,
                             int64_t group, int64_t d, int64_t splits);

/* ---- K3: softmax over tiles [bm, bn] ---------------------------------- */
/* f32 IO.  Tile (i, j) covers rows i*bm.., cols j*bn..; every tile row is
 * normalised on its own (row softmax iff bn == n).  Columns beyond n read as 0
 * and are not stored (zero padded loads, masked stores). */
void orc_softmax_f32(const float* x, float* y, int64_t m, int64_t n, int64_t bm, int64_t bn);
/* f16 IO, f32 statistics */
void orc_softmax_f16(const uint16_t* x, uint16_t* y, int64_t m, int64_t n, int64_t bm, int64_t bn);

/* ---- K4: GEMM ---------------------------------------------------------- */
void orc_cpu_gemm_f32(const float* x, const float* y, float* z, int64_t m, int64_t n, int64_t k);
/* bf16 A[m,k], B[k,n] row-major, f32 accumulate in k order, bf16 C.  If
 * rows != NULL only the listed n_rows rows of C are computed into c (packed
 * [n_rows, n]). */
void orc_gemm_bf16(const uint16_t* a, const uint16_t* b, uint16_t* c, int64_t m, int64_t n,
                   int64_t k, const int64_t* rows, int64_t n_rows);
/* same with f32 result (no output rounding) */
void orc_gemm_bf16_f32out(const uint16_t* a, const uint16_t* b, float* c, int64_t m, int64_t n,
                          int64_t k, const int64_t* rows, int64_t n_rows);

/* ---- K5: FMHA ---------------------------------------------------------- */
/* q (b,h,m,d), k/v (b,hkv,m,d), out (b,h,m,d), all f32.  If rows != NULL only
 * the n_rows listed global query rows (index into b*h*m) are computed, packed
 * [n_rows, d]. */
void orc_fmha_ref_cpu(const float* q, const float* k, const float* v, float* out, int64_t bsz,
                      int64_t hsz, int64_t hkv, int64_t m, int64_t dsz, float qk_scale,
                      int64_t input_pos, int64_t query_group_size, int causal,
                      const int64_t* rows, int64_t n_rows);

/* ---- K6: MX block-scaled fp8 GEMM ------------------------------------- */
/* Quantise src[rows, k] (f32) per 32 contiguous K elements: scale byte e8m0,
 * data bytes e4m3fn.  scales is [rows, k/32]. */
void orc_mx_quantize_e4m3(const float* src, uint8_t* data, uint8_t* scales, int64_t rows,
                          int64_t k);
void orc_mx_dequantize_e4m3(const uint8_t* data, const uint8_t* scales, float* dst, int64_t rows,
                            int64_t k);
/* z[m,n] = alpha * sum_k x[i,k] sx[i,k/32] * y[j,k] sy[j,k/32]; y is stored
 * [n,k].  f32 accumulate in k order.  Row subset as for orc_gemm_bf16. */
void orc_mx_gemm_f32(const uint8_t* x, const uint8_t* y, const uint8_t* xs, const uint8_t* ys,
                     float* z, int64_t m, int64_t n, int64_t k, float alpha, const int64_t* rows,
                     int64_t n_rows);

/* ---- NVFP4 block-scaled GEMM (cutile-examples/examples/nvfp4.rs:24-78) -------------------- */
float orc_e2m1_to_f32(uint8_t nibble);   /* magnitudes 0, 0.5, 1, 1.5, 2, 3, 4, 6; bit 3 = sign */
uint8_t orc_f32_to_e2m1(float f);        /* nearest, ties to even mantissa, saturating */
/* scale per 16 K values = e4m3fn(amax / 6); data packed two per byte, even element in the low nibble */
void orc_nvfp4_quantize(const float* src, uint8_t* data, uint8_t* scales, int64_t rows, int64_t k);
void orc_nvfp4_dequantize(const uint8_t* data, const uint8_t* scales, float* dst, int64_t rows, int64_t k);
void orc_nvfp4_gemm_f32(const uint8_t* x, const uint8_t* y, const uint8_t* xs, const uint8_t* ys, float* z, int64_t m,
                        int64_t n, int64_t k, float alpha, const int64_t* rows, int64_t n_rows);

/* ---- device random fills (cutile_rng_*; the reference binds cuRAND: cuda-core/src/api.rs:214-293) ----------
 * Philox4x32-10 as published (Salmon et al., SC'11; multipliers 0xD2511F53 / 0xCD9E8D57, Weyl keys 0x9E3779B9 /
 * 0xBB67AE85), pinned by the Random123 known-answer vectors; the fills restate the layout of the fill kernels:
 * f32 element e = word e % 4 of block offset + e / 4, f64 element e = words 2(e % 2), 2(e % 2) + 1 of block
 * offset + e / 2, counter (block, 0), key = seed; uniform in [0, 1); normal by Box-Muller per pair.  The value
 * stream is this build's own (cuRAND's cannot be reproduced): parity against the reference's stream is unpinned,
 * the distribution is what the tests check. */
void orc_philox4x32_10(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4]);
void orc_rng_fill_f32(float* out, size_t n, uint64_t seed, uint64_t offset, int kind, float mean, float std);
void orc_rng_fill_f64(double* out, size_t n, uint64_t seed, uint64_t offset, int kind, double mean, double std);

#ifdef __cplusplus
}
#endif
#endif
