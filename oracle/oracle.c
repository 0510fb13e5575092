/*
 * CPU oracle for the tile-kernel path.  TEST INFRASTRUCTURE ONLY (see oracle.h):
 * the shipped library never links or calls this file.
 *
 * Build: gcc -O3 -ffp-contract=off -fopenmp (the Makefile beside this file).
 * -ffp-contract=off keeps `acc += a * b` a separate multiply and add, as the
 * reference's Rust loops are; the one fused operation is the explicit fmaf in
 * orc_saxpy_f32.
 */
#include "oracle.h"

#include <math.h>
#include <omp.h>
#include <stdlib.h>
#include <string.h>

int orc_num_threads(void) { return omp_get_max_threads(); }
void orc_set_num_threads(int n) {
  if (n > 0) omp_set_num_threads(n);
}

/* ------------------------------------------------------------------------ */
/* codecs                                                                    */
/* ------------------------------------------------------------------------ */
static inline uint32_t f32_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
static inline float bits_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}

uint16_t orc_f32_to_f16(float f) {
  uint32_t x = f32_bits(f);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t abs = x & 0x7fffffffu;
  if (abs >= 0x7f800000u) { /* inf / nan */
    return (uint16_t)(sign | 0x7c00u | (abs > 0x7f800000u ? 0x0200u | ((abs >> 13) & 0x3ffu) : 0));
  }
  if (abs >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (abs < 0x38800000u) { /* below the smallest normal half 2^-14: subnormal */
    if (abs < 0x33000000u) return (uint16_t)sign; /* < 2^-25 -> 0 (ties to even gives 0) */
    int e = (int)(abs >> 23);                      /* biased f32 exponent */
    uint32_t man = (abs & 0x7fffffu) | 0x800000u;  /* 24-bit significand */
    int shift = 126 - e;                           /* bits dropped to reach 2^-24 units */
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint16_t)(sign | q);
  }
  uint32_t e = (abs >> 23) - 112u; /* rebias 127 -> 15 */
  uint32_t man = abs & 0x7fffffu;
  uint32_t h = (e << 10) | (man >> 13);
  uint32_t rem = man & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++; /* carry may bump the exponent */
  return (uint16_t)(sign | h);
}

float orc_f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  if (e == 0) {
    if (man == 0) return bits_f32(sign);
    float v = (float)man * (1.0f / 16777216.0f); /* man * 2^-24 */
    return sign ? -v : v;
  }
  if (e == 31) return bits_f32(sign | 0x7f800000u | (man << 13));
  return bits_f32(sign | ((e + 112u) << 23) | (man << 13));
}

uint16_t orc_f32_to_bf16(float f) {
  uint32_t x = f32_bits(f);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x0040u); /* quiet nan */
  uint32_t lsb = (x >> 16) & 1u;
  x += 0x7fffu + lsb;
  return (uint16_t)(x >> 16);
}

float orc_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

float orc_e4m3fn_to_f32(uint8_t b) {
  int sign = b >> 7;
  int e = (b >> 3) & 0xf;
  int man = b & 7;
  float v;
  if (e == 15 && man == 7) return NAN;
  if (e == 0)
    v = ldexpf((float)man, -9); /* man/8 * 2^-6 */
  else
    v = ldexpf(1.0f + (float)man / 8.0f, e - 7);
  return sign ? -v : v;
}

uint8_t orc_f32_to_e4m3fn(float f) {
  if (isnan(f)) return 0x7f;
  uint8_t sign = signbit(f) ? 0x80 : 0;
  float a = fabsf(f);
  if (a >= 448.0f) return (uint8_t)(sign | 0x7e); /* saturate (also +-inf) */
  if (a < 0.015625f) {                              /* < 2^-6: subnormal grid, step 2^-9 */
    int q = (int)nearbyintf(a * 512.0f);            /* ties-to-even under the default mode */
    return (uint8_t)(sign | q);                     /* q == 8 is exactly code 0x08 = 2^-6 */
  }
  int e;
  float m = frexpf(a, &e); /* a = m * 2^e, m in [0.5, 1) */
  m *= 2.0f;
  e -= 1; /* m in [1, 2) */
  int q = (int)nearbyintf((m - 1.0f) * 8.0f);
  if (q == 8) {
    q = 0;
    e += 1;
  }
  if (e > 8 || (e == 8 && q == 7)) return (uint8_t)(sign | 0x7e);
  return (uint8_t)(sign | ((e + 7) << 3) | q);
}

float orc_e8m0_to_f32(uint8_t b) {
  if (b == 0xff) return NAN;
  return ldexpf(1.0f, (int)b - 127);
}

void orc_f32_to_f16_n(const float* src, uint16_t* dst, size_t n) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; i++) dst[i] = orc_f32_to_f16(src[i]);
}
void orc_f16_to_f32_n(const uint16_t* src, float* dst, size_t n) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; i++) dst[i] = orc_f16_to_f32(src[i]);
}
void orc_f32_to_bf16_n(const float* src, uint16_t* dst, size_t n) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; i++) dst[i] = orc_f32_to_bf16(src[i]);
}
void orc_bf16_to_f32_n(const uint16_t* src, float* dst, size_t n) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; i++) dst[i] = orc_bf16_to_f32(src[i]);
}

/* ------------------------------------------------------------------------ */
/* seeded inputs                                                             */
/* ------------------------------------------------------------------------ */
/* SplitMix64 evaluated as a counter-based generator: element i depends only on
 * (seed, i), so fills are identical for any thread count. */
static inline uint64_t splitmix64_at(uint64_t seed, uint64_t i) {
  uint64_t z = seed + (i + 1) * 0x9e3779b97f4a7c15ull;
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  return z ^ (z >> 31);
}
static inline double u01(uint64_t r) { return (double)(r >> 11) * (1.0 / 9007199254740992.0); }

void orc_fill_uniform_f32(float* dst, size_t n, uint64_t seed, float lo, float hi) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; i++) {
    double u = u01(splitmix64_at(seed, i));
    dst[i] = (float)((double)lo + ((double)hi - (double)lo) * u);
  }
}

void orc_fill_normal_f32(float* dst, size_t n, uint64_t seed, float mean, float std) {
  /* Box-Muller, one pair of uniforms per output element (cos branch). */
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; i++) {
    double u1 = u01(splitmix64_at(seed, 2 * i));
    double u2 = u01(splitmix64_at(seed, 2 * i + 1));
    if (u1 < 1e-300) u1 = 1e-300;
    double r = sqrt(-2.0 * log(u1));
    dst[i] = (float)((double)mean + (double)std * r * cos(6.283185307179586476925 * u2));
  }
}

/* ------------------------------------------------------------------------ */
/* K1                                                                        */
/* ------------------------------------------------------------------------ */
void orc_saxpy_f32(size_t n, float a, const float* x, const float* y, float* z) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; i++) z[i] = fmaf(a, x[i], y[i]);
}

void orc_add_f32(size_t n, const float* x, const float* y, float* z) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; i++) z[i] = x[i] + y[i];
}

/* ------------------------------------------------------------------------ */
/* K2                                                                        */
/* ------------------------------------------------------------------------ */
void orc_rms_norm_f16(const uint16_t* x, const uint16_t* w, uint16_t* out, int64_t rows,
                      int64_t n, float eps, int64_t block) {
  if (block <= 0 || block > n) block = n;
#pragma omp parallel
  {
    float* lanes = (float*)malloc(sizeof(float) * (size_t)block);
#pragma omp for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
      const uint16_t* xr = x + r * n;
      for (int64_t l = 0; l < block; l++) lanes[l] = 0.0f;
      for (int64_t j = 0; j < n; j += block) { /* rms = rms + tx * tx, per lane */
        int64_t lim = n - j < block ? n - j : block;
        for (int64_t l = 0; l < lim; l++) {
          float v = orc_f16_to_f32(xr[j + l]);
          lanes[l] = lanes[l] + v * v;
        }
      }
      float ss = 0.0f;
      for (int64_t l = 0; l < block; l++) ss += lanes[l];
      float inv = 1.0f / sqrtf(ss / (float)n + eps);
      for (int64_t j = 0; j < n; j++) {
        float v = orc_f16_to_f32(xr[j]);
        float o = v * inv * orc_f16_to_f32(w[j]); /* (x * inv) * w */
        out[r * n + j] = orc_f32_to_f16(o);
      }
    }
    free(lanes);
  }
}

void orc_rms_norm_f16_f64(const uint16_t* x, const uint16_t* w, uint16_t* out, int64_t rows,
                          int64_t n, double eps) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; r++) {
    const uint16_t* xr = x + r * n;
    double ss = 0.0;
    for (int64_t j = 0; j < n; j++) {
      double v = (double)orc_f16_to_f32(xr[j]);
      ss += v * v;
    }
    double inv = 1.0 / sqrt(ss / (double)n + eps);
    for (int64_t j = 0; j < n; j++) {
      double o = (double)orc_f16_to_f32(xr[j]) * inv * (double)orc_f16_to_f32(w[j]);
      out[r * n + j] = orc_f32_to_f16((float)o);
    }
  }
}

/* ------------------------------------------------------------------------ */
/* Transformer-block kernels (cutile-kernels/src/{norms,pointwise,positional}.rs) */
/* ------------------------------------------------------------------------ */
/* Lane-wise sum of squares as the kernel bodies do it: a [1, block] f32
 * accumulator tile, lane l takes columns l, l + block, ...; lanes summed in
 * ascending order (reduce_sum). */
static float lane_sum_of_squares(const float* row, int64_t n, int64_t block, float* lanes) {
  for (int64_t l = 0; l < block; l++) lanes[l] = 0.0f;
  for (int64_t j = 0; j < n; j += block) {
    int64_t lim = n - j < block ? n - j : block;
    for (int64_t l = 0; l < lim; l++) lanes[l] = lanes[l] + row[j + l] * row[j + l];
  }
  float ss = 0.0f;
  for (int64_t l = 0; l < block; l++) ss += lanes[l];
  return ss;
}

/* norms.rs:68-136: combined = f32(residual) + f32(x) (kept in f32); rms over combined;
 * out = f16(combined * inv * w); residual_out = f16(combined). */
void orc_add_rms_norm_f16(const uint16_t* residual, const uint16_t* x, const uint16_t* w,
                          uint16_t* out, uint16_t* residual_out, int64_t rows, int64_t n, float eps,
                          int64_t block) {
  if (block <= 0 || block > n) block = n;
#pragma omp parallel
  {
    float* lanes = (float*)malloc(sizeof(float) * (size_t)block);
    float* comb = (float*)malloc(sizeof(float) * (size_t)n);
#pragma omp for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
      for (int64_t j = 0; j < n; j++)
        comb[j] = orc_f16_to_f32(residual[r * n + j]) + orc_f16_to_f32(x[r * n + j]);
      float ss = lane_sum_of_squares(comb, n, block, lanes);
      float inv = 1.0f / sqrtf(ss / (float)n + eps);
      for (int64_t j = 0; j < n; j++) {
        out[r * n + j] = orc_f32_to_f16(comb[j] * inv * orc_f16_to_f32(w[j]));
        residual_out[r * n + j] = orc_f32_to_f16(comb[j]);
      }
    }
    free(lanes);
    free(comb);
  }
}

/* norms.rs:143-216: output row r < q_rows is RMSNorm(q[r]) with q_weight, row
 * q_rows + r is RMSNorm(k[r]) with k_weight. */
void orc_qk_norm_f16(const uint16_t* q, const uint16_t* k, const uint16_t* qw, const uint16_t* kw,
                     uint16_t* out, int64_t q_rows, int64_t k_rows, int64_t n, float eps,
                     int64_t block) {
  if (block <= 0 || block > n) block = n;
#pragma omp parallel
  {
    float* lanes = (float*)malloc(sizeof(float) * (size_t)block);
    float* row = (float*)malloc(sizeof(float) * (size_t)n);
#pragma omp for schedule(static)
    for (int64_t r = 0; r < q_rows + k_rows; r++) {
      const int is_q = r < q_rows;
      const uint16_t* src = is_q ? q + r * n : k + (r - q_rows) * n;
      const uint16_t* wt = is_q ? qw : kw;
      for (int64_t j = 0; j < n; j++) row[j] = orc_f16_to_f32(src[j]);
      float ss = lane_sum_of_squares(row, n, block, lanes);
      float inv = 1.0f / sqrtf(ss / (float)n + eps);
      for (int64_t j = 0; j < n; j++) out[r * n + j] = orc_f32_to_f16(row[j] * inv * orc_f16_to_f32(wt[j]));
    }
    free(lanes);
    free(row);
  }
}

/* pointwise.rs:15-40: f16 + f16 (one rounding: the f32 sum of two f16 values is exact). */
void orc_add_f16(size_t n, const uint16_t* lhs, const uint16_t* rhs, uint16_t* out) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; i++) out[i] = orc_f32_to_f16(orc_f16_to_f32(lhs[i]) + orc_f16_to_f32(rhs[i]));
}

/* pointwise.rs:46-78: sigmoid = 1 / (1 + exp(0 - gate)); y = f16(sigmoid * gate * up), f32 math. */
void orc_silu_mul_f16(size_t n, const uint16_t* gate, const uint16_t* up, uint16_t* out) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; i++) {
    float g = orc_f16_to_f32(gate[i]), u = orc_f16_to_f32(up[i]);
    float sig = 1.0f / (1.0f + expf(0.0f - g));
    out[i] = orc_f32_to_f16(sig * g * u);
  }
}

/* positional.rs:13-64 (rope_seq_f16; the dynpos forms differ only in where the
 * start position comes from): x [seq, heads, d], halves lo = [..., :d/2], hi =
 * [..., d/2:]; theta = f32(position_start + s) * inv_freq[i];
 * y_lo = x_lo cos - x_hi sin; y_hi = x_hi cos + x_lo sin. */
void orc_rope_seq_f16(const uint16_t* x, const float* inv_freq, uint16_t* out, int64_t seq,
                      int64_t heads, int64_t d, int32_t position_start) {
  const int64_t half = d / 2;
#pragma omp parallel for schedule(static)
  for (int64_t s = 0; s < seq; s++) {
    const float pos = (float)(position_start + (int32_t)s);
    for (int64_t h = 0; h < heads; h++) {
      const uint16_t* xr = x + (s * heads + h) * d;
      uint16_t* orow = out + (s * heads + h) * d;
      for (int64_t i = 0; i < half; i++) {
        float theta = pos * inv_freq[i];
        float c = cosf(theta), sn = sinf(theta);
        float lo = orc_f16_to_f32(xr[i]), hi = orc_f16_to_f32(xr[half + i]);
        orow[i] = orc_f32_to_f16(lo * c - hi * sn);
        orow[half + i] = orc_f32_to_f16(hi * c + lo * sn);
      }
    }
  }
}

/* ------------------------------------------------------------------------ */
/* KV cache update and decode attention (cutile-kernels/src/{kv_cache,attention}.rs) */
/* ------------------------------------------------------------------------ */
/* kv_cache.rs:15-49 and :58-97: cache[h, position_start + s, :] = new[s, h, :] for s < seq_len.
 * new_* are [seq, heads, d]; caches are [heads, max_seq, d]. */
void orc_kv_cache_update_f16(const uint16_t* new_k, const uint16_t* new_v, uint16_t* k_cache,
                             uint16_t* v_cache, int64_t heads, int64_t d, int64_t max_seq,
                             int64_t position_start, int64_t seq_len) {
  for (int64_t s = 0; s < seq_len; s++)
    for (int64_t h = 0; h < heads; h++) {
      const int64_t src = (s * heads + h) * d, dst = (h * max_seq + position_start + s) * d;
      memcpy(k_cache + dst, new_k + src, (size_t)d * 2);
      memcpy(v_cache + dst, new_v + src, (size_t)d * 2);
    }
}

/* attention.rs:737-902 fmha_decode_gqa_split, restated tile by tile.
 * q [kv_heads, group, d]; k, v [kv_heads, max_seq, d]; s_kv = input_pos + 1 keys are visible.
 * att_out [kv_heads, splits * group, d] (f16), lse_out [kv_heads, splits * group] (f32, log2 domain).
 * Per split: KV tiles [start_tile, end_tile) of bn rows; running max m (init -1e30), per-lane
 * sums l[bn][group] (init 1), acc[d][group]; only the last tile of the sequence is masked
 * (+ -1e30 before scaling); p is rounded to f16 for the P·V product; att = acc / max(sum l, 1e-8);
 * lse = m + log2(max(sum l, 1e-8)). */
void orc_fmha_decode_gqa_split(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                               uint16_t* att_out, float* lse_out, int64_t kv_heads, int64_t group,
                               int64_t d, int64_t max_seq, int64_t bn, int64_t splits,
                               float qk_scale, int64_t input_pos) {
  const int64_t s_kv = input_pos + 1;
  const int64_t tiles = (s_kv + bn - 1) / bn;
  const int64_t per_split = (tiles + splits - 1) / splits;
  const float scale_log2 = qk_scale / logf(2.0f);
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t h = 0; h < kv_heads; h++)
    for (int64_t sp = 0; sp < splits; sp++) {
      int64_t start = sp * per_split, end = start + per_split;
      if (end > tiles) end = tiles;
      float* m = (float*)malloc(sizeof(float) * (size_t)group);
      float* l = (float*)malloc(sizeof(float) * (size_t)(bn * group));
      float* acc = (float*)calloc((size_t)(d * group), sizeof(float));
      float* qk = (float*)malloc(sizeof(float) * (size_t)(bn * group));
      for (int64_t g = 0; g < group; g++) m[g] = -1.0e30f;
      for (int64_t i = 0; i < bn * group; i++) l[i] = 1.0f;
      for (int64_t j = start; j < end; j++) {
        for (int64_t n = 0; n < bn; n++) {
          const int64_t row = j * bn + n;
          for (int64_t g = 0; g < group; g++) {
            float a = 0.0f;
            if (row < max_seq)
              for (int64_t c = 0; c < d; c++)
                a += orc_f16_to_f32(k[(h * max_seq + row) * d + c]) * orc_f16_to_f32(q[(h * group + g) * d + c]);
            if (j == tiles - 1) a = a + (row < s_kv ? 0.0f : -1.0e30f);
            qk[n * group + g] = a * scale_log2;
          }
        }
        for (int64_t g = 0; g < group; g++) {
          float mx = -INFINITY;
          for (int64_t n = 0; n < bn; n++) mx = fmaxf(mx, qk[n * group + g]);
          const float m_new = fmaxf(m[g], mx);
          const float alpha = exp2f(m[g] - m_new);
          for (int64_t c = 0; c < d; c++) acc[c * group + g] *= alpha;
          for (int64_t n = 0; n < bn; n++) {
            const float p = exp2f(qk[n * group + g] - m_new);
            l[n * group + g] = l[n * group + g] * alpha + p;
            const float ph = orc_f16_to_f32(orc_f32_to_f16(p));
            const int64_t row = j * bn + n;
            if (row < max_seq && ph != 0.0f)
              for (int64_t c = 0; c < d; c++)
                acc[c * group + g] += orc_f16_to_f32(v[(h * max_seq + row) * d + c]) * ph;
          }
          m[g] = m_new;
        }
      }
      for (int64_t g = 0; g < group; g++) {
        float ls = 0.0f;
        for (int64_t n = 0; n < bn; n++) ls += l[n * group + g];
        const float safe = fmaxf(ls, 1.0e-8f);
        for (int64_t c = 0; c < d; c++)
          att_out[((h * splits + sp) * group + g) * d + c] = orc_f32_to_f16(acc[c * group + g] / safe);
        lse_out[(h * splits + sp) * group + g] = m[g] + log2f(safe);
      }
      free(m); free(l); free(acc); free(qk);
    }
}

/* cutile-kernels/src/experimental/attention.rs:385-846 attention_decode_kernel_grouped, contiguous tensors:
 * q [b, h, g, d]; k, v [b, h, s_max, d]; att [b, h, g, splits, d]; lse [b, h, g, splits].
 * Split t: start = t * kv_len_per_split, end = min(start + kv_len_per_split, s_kv) (629-633); without keys it
 * yields acc = 0, l = 1 per lane, m = -inf (775-780).  Otherwise cdiv(kv_len_per_split, tile_n) tiles from tile
 * start / tile_n on (638-641, 685-687): qk = K . Q^T (703), rows at or beyond s_kv replaced by -1e6 when the tile
 * crosses s_kv (705-725), scaled by softmax_scale * 1.44269502 (603-606, 729-730), online softmax in base 2 with
 * l kept per (row of the tile, head) (732-760), acc *= alpha, acc += V^T . f16(p) (762-769); then
 * att = f16(acc / sum_rows l), lse = m + log2(sum l) (786-807).  Tile rows beyond s_max read as zeros. */
void orc_attention_decode_grouped_f16(const uint16_t* q, const uint16_t* k, const uint16_t* v, uint16_t* att, float* lse,
                                      int64_t batch, int64_t heads, int64_t group, int64_t d, int64_t s_max,
                                      int64_t splits, int64_t tile_n, int64_t kv_len_per_split, float softmax_scale,
                                      int64_t s_kv) {
  const float qk_scale = softmax_scale * 1.44269502f;
  const int64_t num_tiles = (kv_len_per_split + tile_n - 1) / tile_n;
#pragma omp parallel for collapse(3) schedule(static)
  for (int64_t b = 0; b < batch; b++)
    for (int64_t h = 0; h < heads; h++)
      for (int64_t sp = 0; sp < splits; sp++) {
        const int64_t bh = b * heads + h;
        const int64_t start = sp * kv_len_per_split;
        const int64_t end = start + kv_len_per_split < s_kv ? start + kv_len_per_split : s_kv;
        float* m = (float*)malloc(sizeof(float) * (size_t)group);
        float* l = (float*)malloc(sizeof(float) * (size_t)(tile_n * group));
        float* acc = (float*)calloc((size_t)(d * group), sizeof(float));
        float* qk = (float*)malloc(sizeof(float) * (size_t)(tile_n * group));
        for (int64_t g = 0; g < group; g++) m[g] = -INFINITY;
        for (int64_t i = 0; i < tile_n * group; i++) l[i] = 1.0f;
        if (end > start) {
          const int64_t start_tile = start / tile_n;
          for (int64_t idx = 0; idx < num_tiles; idx++) {
            const int64_t curr_n = (start_tile + idx) * tile_n;
            const int boundary = curr_n + tile_n > s_kv;
            for (int64_t n = 0; n < tile_n; n++) {
              const int64_t row = curr_n + n;
              for (int64_t g = 0; g < group; g++) {
                float a = 0.0f;
                if (row < s_max)
                  for (int64_t c = 0; c < d; c++)
                    a += orc_f16_to_f32(k[(bh * s_max + row) * d + c]) * orc_f16_to_f32(q[(bh * group + g) * d + c]);
                if (boundary && !(row < s_kv)) a = -1000000.0f;
                qk[n * group + g] = a * qk_scale;
              }
            }
            for (int64_t g = 0; g < group; g++) {
              float mx = -INFINITY;
              for (int64_t n = 0; n < tile_n; n++) mx = fmaxf(mx, qk[n * group + g]);
              const float m_new = fmaxf(m[g], mx);
              const float alpha = exp2f(m[g] - m_new);
              for (int64_t c = 0; c < d; c++) acc[c * group + g] *= alpha;
              for (int64_t n = 0; n < tile_n; n++) {
                const float p = exp2f(qk[n * group + g] - m_new);
                l[n * group + g] = fmaf(l[n * group + g], alpha, p);
                const float ph = orc_f16_to_f32(orc_f32_to_f16(p));
                const int64_t row = curr_n + n;
                if (row < s_max && ph != 0.0f)
                  for (int64_t c = 0; c < d; c++) acc[c * group + g] += orc_f16_to_f32(v[(bh * s_max + row) * d + c]) * ph;
              }
              m[g] = m_new;
            }
          }
        }
        for (int64_t g = 0; g < group; g++) {
          float ls = 0.0f;
          for (int64_t n = 0; n < tile_n; n++) ls += l[n * group + g];
          for (int64_t c = 0; c < d; c++) att[(((bh * group) + g) * splits + sp) * d + c] = orc_f32_to_f16(acc[c * group + g] / ls);
          lse[(bh * group + g) * splits + sp] = m[g] + log2f(ls);
        }
        free(m); free(l); free(acc); free(qk);
      }
}

/* attention.rs:917-1013 splitk_reduce_merge: weights = exp2(lse - max) / max(sum, 1e-8) over
 * the splits; out[h, g, :] = sum_s weights[g, s] * att[h, s, g, :], f16. */
void orc_splitk_reduce_merge(const uint16_t* att, const float* lse, uint16_t* out, int64_t kv_heads,
                             int64_t group, int64_t d, int64_t splits) {
#pragma omp parallel for schedule(static)
  for (int64_t h = 0; h < kv_heads; h++)
    for (int64_t g = 0; g < group; g++) {
      float mx = -INFINITY, sum = 0.0f;
      for (int64_t s = 0; s < splits; s++) mx = fmaxf(mx, lse[(h * splits + s) * group + g]);
      for (int64_t s = 0; s < splits; s++) sum += exp2f(lse[(h * splits + s) * group + g] - mx);
      const float safe = fmaxf(sum, 1.0e-8f);
      for (int64_t c = 0; c < d; c++) {
        float o = 0.0f;
        for (int64_t s = 0; s < splits; s++) {
          const float w = exp2f(lse[(h * splits + s) * group + g] - mx) / safe;
          o += orc_f16_to_f32(att[((h * splits + s) * group + g) * d + c]) * w;
        }
        out[(h * group + g) * d + c] = orc_f32_to_f16(o);
      }
    }
}

/* ------------------------------------------------------------------------ */
/* K3                                                                        */
/* ------------------------------------------------------------------------ */
static void softmax_tile_row(const float* xin, float* yout, int64_t valid, int64_t bn) {
  /* the tile row has bn lanes; lanes >= valid were zero padded on load */
  float mx = -INFINITY;
  for (int64_t j = 0; j < valid; j++) mx = fmaxf(mx, xin[j]);
  if (valid < bn) mx = fmaxf(mx, 0.0f);
  float den = 0.0f;
  for (int64_t j = 0; j < valid; j++) {
    yout[j] = expf(xin[j] - mx);
    den += yout[j];
  }
  if (valid < bn) den += (float)(bn - valid) * expf(0.0f - mx);
  for (int64_t j = 0; j < valid; j++) yout[j] = yout[j] / den;
}

void orc_softmax_f32(const float* x, float* y, int64_t m, int64_t n, int64_t bm, int64_t bn) {
  (void)bm; /* rows are independent; bm only shapes the launch grid */
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < m; r++) {
    for (int64_t c0 = 0; c0 < n; c0 += bn) {
      int64_t valid = n - c0 < bn ? n - c0 : bn;
      softmax_tile_row(x + r * n + c0, y + r * n + c0, valid, bn);
    }
  }
}

void orc_softmax_f16(const uint16_t* x, uint16_t* y, int64_t m, int64_t n, int64_t bm, int64_t bn) {
  (void)bm;
#pragma omp parallel
  {
    float* xin = (float*)malloc(sizeof(float) * (size_t)bn * 2);
    float* yout = xin + bn;
#pragma omp for schedule(static)
    for (int64_t r = 0; r < m; r++) {
      for (int64_t c0 = 0; c0 < n; c0 += bn) {
        int64_t valid = n - c0 < bn ? n - c0 : bn;
        for (int64_t j = 0; j < valid; j++) xin[j] = orc_f16_to_f32(x[r * n + c0 + j]);
        softmax_tile_row(xin, yout, valid, bn);
        for (int64_t j = 0; j < valid; j++) y[r * n + c0 + j] = orc_f32_to_f16(yout[j]);
      }
    }
    free(xin);
  }
}

/* ------------------------------------------------------------------------ */
/* K4                                                                        */
/* ------------------------------------------------------------------------ */
void orc_cpu_gemm_f32(const float* x, const float* y, float* z, int64_t m, int64_t n, int64_t k) {
  /* acc += x[row*k+inner] * y[inner*n+col] with inner ascending.  The loops are
   * ordered row / inner / col so the compiler can vectorise across col; every
   * output element still sees the same sequence of operations. */
#pragma omp parallel for schedule(static)
  for (int64_t row = 0; row < m; row++) {
    float* acc = z + row * n;
    for (int64_t col = 0; col < n; col++) acc[col] = 0.0f;
    for (int64_t inner = 0; inner < k; inner++) {
      float xv = x[row * k + inner];
      const float* yr = y + inner * n;
      for (int64_t col = 0; col < n; col++) acc[col] += xv * yr[col];
    }
  }
}

void orc_gemm_bf16_f32out(const uint16_t* a, const uint16_t* b, float* c, int64_t m, int64_t n,
                          int64_t k, const int64_t* rows, int64_t n_rows) {
  int64_t count = rows ? n_rows : m;
#pragma omp parallel for schedule(dynamic, 1)
  for (int64_t ri = 0; ri < count; ri++) {
    int64_t row = rows ? rows[ri] : ri;
    float* acc = c + ri * n;
    for (int64_t col = 0; col < n; col++) acc[col] = 0.0f;
    for (int64_t inner = 0; inner < k; inner++) {
      float xv = orc_bf16_to_f32(a[row * k + inner]);
      const uint16_t* br = b + inner * n;
      for (int64_t col = 0; col < n; col++) acc[col] += xv * orc_bf16_to_f32(br[col]);
    }
  }
}

void orc_gemm_bf16(const uint16_t* a, const uint16_t* b, uint16_t* c, int64_t m, int64_t n,
                   int64_t k, const int64_t* rows, int64_t n_rows) {
  int64_t count = rows ? n_rows : m;
  float* tmp = (float*)malloc(sizeof(float) * (size_t)count * (size_t)n);
  orc_gemm_bf16_f32out(a, b, tmp, m, n, k, rows, n_rows);
  orc_f32_to_bf16_n(tmp, c, (size_t)count * (size_t)n);
  free(tmp);
}

/* ------------------------------------------------------------------------ */
/* K5                                                                        */
/* ------------------------------------------------------------------------ */
static inline int64_t idx4(int64_t a, int64_t b, int64_t c, int64_t d, int64_t hsz, int64_t m,
                           int64_t dsz) {
  return (((a * hsz + b) * m + c) * dsz) + d;
}

void orc_fmha_ref_cpu(const float* q, const float* k, const float* v, float* out, int64_t bsz,
                      int64_t hsz, int64_t hkv, int64_t m, int64_t dsz, float qk_scale,
                      int64_t input_pos, int64_t query_group_size, int causal,
                      const int64_t* rows, int64_t n_rows) {
  int64_t count = rows ? n_rows : bsz * hsz * m;
#pragma omp parallel
  {
    float* scores = (float*)malloc(sizeof(float) * (size_t)m);
#pragma omp for schedule(dynamic, 16)
    for (int64_t ri = 0; ri < count; ri++) {
      int64_t g = rows ? rows[ri] : ri;
      int64_t i = g % m;
      int64_t h = (g / m) % hsz;
      int64_t b = g / (m * hsz);
      int64_t kv_h = h / query_group_size;
      float max_logit = -INFINITY;
      for (int64_t j = 0; j < m; j++) {
        if (causal && j > i + input_pos) {
          scores[j] = -INFINITY;
          continue;
        }
        float dot = 0.0f;
        for (int64_t dd = 0; dd < dsz; dd++)
          dot += q[idx4(b, h, i, dd, hsz, m, dsz)] * k[idx4(b, kv_h, j, dd, hkv, m, dsz)];
        scores[j] = dot * qk_scale;
        max_logit = fmaxf(max_logit, scores[j]);
      }
      float denom = 0.0f;
      for (int64_t j = 0; j < m; j++) {
        scores[j] = expf(scores[j] - max_logit);
        denom += scores[j];
      }
      float* o = rows ? out + ri * dsz : out + idx4(b, h, i, 0, hsz, m, dsz);
      for (int64_t dd = 0; dd < dsz; dd++) {
        float val = 0.0f;
        for (int64_t j = 0; j < m; j++) {
          float p = scores[j] / denom;
          val += p * v[idx4(b, kv_h, j, dd, hkv, m, dsz)];
        }
        o[dd] = val;
      }
    }
    free(scores);
  }
}

/* The sequence-layout attention kernels of cutile-kernels/src/attention.rs: flash_attn_causal_seq_f16 (:21-116) and
 * its dynpos form (:128-231), fmha_prefill_causal (:242-391), fmha_prefill_gqa (:408-587), fmha_causal (:598-726).
 * q, out [q_len, q_heads, d]; k, v [kv_heads, max_seq, d].  Query i stands at position query_start + i (:44-49) and
 * key j counts iff j < kv_len and (not causal or position >= j) (:83-88); kv head = q head / query_group_size (:34);
 * scores are q.k * qk_scale, weights exp(score - max) / max(sum, 1e-8) (:90-110), so a query without any key gets zeros.
 * The kernels stream the keys in tiles with a running maximum; evaluated here over the whole row at once, which is
 * the same function. */
void orc_attention_seq_ref(const float* q, const float* k, const float* v, float* out, int64_t q_len,
                           int64_t q_heads, int64_t kv_heads, int64_t max_seq, int64_t dsz, float qk_scale,
                           int64_t query_group_size, int64_t kv_len, int64_t query_start, int causal) {
  (void)kv_heads;
  if (kv_len > max_seq) kv_len = max_seq;
#pragma omp parallel
  {
    float* scores = (float*)malloc(sizeof(float) * (size_t)(kv_len > 0 ? kv_len : 1));
#pragma omp for schedule(dynamic, 16)
    for (int64_t g = 0; g < q_len * q_heads; g++) {
      int64_t i = g / q_heads, h = g % q_heads;
      int64_t kv_h = h / query_group_size;
      const float* qrow = q + (i * q_heads + h) * dsz;
      const float* kb = k + kv_h * max_seq * dsz;
      const float* vb = v + kv_h * max_seq * dsz;
      float* o = out + (i * q_heads + h) * dsz;
      int64_t n = kv_len;
      if (causal && query_start + i + 1 < n) n = query_start + i + 1;   /* keys 0 .. position */
      float max_logit = -INFINITY;
      for (int64_t j = 0; j < n; j++) {
        float dot = 0.0f;
        for (int64_t dd = 0; dd < dsz; dd++) dot += qrow[dd] * kb[j * dsz + dd];
        scores[j] = dot * qk_scale;
        max_logit = fmaxf(max_logit, scores[j]);
      }
      float denom = 0.0f;
      for (int64_t j = 0; j < n; j++) {
        scores[j] = expf(scores[j] - max_logit);
        denom += scores[j];
      }
      denom = fmaxf(denom, 1.0e-8f);
      for (int64_t dd = 0; dd < dsz; dd++) {
        float val = 0.0f;
        for (int64_t j = 0; j < n; j++) val += scores[j] * vb[j * dsz + dd];
        o[dd] = val / denom;
      }
    }
    free(scores);
  }
}

/* ------------------------------------------------------------------------ */
/* K6                                                                        */
/* ------------------------------------------------------------------------ */
void orc_mx_quantize_e4m3(const float* src, uint8_t* data, uint8_t* scales, int64_t rows,
                          int64_t k) {
  int64_t kb = k / 32;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; r++) {
    for (int64_t blk = 0; blk < kb; blk++) {
      const float* s = src + r * k + blk * 32;
      float amax = 0.0f;
      for (int j = 0; j < 32; j++) amax = fmaxf(amax, fabsf(s[j]));
      /* OCP MX v1.0: shared exponent = floor(log2(amax)) - emax(e4m3 = 8),
       * clamped to the e8m0 range; an all-zero block takes scale 2^0. */
      int se = 0;
      if (amax > 0.0f && isfinite(amax)) {
        int e;
        frexpf(amax, &e); /* amax = f * 2^e, f in [0.5,1) -> floor(log2) = e-1 */
        se = (e - 1) - 8;
        if (se < -127) se = -127;
        if (se > 127) se = 127;
      }
      scales[r * kb + blk] = (uint8_t)(se + 127);
      float inv = ldexpf(1.0f, -se);
      for (int j = 0; j < 32; j++) data[r * k + blk * 32 + j] = orc_f32_to_e4m3fn(s[j] * inv);
    }
  }
}

void orc_mx_dequantize_e4m3(const uint8_t* data, const uint8_t* scales, float* dst, int64_t rows,
                            int64_t k) {
  int64_t kb = k / 32;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; r++)
    for (int64_t j = 0; j < k; j++)
      dst[r * k + j] = orc_e4m3fn_to_f32(data[r * k + j]) * orc_e8m0_to_f32(scales[r * kb + j / 32]);
}

void orc_mx_gemm_f32(const uint8_t* x, const uint8_t* y, const uint8_t* xs, const uint8_t* ys,
                     float* z, int64_t m, int64_t n, int64_t k, float alpha, const int64_t* rows,
                     int64_t n_rows) {
  int64_t count = rows ? n_rows : m;
  int64_t kb = k / 32;
  float lut[256];
  for (int i = 0; i < 256; i++) lut[i] = orc_e4m3fn_to_f32((uint8_t)i);
#pragma omp parallel
  {
    float* xrow = (float*)malloc(sizeof(float) * (size_t)k);
#pragma omp for schedule(dynamic, 1)
    for (int64_t ri = 0; ri < count; ri++) {
      int64_t row = rows ? rows[ri] : ri;
      for (int64_t j = 0; j < k; j++)
        xrow[j] = lut[x[row * k + j]] * orc_e8m0_to_f32(xs[row * kb + j / 32]);
      for (int64_t col = 0; col < n; col++) {
        const uint8_t* yr = y + col * k;
        float acc = 0.0f;
        for (int64_t blk = 0; blk < kb; blk++) {
          float sy = orc_e8m0_to_f32(ys[col * kb + blk]);
          for (int j = 0; j < 32; j++) acc += xrow[blk * 32 + j] * (lut[yr[blk * 32 + j]] * sy);
        }
        z[ri * n + col] = alpha * acc;
      }
    }
    free(xrow);
  }
}

/* ------------------------------------------------------------------------ */
/* NVFP4 block-scaled GEMM (cutile-examples/examples/nvfp4.rs:24-78)         */
/* ------------------------------------------------------------------------ */
/* e2m1: sign, two exponent bits (bias 1), one mantissa bit; no inf, no NaN.
 * Magnitudes 0, 0.5, 1, 1.5, 2, 3, 4, 6 (OCP MX v1.0 table 5; dtype.rs:225-229 uses
 * nibble 0x2 as one()). */
float orc_e2m1_to_f32(uint8_t nibble) {
  int e = (nibble >> 1) & 3, m = nibble & 1;
  float v = e == 0 ? 0.5f * (float)m : ldexpf(1.0f + 0.5f * (float)m, e - 1);
  return (nibble & 8) ? -v : v;
}

/* round to nearest representable magnitude, ties to the even mantissa, saturating at 6 */
uint8_t orc_f32_to_e2m1(float f) {
  uint8_t sign = signbit(f) ? 8 : 0;
  float a = fabsf(f);
  if (!(a == a)) return (uint8_t)(sign | 7); /* NaN has no encoding: saturate */
  uint8_t best = 0;
  float best_d = INFINITY;
  for (uint8_t c = 0; c < 8; c++) {
    float d = fabsf(a - orc_e2m1_to_f32(c));
    if (d < best_d || (d == best_d && (c & 1) == 0)) {
      best = c;
      best_d = d;
    }
  }
  return (uint8_t)(sign | best);
}

/* Quantise src[rows, k] (f32), one e4m3fn scale per 16 contiguous K values: scale =
 * e4m3(amax / 6) (the largest magnitude maps to the largest e2m1 value), data = e2m1(src /
 * scale), packed two per byte with the even element in the low nibble.  Not in the
 * reference (its example fills ones): used to build test operands. */
void orc_nvfp4_quantize(const float* src, uint8_t* data, uint8_t* scales, int64_t rows, int64_t k) {
  int64_t kb = k / 16;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; r++)
    for (int64_t blk = 0; blk < kb; blk++) {
      const float* s = src + r * k + blk * 16;
      float amax = 0.0f;
      for (int j = 0; j < 16; j++) amax = fmaxf(amax, fabsf(s[j]));
      uint8_t sc = orc_f32_to_e4m3fn(amax / 6.0f);
      float sf = orc_e4m3fn_to_f32(sc);
      scales[r * kb + blk] = sc;
      for (int j = 0; j < 16; j += 2) {
        uint8_t lo = sf > 0.0f ? orc_f32_to_e2m1(s[j] / sf) : 0, hi = sf > 0.0f ? orc_f32_to_e2m1(s[j + 1] / sf) : 0;
        data[r * (k / 2) + blk * 8 + j / 2] = (uint8_t)(lo | (hi << 4));
      }
    }
}

void orc_nvfp4_dequantize(const uint8_t* data, const uint8_t* scales, float* dst, int64_t rows, int64_t k) {
  int64_t kb = k / 16;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; r++)
    for (int64_t j = 0; j < k; j++) {
      uint8_t byte = data[r * (k / 2) + j / 2];
      dst[r * k + j] = orc_e2m1_to_f32((j & 1) ? (uint8_t)(byte >> 4) : (uint8_t)(byte & 15)) * orc_e4m3fn_to_f32(scales[r * kb + j / 16]);
    }
}

/* z[m,n] = alpha * sum_k (x[i,k] sx[i,k/16]) * (y[j,k] sy[j,k/16]); x [m,k/2], y [n,k/2] packed,
 * f32 accumulate in k order.  Row subset as for orc_gemm_bf16. */
void orc_nvfp4_gemm_f32(const uint8_t* x, const uint8_t* y, const uint8_t* xs, const uint8_t* ys, float* z, int64_t m,
                        int64_t n, int64_t k, float alpha, const int64_t* rows, int64_t n_rows) {
  int64_t count = rows ? n_rows : m;
  float* yd = (float*)malloc(sizeof(float) * (size_t)n * (size_t)k);
  orc_nvfp4_dequantize(y, ys, yd, n, k);
#pragma omp parallel
  {
    float* xrow = (float*)malloc(sizeof(float) * (size_t)k);
#pragma omp for schedule(dynamic, 1)
    for (int64_t ri = 0; ri < count; ri++) {
      int64_t row = rows ? rows[ri] : ri;
      orc_nvfp4_dequantize(x + row * (k / 2), xs + row * (k / 16), xrow, 1, k);
      for (int64_t col = 0; col < n; col++) {
        const float* yr = yd + col * k;
        float acc = 0.0f;
        for (int64_t j = 0; j < k; j++) acc += xrow[j] * yr[j];
        z[ri * n + col] = alpha * acc;
      }
    }
    free(xrow);
  }
  free(yd);
}

/* ---- greedy sampling (cutile-kernels/src/argmax.rs) ------------------------------------------------------ */
static void block_winner(const float* vals, const int64_t* idx, int64_t n, float* out_max, uint32_t* out_idx,
                         int64_t no_candidate) {
  /* reduce_max, then reduce_min over the indices of the positions that attain it (argmax.rs:45-55) */
  float mx = vals[0];
  for (int64_t i = 1; i < n; i++) mx = fmaxf(mx, vals[i]);
  int64_t best = INT64_MAX;
  for (int64_t i = 0; i < n; i++) {
    int64_t candidate = vals[i] == mx ? idx[i] : no_candidate;   /* select(is_max, indices, invalid_idx) */
    if (candidate < best) best = candidate;
  }
  *out_max = mx;
  *out_idx = (uint32_t)(int32_t)best;
}

/* argmax_blocks_f16<BLOCK_SIZE> (argmax.rs:21-71): block b covers logits[b*BLOCK_SIZE ..]; positions beyond the
 * tensor load as zero (padded tile load), positions >= len count as -1e30 (:36-43); the index is the smallest one
 * attaining the maximum, len + 1 if none (:47-55). */
void orc_argmax_blocks_f16(const uint16_t* logits, int64_t n, int64_t block_size, int64_t len, float* block_max,
                           uint32_t* block_idx, int64_t num_blocks) {
  float* vals = (float*)malloc(sizeof(float) * (size_t)block_size);
  int64_t* idx = (int64_t*)malloc(sizeof(int64_t) * (size_t)block_size);
  for (int64_t b = 0; b < num_blocks; b++) {
    for (int64_t o = 0; o < block_size; o++) {
      int64_t i = b * block_size + o;
      float v = i < n ? orc_f16_to_f32(logits[i]) : 0.0f;
      vals[o] = i < len ? v : -1.0e30f;
      idx[o] = i;
    }
    block_winner(vals, idx, block_size, &block_max[b], &block_idx[b], len + 1);
  }
  free(vals);
  free(idx);
}

/* lm_head_argmax_blocks_f16<K> (argmax.rs:88-158): logits of 64 rows per block, accumulated in f32 over K / 32 tiles
 * of 32 columns (each tile's 32 products summed, then added to the accumulator, :108-120), rows >= vocab_size masked
 * to -1e30 (:127-132), then the block winner as above with vocab_size + 1 for "none" (:139-143). */
void orc_lm_head_argmax_blocks_f16(const uint16_t* weights, const uint16_t* hidden, int64_t rows, int64_t k,
                                   int64_t vocab_size, float* block_max, uint32_t* block_idx, int64_t num_blocks) {
  float* h = (float*)malloc(sizeof(float) * (size_t)k);
  for (int64_t i = 0; i < k; i++) h[i] = orc_f16_to_f32(hidden[i]);
#pragma omp parallel for schedule(dynamic, 4)
  for (int64_t b = 0; b < num_blocks; b++) {
    float vals[64];
    int64_t idx[64];
    for (int64_t o = 0; o < 64; o++) {
      int64_t r = b * 64 + o;
      float acc = 0.0f;
      if (r < rows)
        for (int64_t kb = 0; kb + 32 <= k; kb += 32) {
          float partial = 0.0f;
          for (int64_t j = 0; j < 32; j++) partial += orc_f16_to_f32(weights[r * k + kb + j]) * h[kb + j];
          acc += partial;
        }
      vals[o] = r < vocab_size ? acc : -1.0e30f;
      idx[o] = r;
    }
    block_winner(vals, idx, 64, &block_max[b], &block_idx[b], vocab_size + 1);
  }
  free(h);
}

/* argmax_reduce_blocks_to_u32<BLOCK_SIZE> (argmax.rs:173-213): one tile of BLOCK_SIZE (value, index) pairs, entries
 * beyond the tensors read as zero, entries >= num_blocks masked to -1e30; the result is the smallest index among the
 * entries attaining the maximum (2147483647 if none). */
uint32_t orc_argmax_reduce_blocks_to_u32(const float* block_max, const uint32_t* block_idx, int64_t n,
                                         int64_t block_size, int64_t num_blocks) {
  float* vals = (float*)malloc(sizeof(float) * (size_t)block_size);
  int64_t* idx = (int64_t*)malloc(sizeof(int64_t) * (size_t)block_size);
  for (int64_t o = 0; o < block_size; o++) {
    vals[o] = o < num_blocks ? (o < n ? block_max[o] : 0.0f) : -1.0e30f;
    idx[o] = o < n ? (int64_t)(int32_t)block_idx[o] : 0;
  }
  float mx;
  uint32_t out;
  block_winner(vals, idx, block_size, &mx, &out, 2147483647);
  free(vals);
  free(idx);
  return out;
}

/* qk_norm_rope_kv_prefill_raw_f16 (cutile-kernels/src/experimental/fused_transformer.rs:22-345; the decode form
 * :356-625 is the same for seq_len = 1).  q [seq, nq, d], k and v [seq, nkv, d], caches [nkv, max_seq, d].  Per row:
 * ss = sum(x_lo^2 + x_hi^2) (:182-184), inv = rsqrt(ss / D + eps) (:185-189), norm = x * inv * w in f32 (:239-240),
 * theta = f32(position_start + s) * inv_freq (:249-254), y_lo = n_lo cos - n_hi sin, y_hi = n_hi cos + n_lo sin
 * (:257-258), one rounding to f16 (:259-260); q rows to q_out, k rows to k_cache[h, position], v copied (:263-341). */
void orc_qk_norm_rope_kv_f16(const uint16_t* q, const uint16_t* k, const uint16_t* v, const uint16_t* qw,
                             const uint16_t* kw, const float* inv_freq, uint16_t* q_out, uint16_t* k_cache,
                             uint16_t* v_cache, float eps, int64_t position_start, int64_t seq_len, int64_t nq,
                             int64_t nkv, int64_t d, int64_t max_seq) {
  const int64_t half = d / 2;
  for (int64_t s = 0; s < seq_len; s++) {
    const int64_t pos_i = position_start + s;
    const float pos = (float)pos_i;
    for (int64_t r = 0; r < nq + nkv; r++) {
      const int is_q = r < nq;
      const uint16_t* x = is_q ? q + (s * nq + r) * d : k + (s * nkv + (r - nq)) * d;
      const uint16_t* w = is_q ? qw : kw;
      uint16_t* dst = is_q ? q_out + (s * nq + r) * d : k_cache + ((r - nq) * max_seq + pos_i) * d;
      if (!is_q && (pos_i < 0 || pos_i >= max_seq)) continue;
      float ss = 0.0f;
      for (int64_t i = 0; i < half; i++) {
        float lo = orc_f16_to_f32(x[i]), hi = orc_f16_to_f32(x[half + i]);
        ss += lo * lo + hi * hi;
      }
      const float inv = 1.0f / sqrtf(ss / (float)d + eps);
      for (int64_t i = 0; i < half; i++) {
        const float nl = orc_f16_to_f32(x[i]) * inv * orc_f16_to_f32(w[i]);
        const float nh = orc_f16_to_f32(x[half + i]) * inv * orc_f16_to_f32(w[half + i]);
        const float theta = pos * inv_freq[i];
        const float cs = cosf(theta), sn = sinf(theta);
        dst[i] = orc_f32_to_f16(nl * cs - nh * sn);
        dst[half + i] = orc_f32_to_f16(nh * cs + nl * sn);
      }
    }
    if (pos_i >= 0 && pos_i < max_seq)
      for (int64_t h = 0; h < nkv; h++)
        memcpy(v_cache + (h * max_seq + pos_i) * d, v + (s * nkv + h) * d, sizeof(uint16_t) * (size_t)d);
  }
}

/* rms_norm<N, BLOCK_SIZE> f32 (cutile-examples/examples/rms_norm.rs:17-61): a [1, BLOCK] vector accumulates x*x over
 * the N / BLOCK chunks of the row and is then summed (:33-41); scale = sqrt(1 / (sum / N + eps)) with the square root
 * rounded toward minus infinity (:42-46); out = x * scale * w (:56).  block = 0 means one chunk (BLOCK = N). */
void orc_rms_norm_f32_example(const float* x, const float* w, float* out, int64_t rows, int64_t n, float eps,
                              int64_t block) {
  if (block <= 0 || block > n) block = n;
  float* acc = (float*)malloc(sizeof(float) * (size_t)block);
  for (int64_t r = 0; r < rows; r++) {
    const float* xr = x + r * n;
    for (int64_t i = 0; i < block; i++) acc[i] = 0.0f;
    for (int64_t j = 0; j + block <= n; j += block)
      for (int64_t i = 0; i < block; i++) acc[i] = acc[i] + xr[j + i] * xr[j + i];
    /* reduce_sum over the BLOCK lanes: pairwise (a tile reduction is a tree; the order is not part of the contract) */
    for (int64_t width = block; width > 1; width = (width + 1) / 2)
      for (int64_t i = 0; i < width / 2; i++) acc[i] = acc[i] + acc[i + (width + 1) / 2];
    const float sum = acc[0];
    const float v = 1.0f / (sum / (float)n + eps);
    float scale = sqrtf(v);                                   /* correctly rounded to nearest */
    if (fmaf(scale, scale, -v) > 0.0f) scale = nextafterf(scale, 0.0f);   /* toward minus infinity */
    for (int64_t j = 0; j < n; j++) out[r * n + j] = xr[j] * scale * w[j];
  }
  free(acc);
}

/* ---- Philox4x32-10 and the random fills ------------------------------------------------------------ */
void orc_philox4x32_10(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4]) {
  uint32_t c0 = counter[0], c1 = counter[1], c2 = counter[2], c3 = counter[3], k0 = key[0], k1 = key[1];
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    c0 = n0; c1 = (uint32_t)p1; c2 = n2; c3 = (uint32_t)p0;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

void orc_rng_fill_f32(float* out, size_t n, uint64_t seed, uint64_t offset, int kind, float mean, float std) {
  const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  const size_t blocks = (n + 3) / 4;
  for (size_t b = 0; b < blocks; ++b) {
    const uint64_t ctr = offset + b;
    const uint32_t counter[4] = {(uint32_t)ctr, (uint32_t)(ctr >> 32), 0u, 0u};
    uint32_t r[4];
    orc_philox4x32_10(counter, key, r);
    float v[4];
    if (kind == 0) {
      for (int i = 0; i < 4; ++i) v[i] = (float)(r[i] >> 8) * 5.9604644775390625e-8f;
    } else {
      for (int pair = 0; pair < 2; ++pair) {
        const float u1 = (float)((r[2 * pair] >> 8) + 1u) * 5.9604644775390625e-8f;
        const float u2 = (float)(r[2 * pair + 1] >> 8) * 5.9604644775390625e-8f;
        const float rad = sqrtf(-2.0f * logf(u1)), t = 6.283185307179586f * u2;
        v[2 * pair] = fmaf(std, rad * cosf(t), mean);
        v[2 * pair + 1] = fmaf(std, rad * sinf(t), mean);
      }
    }
    for (int i = 0; i < 4; ++i)
      if (b * 4 + i < n) out[b * 4 + i] = v[i];
  }
}

void orc_rng_fill_f64(double* out, size_t n, uint64_t seed, uint64_t offset, int kind, double mean, double std) {
  const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  const size_t blocks = (n + 1) / 2;
  for (size_t b = 0; b < blocks; ++b) {
    const uint64_t ctr = offset + b;
    const uint32_t counter[4] = {(uint32_t)ctr, (uint32_t)(ctr >> 32), 0u, 0u};
    uint32_t r[4];
    orc_philox4x32_10(counter, key, r);
    double v0 = (double)((((uint64_t)r[1]) << 21) ^ (uint64_t)(r[0] >> 11)) * 1.1102230246251565e-16;
    double v1 = (double)((((uint64_t)r[3]) << 21) ^ (uint64_t)(r[2] >> 11)) * 1.1102230246251565e-16;
    if (kind != 0) {
      const double rad = sqrt(-2.0 * log(v0 + 1.1102230246251565e-16)), t = 6.283185307179586476925 * v1;
      v0 = fma(std, rad * cos(t), mean);
      v1 = fma(std, rad * sin(t), mean);
    }
    if (b * 2 < n) out[b * 2] = v0;
    if (b * 2 + 1 < n) out[b * 2 + 1] = v1;
  }
}
