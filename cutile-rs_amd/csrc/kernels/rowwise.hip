// Row-wise bandwidth kernels for gfx950: RMSNorm (f16 IO, f32 math) and softmax
// over tile rows (f16 or f32 IO, f32 statistics).
//
// Bodies follow the reference's tile programs:
//   rms_norm_f16   cutile-kernels/src/norms.rs:16-60
//                  ss = sum x^2 (f32); inv = rsqrt(ss/N + eps); out = f16(x * inv * w)
//   softmax        cutile-examples/examples/softmax.rs:11-24,
//                  cutile-benchmarks/benches/softmax.rs:19-35
//                  per tile row: e = exp(x - max); y = e / sum(e)
//
// Also here, on the same row machinery: add_rms_norm_f16 and qk_norm_f16
// (cutile-kernels/src/norms.rs:68-136, 143-216).
//
// The reference reads each RMSNorm row twice (two loops over BLOCK_SIZE chunks).
// Here a row is read from HBM exactly once: it is held in registers as 16-byte
// vectors (one wavefront, or WPR wavefronts, per row; lane-strided so that every
// access of a wavefront is one contiguous 1 KiB burst), reduced with cross-lane
// shuffles (plus one LDS exchange when several wavefronts share a row), scaled
// and written back with 16-byte stores.  Algorithmic traffic is therefore
// x + out (+ w once per row from L2).
//
// A "segment" is one tile row: for RMSNorm a whole tensor row (tile [1, N]); for
// softmax the BN columns of one row that fall in one [BM, BN] tile (row softmax
// iff BN == N).  Padding rule for a ragged last tile: lanes beyond the tensor's
// extent read 0 and take part in max/sum (padding::Zero on load), and are not
// stored.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <type_traits>

#include "kernel_args.h"
#include "lane_exchange.h"

using namespace cutile;

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;
constexpr float kLog2e = 1.4426950408889634f;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

template <typename T>
union Vec16 {
  static constexpr int N = 16 / sizeof(T);
  u32x4 raw;
  T v[N];
  __device__ Vec16() : raw{} {}
};

// Sum / maximum over the 64 lanes, in every lane, without leaving the vector ALU (lane_exchange.h).
__device__ __forceinline__ float wave_sum(float v) { return lanes::across_wave<lanes::Sum>(v); }
__device__ __forceinline__ float wave_max(float v) { return lanes::across_wave<lanes::Max>(v); }

// Reduction across the WPR wavefronts that share a segment.  `slot` is the
// segment's index inside the workgroup, `sub` the wavefront's index inside the
// segment.  Two buffers alternate so back-to-back reductions need one barrier each.
template <int WPR, bool IS_MAX>
__device__ __forceinline__ float group_reduce(float v, float* lds, int slot, int sub) {
  v = IS_MAX ? wave_max(v) : wave_sum(v);
  if constexpr (WPR == 1) {
    return v;
  } else {
    if ((threadIdx.x & 63) == 0) lds[slot * WPR + sub] = v;
    __syncthreads();
    float r = lds[slot * WPR];
#pragma unroll
    for (int i = 1; i < WPR; ++i) r = IS_MAX ? fmaxf(r, lds[slot * WPR + i]) : r + lds[slot * WPR + i];
    return r;
  }
}

struct SegmentMap {
  // segment -> (row, first column, valid columns)
  int32_t n_cols;       // tensor columns
  int32_t seg_len;      // BN (== tile width)
  int32_t segs_per_row; // tiles along columns that the launch grid covers
  int64_t n_segments;
};

// ---- RMSNorm -----------------------------------------------------------------------------
// Rows at or beyond `split` come from (x2, w2) instead of (x, w), indexed from 0
// again: qk_norm_f16's "q rows first, then k rows" (split = rows for plain RMSNorm).
template <int WPR, int VPL>
__device__ __forceinline__ void rms_norm_rows(const _Float16* __restrict__ x, int64_t x_row_stride,
                                              const _Float16* __restrict__ w,
                                              _Float16* __restrict__ out, int64_t out_row_stride,
                                              int32_t n, int64_t rows, float eps,
                                              const _Float16* __restrict__ x2 = nullptr, int64_t x2_row_stride = 0,
                                              const _Float16* __restrict__ w2 = nullptr, int64_t split = INT64_MAX) {
  using V = Vec16<_Float16>;
  constexpr int ROWS_PER_WG = kWaves / WPR;
  __shared__ float lds[kWaves];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int slot = wave / WPR, sub = wave % WPR;
  const int64_t row = (int64_t)blockIdx.x * ROWS_PER_WG + slot;
  const bool live = row < rows;
  const int32_t nvec = n >> 3;
  const int32_t v0 = sub * 64 + lane;

  V xv[VPL];
  float ss = 0.0f;
  const bool second = row >= split;   // same for all wavefronts of a row
  if (live) {
    const u32x4* xr = reinterpret_cast<const u32x4*>(second ? x2 + (row - split) * x2_row_stride : x + row * x_row_stride);
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      int32_t vi = v0 + i * (64 * WPR);
      if (vi < nvec) xv[i].raw = __builtin_nontemporal_load(xr + vi);
    }
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float f = (float)xv[i].v[e];
        ss = __builtin_fmaf(f, f, ss);
      }
    }
  }
  ss = group_reduce<WPR, false>(ss, lds, slot, sub);
  if (!live) return;
  const float inv = __builtin_amdgcn_rsqf(ss / (float)n + eps);
  u32x4* orow = reinterpret_cast<u32x4*>(out + row * out_row_stride);
  const u32x4* wr = reinterpret_cast<const u32x4*>(second ? w2 : w);
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    int32_t vi = v0 + i * (64 * WPR);
    if (vi < nvec) {
      V wv, ov;
      wv.raw = wr[vi];
#pragma unroll
      for (int e = 0; e < 8; ++e) ov.v[e] = (_Float16)(((float)xv[i].v[e] * inv) * (float)wv.v[e]);
      __builtin_nontemporal_store(ov.raw, orow + vi);
    }
  }
}

// Short rows (head-dimension norms: N = 64 .. 256): LPR lanes per row, one
// 16-byte vector per lane, 64 / LPR rows per wavefront and pass, kShortRowPasses passes per
// wavefront with all their loads issued first (64 bytes in flight per lane, as in the long-row
// kernels); the reduction stays inside the LPR-lane group, on the cross-lane data path (sums of
// quad neighbours, then mirrored halves: every step pairs groups that already agree).
// With a wavefront per row most lanes would idle.
constexpr int kShortRowPasses = 4;
template <int LPR>
__device__ __forceinline__ float lane_group_sum(float v) {
  return lanes::across_group<lanes::Sum, LPR>(v);
}
template <int LPR>
__device__ __forceinline__ void rms_norm_rows_short(const _Float16* __restrict__ x, int64_t x_row_stride,
                                                    const _Float16* __restrict__ w,
                                                    _Float16* __restrict__ out, int64_t out_row_stride,
                                                    int32_t n, int64_t rows, float eps,
                                                    const _Float16* __restrict__ x2 = nullptr, int64_t x2_row_stride = 0,
                                                    const _Float16* __restrict__ w2 = nullptr, int64_t split = INT64_MAX) {
  using V = Vec16<_Float16>;
  constexpr int RPW = 64 / LPR, U = kShortRowPasses;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t row0 = ((int64_t)blockIdx.x * kWaves + wave) * (RPW * U) + lane / LPR;
  const int32_t vi = lane % LPR;
  V xv[U];
  bool live[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t row = row0 + u * RPW;
    live[u] = row < rows && vi < (n >> 3);
    if (live[u]) {
      const u32x4* xr = reinterpret_cast<const u32x4*>(row >= split ? x2 + (row - split) * x2_row_stride : x + row * x_row_stride);
      xv[u].raw = __builtin_nontemporal_load(xr + vi);
    }
  }
  V wq, wk;
  if (vi < (n >> 3)) {
    wq.raw = reinterpret_cast<const u32x4*>(w)[vi];
    if (w2) wk.raw = reinterpret_cast<const u32x4*>(w2)[vi];
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    float ss = 0.0f;
    if (live[u]) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float f = (float)xv[u].v[e];
        ss = __builtin_fmaf(f, f, ss);
      }
    }
    ss = lane_group_sum<LPR>(ss);
    if (!live[u]) continue;
    const int64_t row = row0 + u * RPW;
    const float inv = __builtin_amdgcn_rsqf(ss / (float)n + eps);
    const V& wv = row >= split ? wk : wq;
    V ov;
#pragma unroll
    for (int e = 0; e < 8; ++e) ov.v[e] = (_Float16)(((float)xv[u].v[e] * inv) * (float)wv.v[e]);
    __builtin_nontemporal_store(ov.raw, reinterpret_cast<u32x4*>(out + row * out_row_stride) + vi);
  }
}

// add_rms_norm_f16: combined = residual + x stays in f32 registers (it is both
// the normalised quantity and, rounded, the new residual): two rows read, two
// rows written, each once.
template <int WPR, int VPL>
__device__ __forceinline__ void add_rms_norm_rows(const _Float16* __restrict__ residual, int64_t res_row_stride,
                                                  const _Float16* __restrict__ x, int64_t x_row_stride,
                                                  const _Float16* __restrict__ w,
                                                  _Float16* __restrict__ out, int64_t out_row_stride,
                                                  _Float16* __restrict__ res_out, int64_t res_out_row_stride,
                                                  int32_t n, int64_t rows, float eps) {
  using V = Vec16<_Float16>;
  constexpr int ROWS_PER_WG = kWaves / WPR;
  __shared__ float lds[kWaves];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int slot = wave / WPR, sub = wave % WPR;
  const int64_t row = (int64_t)blockIdx.x * ROWS_PER_WG + slot;
  const bool live = row < rows;
  const int32_t nvec = n >> 3;
  const int32_t v0 = sub * 64 + lane;

  float cv[VPL][8];
  float ss = 0.0f;
  if (live) {
    const u32x4* rr = reinterpret_cast<const u32x4*>(residual + row * res_row_stride);
    const u32x4* xr = reinterpret_cast<const u32x4*>(x + row * x_row_stride);
    V rv[VPL], xv[VPL];
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      int32_t vi = v0 + i * (64 * WPR);
      if (vi < nvec) {
        rv[i].raw = __builtin_nontemporal_load(rr + vi);
        xv[i].raw = __builtin_nontemporal_load(xr + vi);
      }
    }
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        cv[i][e] = (float)rv[i].v[e] + (float)xv[i].v[e];
        ss = __builtin_fmaf(cv[i][e], cv[i][e], ss);
      }
    }
  }
  ss = group_reduce<WPR, false>(ss, lds, slot, sub);
  if (!live) return;
  const float inv = __builtin_amdgcn_rsqf(ss / (float)n + eps);
  u32x4* orow = reinterpret_cast<u32x4*>(out + row * out_row_stride);
  u32x4* rrow = reinterpret_cast<u32x4*>(res_out + row * res_out_row_stride);
  const u32x4* wr = reinterpret_cast<const u32x4*>(w);
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    int32_t vi = v0 + i * (64 * WPR);
    if (vi < nvec) {
      V wv, ov, cvh;
      wv.raw = wr[vi];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        ov.v[e] = (_Float16)((cv[i][e] * inv) * (float)wv.v[e]);
        cvh.v[e] = (_Float16)cv[i][e];
      }
      __builtin_nontemporal_store(ov.raw, orow + vi);
      __builtin_nontemporal_store(cvh.raw, rrow + vi);
    }
  }
}

// Any N / any strides for the two fused forms: one workgroup per row, inputs re-read (L2).
__device__ __forceinline__ void fused_norm_row_generic(const TensorArg<2>& a, const TensorArg<2>* b_add,
                                                       const TensorArg<2>* b_alt, const TensorArg<1>& w,
                                                       const TensorArg<1>* w_alt, const PartitionArg<2>& out,
                                                       const PartitionArg<2>* out2, float eps, int64_t rows,
                                                       int64_t split) {
  // b_add: second addend (add_rms_norm); b_alt / w_alt: source and weight for rows >= split (qk_norm)
  __shared__ float lds[kWaves];
  const int wave = threadIdx.x >> 6;
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const bool second = b_alt && row >= split;
    const TensorArg<2>& src = second ? *b_alt : a;
    const int64_t srow = second ? row - split : row;
    const TensorArg<1>& wt = second ? *w_alt : w;
    const _Float16* xr = (const _Float16*)src.ptr + srow * src.strides[0];
    const _Float16* ar = b_add ? (const _Float16*)b_add->ptr + row * b_add->strides[0] : nullptr;
    const int32_t n = src.shape[1];
    auto value = [&](int32_t j) -> float {
      float f = (float)xr[(int64_t)j * src.strides[1]];
      return ar ? f + (float)ar[(int64_t)j * b_add->strides[1]] : f;
    };
    float ss = 0.0f;
    for (int32_t j = threadIdx.x; j < n; j += kThreads) {
      float f = value(j);
      ss = __builtin_fmaf(f, f, ss);
    }
    ss = group_reduce<kWaves, false>(ss, lds, 0, wave);
    const float inv = __builtin_amdgcn_rsqf(ss / (float)n + eps);
    _Float16* orow = (_Float16*)out.ptr + row * out.strides[0];
    _Float16* o2row = out2 ? (_Float16*)out2->ptr + row * out2->strides[0] : nullptr;
    const int32_t n_out = out.shape[1] < n ? out.shape[1] : n;
    for (int32_t j = threadIdx.x; j < n_out; j += kThreads) {
      float f = value(j);
      float wv = j < wt.shape[0] ? (float)((const _Float16*)wt.ptr)[(int64_t)j * wt.strides[0]] : 0.0f;
      orow[(int64_t)j * out.strides[1]] = (_Float16)((f * inv) * wv);
      if (o2row && j < out2->shape[1]) o2row[(int64_t)j * out2->strides[1]] = (_Float16)f;
    }
    __syncthreads();
  }
}

// Any N / any strides: one workgroup per row, the row is re-read for the second
// pass (it is still in L2).
__device__ __forceinline__ void rms_norm_row_generic(const TensorArg<2>& x, const TensorArg<1>& w,
                                                     const PartitionArg<2>& out, float eps,
                                                     int64_t rows) {
  __shared__ float lds[kWaves];
  const int wave = threadIdx.x >> 6;
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const _Float16* xr = (const _Float16*)x.ptr + row * x.strides[0];
    const int32_t n = x.shape[1];
    float ss = 0.0f;
    for (int32_t j = threadIdx.x; j < n; j += kThreads) {
      float f = (float)xr[(int64_t)j * x.strides[1]];
      ss = __builtin_fmaf(f, f, ss);
    }
    ss = group_reduce<kWaves, false>(ss, lds, 0, wave);
    const float inv = __builtin_amdgcn_rsqf(ss / (float)n + eps);
    _Float16* orow = (_Float16*)out.ptr + row * out.strides[0];
    const int32_t n_out = out.shape[1] < n ? out.shape[1] : n;
    for (int32_t j = threadIdx.x; j < n_out; j += kThreads) {
      float f = (float)xr[(int64_t)j * x.strides[1]];
      float wv = j < w.shape[0] ? (float)((const _Float16*)w.ptr)[(int64_t)j * w.strides[0]] : 0.0f;
      orow[(int64_t)j * out.strides[1]] = (_Float16)((f * inv) * wv);
    }
    __syncthreads();  // lds is reused by the next row
  }
}

// ---- softmax -----------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ float to_f32(T v) {
  return (float)v;
}

template <typename T, int WPR, int VPL>
__device__ __forceinline__ void softmax_segments(const T* __restrict__ x, int64_t x_row_stride,
                                                 T* __restrict__ y, int64_t y_row_stride,
                                                 int32_t x_cols, int32_t y_cols, int32_t seg_len,
                                                 int32_t segs_per_row, int64_t n_segments) {
  using V = Vec16<T>;
  constexpr int E = V::N;
  constexpr int SEGS_PER_WG = kWaves / WPR;
  __shared__ float lds[2][kWaves];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int slot = wave / WPR, sub = wave % WPR;
  const int64_t seg = (int64_t)blockIdx.x * SEGS_PER_WG + slot;
  const bool live = seg < n_segments;
  // whole rows (one segment per row) are the common case: no 64-bit division on the way to the first load
  const int64_t row = !live ? 0 : segs_per_row == 1 ? seg : seg / segs_per_row;
  const int32_t col0 = !live || segs_per_row == 1 ? 0 : (int32_t)(seg % segs_per_row) * seg_len;
  const int32_t seg_vec = seg_len / E;                 // vectors in a full segment
  const int32_t x_valid = live ? max(0, min(seg_len, x_cols - col0)) / E : 0;  // readable vectors
  const int32_t y_valid = live ? max(0, min(seg_len, y_cols - col0)) / E : 0;  // storable vectors
  const int32_t v0 = sub * 64 + lane;

  V xv[VPL];
  float m = -INFINITY;
  const u32x4* xr = reinterpret_cast<const u32x4*>(x + row * x_row_stride + col0);
  // every load is requested before the first value is looked at: a use between two loads makes the second
  // wait for the first, and the row would cost VPL memory latencies instead of one
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    int32_t vi = v0 + i * (64 * WPR);
    if (vi < x_valid) xv[i].raw = __builtin_nontemporal_load(xr + vi);  // else stays 0 (padding)
  }
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    int32_t vi = v0 + i * (64 * WPR);
    if (live && vi < seg_vec) {
#pragma unroll
      for (int e = 0; e < E; ++e) m = fmaxf(m, to_f32(xv[i].v[e]));
    }
  }
  m = group_reduce<WPR, true>(m, lds[0], slot, sub);
  const float mb = m * kLog2e;
  float ev[VPL][E];
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    int32_t vi = v0 + i * (64 * WPR);
    if (live && vi < seg_vec) {
#pragma unroll
      for (int e = 0; e < E; ++e) {
        ev[i][e] = __builtin_amdgcn_exp2f(__builtin_fmaf(to_f32(xv[i].v[e]), kLog2e, -mb));
        s += ev[i][e];
      }
    }
  }
  s = group_reduce<WPR, false>(s, lds[1], slot, sub);
  if (!live) return;
  const float inv = 1.0f / s;
  u32x4* yr = reinterpret_cast<u32x4*>(y + row * y_row_stride + col0);
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    int32_t vi = v0 + i * (64 * WPR);
    if (vi < y_valid) {
      V ov;
#pragma unroll
      for (int e = 0; e < E; ++e) {
        if constexpr (sizeof(T) == 4)
          ov.v[e] = (T)(ev[i][e] / s);
        else
          ov.v[e] = (T)(ev[i][e] * inv);
      }
      __builtin_nontemporal_store(ov.raw, yr + vi);
    }
  }
}

// Any tile width / any strides: one workgroup per segment, three passes (the
// segment stays in L2 between them).
template <typename T>
__device__ __forceinline__ void softmax_segment_generic(const TensorArg<2>& x,
                                                        const PartitionArg<2>& y,
                                                        int32_t segs_per_row, int64_t n_segments) {
  __shared__ float lds[2][kWaves];
  const int wave = threadIdx.x >> 6;
  const int32_t bn = y.pshape[1];
  for (int64_t seg = blockIdx.x; seg < n_segments; seg += gridDim.x) {
    const int64_t row = seg / segs_per_row;
    const int32_t col0 = (int32_t)(seg % segs_per_row) * bn;
    const bool row_ok = row < x.shape[0];
    const T* xr = (const T*)x.ptr + row * x.strides[0];
    auto ld = [&](int32_t j) -> float {
      int32_t c = col0 + j;
      return (row_ok && c < x.shape[1]) ? to_f32(xr[(int64_t)c * x.strides[1]]) : 0.0f;
    };
    float m = -INFINITY;
    for (int32_t j = threadIdx.x; j < bn; j += kThreads) m = fmaxf(m, ld(j));
    m = group_reduce<kWaves, true>(m, lds[0], 0, wave);
    const float mb = m * kLog2e;
    float s = 0.0f;
    for (int32_t j = threadIdx.x; j < bn; j += kThreads)
      s += __builtin_amdgcn_exp2f(__builtin_fmaf(ld(j), kLog2e, -mb));
    s = group_reduce<kWaves, false>(s, lds[1], 0, wave);
    if (row < y.shape[0]) {
      T* yr = (T*)y.ptr + row * y.strides[0];
      for (int32_t j = threadIdx.x; j < bn; j += kThreads) {
        int32_t c = col0 + j;
        if (c < y.shape[1])
          yr[(int64_t)c * y.strides[1]] =
              (T)(__builtin_amdgcn_exp2f(__builtin_fmaf(ld(j), kLog2e, -mb)) / s);
      }
    }
    __syncthreads();
  }
}

}  // namespace

// rms_norm_f16(x, w, out: [1, N] tiles, eps).  g.x = number of rows the launch covers.
#define RMS_NORM_KERNEL(WPR, VPL)                                                                   \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      rms_norm_f16_entry__w##WPR##v##VPL(TensorArg<2> x, TensorArg<1> w, PartitionArg<2> out,       \
                                         float eps, TileGrid g) {                                   \
    int64_t rows = min((int64_t)g.x, (int64_t)out.shape[0]);                                       \
    rms_norm_rows<WPR, VPL>((const _Float16*)x.ptr, x.strides[0], (const _Float16*)w.ptr,          \
                            (_Float16*)out.ptr, out.strides[0], x.shape[1], rows, eps);            \
  }

RMS_NORM_KERNEL(1, 1)
RMS_NORM_KERNEL(1, 2)
RMS_NORM_KERNEL(1, 4)
RMS_NORM_KERNEL(1, 8)
RMS_NORM_KERNEL(1, 16)
RMS_NORM_KERNEL(2, 2)
RMS_NORM_KERNEL(2, 4)
RMS_NORM_KERNEL(2, 8)
RMS_NORM_KERNEL(4, 1)
RMS_NORM_KERNEL(4, 2)
RMS_NORM_KERNEL(4, 4)
RMS_NORM_KERNEL(4, 8)
RMS_NORM_KERNEL(4, 16)

// add_rms_norm_f16(residual, x, w, out: [1, N] tiles, residual_out: [1, N] tiles, eps)
#define ADD_RMS_NORM_KERNEL(WPR, VPL)                                                               \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      add_rms_norm_f16_entry__w##WPR##v##VPL(TensorArg<2> residual, TensorArg<2> x, TensorArg<1> w, \
                                             PartitionArg<2> out, PartitionArg<2> residual_out,     \
                                             float eps, TileGrid g) {                               \
    int64_t rows = min((int64_t)g.x, (int64_t)out.shape[0]);                                       \
    add_rms_norm_rows<WPR, VPL>((const _Float16*)residual.ptr, residual.strides[0],                \
                                (const _Float16*)x.ptr, x.strides[0], (const _Float16*)w.ptr,      \
                                (_Float16*)out.ptr, out.strides[0], (_Float16*)residual_out.ptr,   \
                                residual_out.strides[0], x.shape[1], rows, eps);                   \
  }
// qk_norm_f16(q, k, q_weight, k_weight, out: [1, N] tiles, eps, num_q_rows)
#define QK_NORM_KERNEL(WPR, VPL)                                                                    \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      qk_norm_f16_entry__w##WPR##v##VPL(TensorArg<2> q, TensorArg<2> k, TensorArg<1> qw,            \
                                        TensorArg<1> kw, PartitionArg<2> out, float eps,            \
                                        int32_t num_q_rows, TileGrid g) {                           \
    int64_t rows = min((int64_t)g.x, (int64_t)out.shape[0]);                                       \
    rms_norm_rows<WPR, VPL>((const _Float16*)q.ptr, q.strides[0], (const _Float16*)qw.ptr,         \
                            (_Float16*)out.ptr, out.strides[0], q.shape[1], rows, eps,             \
                            (const _Float16*)k.ptr, k.strides[0], (const _Float16*)kw.ptr,         \
                            (int64_t)num_q_rows);                                                  \
  }
#define RMS_NORM_SHORT_KERNEL(LPR)                                                                  \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      rms_norm_f16_entry__s##LPR(TensorArg<2> x, TensorArg<1> w, PartitionArg<2> out, float eps,    \
                                 TileGrid g) {                                                      \
    int64_t rows = min((int64_t)g.x, (int64_t)out.shape[0]);                                       \
    rms_norm_rows_short<LPR>((const _Float16*)x.ptr, x.strides[0], (const _Float16*)w.ptr,         \
                             (_Float16*)out.ptr, out.strides[0], x.shape[1], rows, eps);           \
  }                                                                                                 \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      qk_norm_f16_entry__s##LPR(TensorArg<2> q, TensorArg<2> k, TensorArg<1> qw, TensorArg<1> kw,   \
                                PartitionArg<2> out, float eps, int32_t num_q_rows, TileGrid g) {   \
    int64_t rows = min((int64_t)g.x, (int64_t)out.shape[0]);                                       \
    rms_norm_rows_short<LPR>((const _Float16*)q.ptr, q.strides[0], (const _Float16*)qw.ptr,        \
                             (_Float16*)out.ptr, out.strides[0], q.shape[1], rows, eps,            \
                             (const _Float16*)k.ptr, k.strides[0], (const _Float16*)kw.ptr,        \
                             (int64_t)num_q_rows);                                                 \
  }
RMS_NORM_SHORT_KERNEL(8)
RMS_NORM_SHORT_KERNEL(16)
RMS_NORM_SHORT_KERNEL(32)

#define FUSED_NORM_VARIANTS(M) \
  M(1, 1) M(1, 2) M(1, 4) M(1, 8) M(2, 2) M(2, 4) M(2, 8) M(4, 1) M(4, 2) M(4, 4) M(4, 8)
FUSED_NORM_VARIANTS(ADD_RMS_NORM_KERNEL)
FUSED_NORM_VARIANTS(QK_NORM_KERNEL)

extern "C" __global__ void __launch_bounds__(kThreads)
    add_rms_norm_f16_entry__generic(TensorArg<2> residual, TensorArg<2> x, TensorArg<1> w, PartitionArg<2> out,
                                    PartitionArg<2> residual_out, float eps, TileGrid g) {
  int64_t rows = min((int64_t)g.x, (int64_t)out.shape[0]);
  fused_norm_row_generic(x, &residual, nullptr, w, nullptr, out, &residual_out, eps, rows, INT64_MAX);
}
extern "C" __global__ void __launch_bounds__(kThreads)
    qk_norm_f16_entry__generic(TensorArg<2> q, TensorArg<2> k, TensorArg<1> qw, TensorArg<1> kw, PartitionArg<2> out,
                               float eps, int32_t num_q_rows, TileGrid g) {
  int64_t rows = min((int64_t)g.x, (int64_t)out.shape[0]);
  fused_norm_row_generic(q, nullptr, &k, qw, &kw, out, nullptr, eps, rows, (int64_t)num_q_rows);
}

extern "C" __global__ void __launch_bounds__(kThreads)
    rms_norm_f16_entry__generic(TensorArg<2> x, TensorArg<1> w, PartitionArg<2> out, float eps,
                                TileGrid g) {
  int64_t rows = min((int64_t)g.x, (int64_t)out.shape[0]);
  rms_norm_row_generic(x, w, out, eps, rows);
}

// rms_norm<N, BLOCK_SIZE>(x: [-1, N] f32, w: [N] f32, out: [1, N] tiles f32, eps) — the f32 example form
// (cutile-examples/examples/rms_norm.rs:17-61): scale = sqrt(1 / (sum(x^2) / N + eps)) with the square root rounded
// toward minus infinity (:44-46), out = x * scale * w (:56).  One workgroup per row, 16-byte accesses where the
// layout allows it; the row is re-read for the second pass (it is still in L2).
__device__ __forceinline__ float sqrt_toward_minus_infinity(float v) {
  float r = __builtin_sqrtf(v);                        // correctly rounded to nearest
  if (__builtin_fmaf(r, r, -v) > 0.0f) r = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, r) - 1u);   // r^2 > v: one ulp down
  return r;
}
extern "C" __global__ void __launch_bounds__(kThreads)
    rms_norm_entry__f32(TensorArg<2> x, TensorArg<1> w, PartitionArg<2> out, float eps, TileGrid g) {
  __shared__ float lds[kWaves];
  const int wave = threadIdx.x >> 6;
  const int64_t rows = min((int64_t)g.x, (int64_t)out.shape[0]);
  const int32_t n = x.shape[1];
  const int32_t n_out = out.shape[1] < n ? out.shape[1] : n;
  const bool vec = n % 4 == 0 && n_out % 4 == 0 && x.strides[1] == 1 && out.strides[1] == 1 && w.strides[0] == 1 &&
                   x.strides[0] % 4 == 0 && out.strides[0] % 4 == 0 && w.shape[0] >= n_out &&
                   (((uintptr_t)x.ptr | (uintptr_t)out.ptr | (uintptr_t)w.ptr) & 15) == 0;
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const float* xr = (const float*)x.ptr + row * x.strides[0];
    float* orow = (float*)out.ptr + row * out.strides[0];
    float ss = 0.0f;
    if (vec) {
      for (int32_t j = threadIdx.x; j < n / 4; j += kThreads) {
        const f32x4 v = reinterpret_cast<const f32x4*>(xr)[j];
        ss = __builtin_fmaf(v[0], v[0], ss);
        ss = __builtin_fmaf(v[1], v[1], ss);
        ss = __builtin_fmaf(v[2], v[2], ss);
        ss = __builtin_fmaf(v[3], v[3], ss);
      }
    } else {
      for (int32_t j = threadIdx.x; j < n; j += kThreads) {
        const float f = xr[(int64_t)j * x.strides[1]];
        ss = __builtin_fmaf(f, f, ss);
      }
    }
    ss = group_reduce<kWaves, false>(ss, lds, 0, wave);
    const float scale = sqrt_toward_minus_infinity(1.0f / (ss / (float)n + eps));
    if (vec) {
      for (int32_t j = threadIdx.x; j < n_out / 4; j += kThreads) {
        const f32x4 v = reinterpret_cast<const f32x4*>(xr)[j];
        const f32x4 wv = reinterpret_cast<const f32x4*>(w.ptr)[j];
        f32x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = (v[e] * scale) * wv[e];
        __builtin_nontemporal_store(o, reinterpret_cast<f32x4*>(orow) + j);
      }
    } else {
      for (int32_t j = threadIdx.x; j < n_out; j += kThreads) {
        const float f = xr[(int64_t)j * x.strides[1]];
        const float wv = j < w.shape[0] ? ((const float*)w.ptr)[(int64_t)j * w.strides[0]] : 0.0f;
        orow[(int64_t)j * out.strides[1]] = (f * scale) * wv;
      }
    }
    __syncthreads();  // lds is reused by the next row
  }
}

// ---- the benchmark programs' all-f16 arithmetic ------------------------------------------------
namespace {
// cutile-benchmarks/benches/rmsnorm.rs:20-66 and benches/softmax.rs:19-35 are written entirely in f16: every
// product, sum, quotient and the square root are f16 operations.  The kernels above compute the statistics in
// f32 (the arithmetic of cutile-kernels/src/norms.rs and of the examples); the two below reproduce the
// benchmark programs' own arithmetic, one rounding to f16 per operation, no fused multiply-add.
//
// The tile programs leave one thing to their compiler: the order in which reduce_sum adds the lanes of a
// tile.  The order here is the stride-halving tree: for step = L/2, L/4, .. 1: a[l] += a[l + step] (l < step)
// over the L lanes of the tile.  A wavefront owns one row; lane t holds the V consecutive tile lanes
// V*t .. V*t+V-1 (and, for a softmax row longer than 512, the same lanes of every 512-wide chunk), so the
// tree's large steps are in-register adds across chunks, the middle steps cross-lane exchanges (both partners
// compute the same IEEE sum, addition being commutative) and the last steps adds inside a lane.
__device__ __forceinline__ _Float16 shfl_xor_f16(_Float16 v, int mask) {
  const int bits = (int)__builtin_bit_cast(uint16_t, v);
  return __builtin_bit_cast(_Float16, (uint16_t)__shfl_xor(bits, mask, 64));
}
// Cross-lane exchange of V halves, two per 32-bit exchange.
template <int V>
__device__ __forceinline__ auto shfl_xor_hv(_Float16 __attribute__((ext_vector_type(V))) v, int mask) {
  typedef _Float16 hv __attribute__((ext_vector_type(V)));
  if constexpr (V == 1) {
    hv r;
    r[0] = shfl_xor_f16(v[0], mask);
    return r;
  } else {
    typedef int iv __attribute__((ext_vector_type(V / 2)));
    iv bits = __builtin_bit_cast(iv, v);
#pragma unroll
    for (int i = 0; i < V / 2; ++i) bits[i] = __shfl_xor(bits[i], mask, 64);
    return __builtin_bit_cast(hv, bits);
  }
}
// a / b rounded once to f16: the correctly rounded f32 quotient of two f16 values rounds to the correctly rounded
// f16 quotient (24 >= 2 * 11 + 2 bits).  The empty asm keeps the division an f32 division: folded into an f16
// division the compiler may use the f16 reciprocal, which is accurate to one unit in the last place only.
__device__ __forceinline__ _Float16 div_f16(_Float16 a, _Float16 b) {
  float q = (float)a / (float)b;
  asm volatile("" : "+v"(q));
  return (_Float16)q;
}
// sqrt(v) rounded toward minus infinity in f16 (rounding::NegativeInf of the tile program): the f32 square
// root of an f16 value, truncated to f16, is at most one f16 step above the exact floor, and exactly when its
// square (exact in f32: 22 bits) exceeds v.
__device__ __forceinline__ _Float16 sqrt_f16_toward_minus_infinity(_Float16 v) {
  const float f = __builtin_sqrtf((float)v);
  if (!(f <= 65504.0f) || f == 0.0f) return (_Float16)f;          // NaN (negative input), +inf, +-0
  uint16_t bits = (uint16_t)((__builtin_bit_cast(uint32_t, f) >> 13) - (112u << 10));   // truncation; sqrt of an f16 is a normal f16
  const float h = (float)__builtin_bit_cast(_Float16, bits);
  if (h * h > (float)v) bits -= 1;
  return __builtin_bit_cast(_Float16, bits);
}

// rms_norm<N, BLOCK_SIZE> of cutile-benchmarks/benches/rmsnorm.rs:20-66.  V = tile lanes per lane of the
// wavefront: BLOCK_SIZE = 64 * V, or BLOCK_SIZE <= 64 with V = 1 (the lanes beyond it hold zeros).
template <int V>
__device__ __forceinline__ void rms_norm_all_f16_rows(const TensorArg<2>& x, const TensorArg<1>& w, const PartitionArg<2>& out,
                                                      float eps_f32, int32_t block_size, int64_t rows) {
#pragma clang fp contract(off)
  typedef _Float16 hv __attribute__((ext_vector_type(V)));
  constexpr int kCached = V >= 16 ? 8 : 16;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int32_t n = x.shape[1], tiles = n / block_size;
  const bool active = lane * V < block_size;
  const _Float16 eps = (_Float16)eps_f32;
  for (int64_t row = (int64_t)blockIdx.x * kWaves + wave; row < rows; row += (int64_t)gridDim.x * kWaves) {
    const _Float16* xr = (const _Float16*)x.ptr + row * x.strides[0];
    _Float16* orow = (_Float16*)out.ptr + row * out.strides[0];
    _Float16 acc[V];
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = (_Float16)0.0f;
    // The first kCached tiles of the row stay in registers for the second pass (all of a row of up to
    // kCached * BLOCK_SIZE elements: read from memory once); their loads are issued together.
    hv cached[kCached];
    if (active) {
#pragma unroll
      for (int j = 0; j < kCached; ++j)     // tiles past the row's end repeat the last one (loaded, never used)
        cached[j] = __builtin_nontemporal_load(reinterpret_cast<const hv*>(xr + (int64_t)min(j, tiles - 1) * block_size + lane * V));
#pragma unroll
      for (int j = 0; j < kCached; ++j)
        if (j < tiles) {
#pragma unroll
          for (int e = 0; e < V; ++e) {
            const _Float16 sq = cached[j][e] * cached[j][e];
            acc[e] = acc[e] + sq;
          }
        }
      for (int32_t j = kCached; j < tiles; ++j) {
        const hv t = *reinterpret_cast<const hv*>(xr + (int64_t)j * block_size + lane * V);
#pragma unroll
        for (int e = 0; e < V; ++e) {
          const _Float16 sq = t[e] * t[e];
          acc[e] = acc[e] + sq;
        }
      }
    }
    {
      hv av;
#pragma unroll
      for (int e = 0; e < V; ++e) av[e] = acc[e];
#pragma unroll
      for (int step = 32; step >= 1; step >>= 1) av = av + shfl_xor_hv<V>(av, step);
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] = av[e];
    }
#pragma unroll
    for (int step = V / 2; step >= 1; step >>= 1)
#pragma unroll
      for (int e = 0; e < step; ++e) acc[e] = acc[e] + acc[e + step];
    // rms = sqrt(1 / (sum / N + eps)), each step an f16 operation (:46-52)
    const _Float16 mean = div_f16(acc[0], (_Float16)(float)n);
    const _Float16 denom = mean + eps;
    const _Float16 inv = div_f16((_Float16)1.0f, denom);
    const _Float16 scale = sqrt_f16_toward_minus_infinity(inv);
    if (active) {
      auto emit = [&](int32_t j, const hv& t, const hv& tw) {
        hv o;
#pragma unroll
        for (int e = 0; e < V; ++e) {
          const _Float16 scaled = t[e] * scale;
          o[e] = scaled * tw[e];
        }
        __builtin_nontemporal_store(o, reinterpret_cast<hv*>(orow + (int64_t)j * block_size + lane * V));
      };
      const _Float16* wl = (const _Float16*)w.ptr + lane * V;
      // The weights of the cached tiles come four tiles at a time, the next four on their way while these are used
      // (tiles past the row's end repeat the last one: loaded, never used).
      constexpr int kGroup = 4, kGroups = kCached / kGroup;
      hv wc[2][kGroup];
      auto fetch_w = [&](int g) {
#pragma unroll
        for (int i = 0; i < kGroup; ++i) wc[g & 1][i] = *reinterpret_cast<const hv*>(wl + (int64_t)min(g * kGroup + i, tiles - 1) * block_size);
      };
      fetch_w(0);
#pragma unroll
      for (int g = 0; g < kGroups; ++g) {
        if (g + 1 < kGroups) fetch_w(g + 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < kGroup; ++i)
          if (g * kGroup + i < tiles) emit(g * kGroup + i, cached[g * kGroup + i], wc[g & 1][i]);
        __builtin_amdgcn_sched_barrier(0);
      }
      for (int32_t j = kCached; j < tiles; ++j)
        emit(j, *reinterpret_cast<const hv*>(xr + (int64_t)j * block_size + lane * V), *reinterpret_cast<const hv*>(wl + (int64_t)j * block_size));
    }
  }
}

// softmax<BM, BN> of cutile-benchmarks/benches/softmax.rs:19-35 over one tile row (a "segment" of BN columns):
// CH chunks of 64 * V columns.  Columns of the tile beyond the tensor read 0 and take part (padding::Zero).
template <int CH, int V>
__device__ __forceinline__ void softmax_all_f16_segments(const TensorArg<2>& x, const PartitionArg<2>& y, int32_t segs_per_row,
                                                         int64_t n_segments) {
#pragma clang fp contract(off)
  typedef _Float16 hv __attribute__((ext_vector_type(V)));
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int32_t bn = y.pshape[1], n_cols = x.shape[1];
  const bool active = lane * V < bn;
  for (int64_t seg = (int64_t)blockIdx.x * kWaves + wave; seg < n_segments; seg += (int64_t)gridDim.x * kWaves) {
    const int64_t row = seg / segs_per_row;
    const int32_t col0 = (int32_t)(seg % segs_per_row) * bn;
    const _Float16* xr = (const _Float16*)x.ptr + row * x.strides[0];
    _Float16* yr = (_Float16*)y.ptr + row * y.strides[0];
    hv a[CH];
    if (bn == CH * 64 * V && col0 + bn <= n_cols) {
      // the whole tile row lies inside the tensor: nothing but vector loads, all requested before the first use
      // (an element-wise path between them would make every chunk wait for the one before: CH memory latencies)
#pragma unroll
      for (int c = 0; c < CH; ++c)
        a[c] = __builtin_nontemporal_load(reinterpret_cast<const hv*>(xr + col0 + c * 64 * V + lane * V));   // streamed: read once
    } else {
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const int32_t col = col0 + c * 64 * V + lane * V;
        if (active && col + V <= n_cols) {
          a[c] = __builtin_nontemporal_load(reinterpret_cast<const hv*>(xr + col));
        } else {
#pragma unroll
          for (int e = 0; e < V; ++e) a[c][e] = (active && col + e < n_cols) ? xr[col + e] : (_Float16)0.0f;
        }
      }
    }
    hv mv = a[0];
#pragma unroll
    for (int c = 1; c < CH; ++c) mv = __builtin_elementwise_max(mv, a[c]);
    _Float16 mx = mv[0];
#pragma unroll
    for (int e = 1; e < V; ++e) mx = mv[e] > mx ? mv[e] : mx;
    if (!active) mx = (_Float16)(-__builtin_inff());
#pragma unroll
    for (int step = 32; step >= 1; step >>= 1) {
      const _Float16 o = shfl_xor_f16(mx, step);
      mx = o > mx ? o : mx;
    }
    // num = exp(x - max): the difference is an f16 operation, the exponential is evaluated in f32 and rounded once
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const hv d = a[c] - mx;
#pragma unroll
      for (int e = 0; e < V; ++e) a[c][e] = active ? (_Float16)__builtin_amdgcn_exp2f((float)d[e] * kLog2e) : (_Float16)0.0f;
      __builtin_amdgcn_sched_barrier(0);      // chunk by chunk: the f32 intermediates of one chunk only are live
    }
    // denom = reduce_sum(num): chunks first (the tree's largest steps), then across lanes, then inside the lane
    constexpr int H = CH > 1 ? CH / 2 : 1;
    hv t[H];
#pragma unroll
    for (int c = 0; c < H; ++c) t[c] = CH > 1 ? a[c] + a[c + H] : a[c];
#pragma unroll
    for (int step = H / 2; step >= 1; step >>= 1)
#pragma unroll
      for (int c = 0; c < step; ++c) t[c] = t[c] + t[c + step];
    hv tot = t[0];
#pragma unroll
    for (int step = 32; step >= 1; step >>= 1) tot = tot + shfl_xor_hv<V>(tot, step);
#pragma unroll
    for (int step = V / 2; step >= 1; step >>= 1)
#pragma unroll
      for (int e = 0; e < step; ++e) tot[e] = tot[e] + tot[e + step];
    // num / denom, rounded once to f16: q0 = num * (1 / denom) corrected by its own residual is within 2^-24 (1 + 2^-20)
    // of the quotient, and the quotient of two f16 values is either exactly on an f16 rounding boundary (then q is
    // exact) or at least 2^-23 away from one, so q rounds to f16 as the exact quotient does.
    const float denom = (float)tot[0];
    const float recip = __builtin_amdgcn_rcpf(denom);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int32_t col = col0 + c * 64 * V + lane * V;
      hv o;
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const float num = (float)a[c][e];
        const float q0 = num * recip;
        o[e] = (_Float16)__builtin_fmaf(__builtin_fmaf(-q0, denom, num), recip, q0);
      }
      if (active && col + V <= n_cols) {
        __builtin_nontemporal_store(o, reinterpret_cast<hv*>(yr + col));
      } else if (active) {
#pragma unroll
        for (int e = 0; e < V; ++e)
          if (col + e < n_cols) yr[col + e] = o[e];
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

}  // namespace

#define RMS_NORM_ALL_F16_KERNEL(V)                                                                                   \
  extern "C" __global__ void __launch_bounds__(kThreads) rms_norm_all_f16_entry__v##V(                               \
      TensorArg<2> x, TensorArg<1> w, PartitionArg<2> out, float eps, int32_t block_size, TileGrid g) {              \
    rms_norm_all_f16_rows<V>(x, w, out, eps, block_size, min((int64_t)g.x, (int64_t)out.shape[0]));                  \
  }
RMS_NORM_ALL_F16_KERNEL(1)
RMS_NORM_ALL_F16_KERNEL(2)
RMS_NORM_ALL_F16_KERNEL(4)
RMS_NORM_ALL_F16_KERNEL(8)
RMS_NORM_ALL_F16_KERNEL(16)

#define SOFTMAX_ALL_F16_KERNEL(CH, V)                                                                                \
  extern "C" __global__ void __launch_bounds__(kThreads) softmax_all_f16_entry__c##CH##v##V(                         \
      TensorArg<2> x, PartitionArg<2> y, TileGrid g) {                                                               \
    const int64_t rows = min((int64_t)g.x * y.pshape[0], (int64_t)y.shape[0]);                                       \
    softmax_all_f16_segments<CH, V>(x, y, (int32_t)g.y, rows * (int64_t)g.y);                                        \
  }
SOFTMAX_ALL_F16_KERNEL(1, 1)
SOFTMAX_ALL_F16_KERNEL(1, 2)
SOFTMAX_ALL_F16_KERNEL(1, 4)
SOFTMAX_ALL_F16_KERNEL(1, 8)
SOFTMAX_ALL_F16_KERNEL(2, 8)
SOFTMAX_ALL_F16_KERNEL(4, 8)
SOFTMAX_ALL_F16_KERNEL(8, 8)
SOFTMAX_ALL_F16_KERNEL(16, 8)
SOFTMAX_ALL_F16_KERNEL(32, 8)

// softmax(x, y: [BM, BN] tiles).  g.x / g.y = tiles covered along rows / columns.
#define SOFTMAX_KERNEL(T, NAME, WPR, VPL)                                                           \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      softmax_entry__##NAME##_w##WPR##v##VPL(TensorArg<2> x, PartitionArg<2> y, TileGrid g) {       \
    int64_t rows = min((int64_t)g.x * y.pshape[0], (int64_t)y.shape[0]);                           \
    softmax_segments<T, WPR, VPL>((const T*)x.ptr, x.strides[0], (T*)y.ptr, y.strides[0],          \
                                  x.shape[1], y.shape[1], y.pshape[1], (int32_t)g.y,               \
                                  rows * (int64_t)g.y);                                            \
  }

#define SOFTMAX_VARIANTS(T, NAME) \
  SOFTMAX_KERNEL(T, NAME, 1, 1)   \
  SOFTMAX_KERNEL(T, NAME, 1, 2)   \
  SOFTMAX_KERNEL(T, NAME, 1, 4)   \
  SOFTMAX_KERNEL(T, NAME, 1, 8)   \
  SOFTMAX_KERNEL(T, NAME, 1, 16)  \
  SOFTMAX_KERNEL(T, NAME, 2, 2)   \
  SOFTMAX_KERNEL(T, NAME, 2, 4)   \
  SOFTMAX_KERNEL(T, NAME, 2, 8)   \
  SOFTMAX_KERNEL(T, NAME, 4, 1)   \
  SOFTMAX_KERNEL(T, NAME, 4, 2)   \
  SOFTMAX_KERNEL(T, NAME, 4, 4)   \
  SOFTMAX_KERNEL(T, NAME, 4, 8)   \
  SOFTMAX_KERNEL(T, NAME, 4, 16)

SOFTMAX_VARIANTS(_Float16, f16)
SOFTMAX_VARIANTS(float, f32)

#define SOFTMAX_GENERIC(T, NAME)                                                                    \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      softmax_entry__##NAME##_generic(TensorArg<2> x, PartitionArg<2> y, TileGrid g) {              \
    int64_t rows = min((int64_t)g.x * y.pshape[0], (int64_t)y.shape[0]);                           \
    softmax_segment_generic<T>(x, y, (int32_t)g.y, rows * (int64_t)g.y);                           \
  }
SOFTMAX_GENERIC(_Float16, f16)
SOFTMAX_GENERIC(float, f32)
