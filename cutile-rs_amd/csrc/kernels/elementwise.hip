// Elementwise and creation kernels for gfx950: saxpy, axpy with a separate
// output, add, full, arange, linspace, eye, convert, and the example programs'
// relu, dropout, scale_ptr and matvec.
//
// Bodies follow the reference's tile programs:
//   saxpy    cutile-examples/examples/saxpy.rs:12-17, async_saxpy.rs:21-30
//   add      README.md:29-38, cutile/tests/gpu/add_basic.rs:16-25
//   full / arange / linspace   cutile/src/kernels/_creation.rs:44-47,79-87,94-108
//   convert  cutile/src/kernels/_conversion.rs:78-85
// Tile semantics kept: an input loaded "like" the output tile reads 0 outside
// its own extent (cutile/src/_core.rs:3405-3504, padding::Zero); stores outside
// the output extent are dropped; only tiles inside the launch grid are written.
//
// These are pure HBM streams, so the only thing that matters is bytes in flight:
// the *_flat variants (contiguous operands of equal shape) ignore tile geometry,
// move 16 bytes per lane per access and keep four accesses per lane in flight.
// The *_tiled variants honour arbitrary strides, extents and partial grids.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_bf16.h>

#include "kernel_args.h"
#include "lane_exchange.h"
#include "mapped_partition.h"

using namespace cutile;

namespace {

constexpr int kThreads = 256;
constexpr int kUnroll = 4;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// 16 bytes moved as one dwordx4 access and viewed as elements of T.
template <typename T>
union Vec16 {
  static constexpr int N = 16 / sizeof(T);
  u32x4 raw;
  T v[N];
  __device__ Vec16() : raw{} {}
};

template <typename T>
__device__ __forceinline__ T fma_t(T a, T x, T y);
template <>
__device__ __forceinline__ float fma_t<float>(float a, float x, float y) {
  return __builtin_fmaf(a, x, y);
}
template <>
__device__ __forceinline__ double fma_t<double>(double a, double x, double y) {
  return __builtin_fma(a, x, y);
}
template <>
__device__ __forceinline__ _Float16 fma_t<_Float16>(_Float16 a, _Float16 x, _Float16 y) {
  return __builtin_fmaf16(a, x, y);
}

// Number of leading elements (flat order) that a rank-1 launch grid covers.
__device__ __forceinline__ size_t covered_1d(int32_t n, int32_t tile, const TileGrid& g) {
  size_t c = (size_t)g.x * (size_t)tile;
  return c < (size_t)n ? c : (size_t)n;
}

// ---- flat streams ------------------------------------------------------------------------
// Each workgroup owns kThreads*kUnroll consecutive 16-byte vectors.  `count` is
// the number of elements to process; the tail (count % N) is handled scalar by
// the last workgroup.
template <typename T, typename F>
__device__ __forceinline__ void flat_stream3(T* __restrict__ out, const T* __restrict__ in0,
                                             const T* __restrict__ in1, size_t count, F f) {
  using V = Vec16<T>;
  const size_t nvec = count / V::N;
  const size_t base = (size_t)blockIdx.x * (kThreads * kUnroll) + threadIdx.x;
  V a[kUnroll], b[kUnroll];
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    size_t i = base + (size_t)u * kThreads;
    if (i < nvec) {
      a[u].raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(in0) + i);
      b[u].raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(in1) + i);
    }
  }
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    size_t i = base + (size_t)u * kThreads;
    if (i < nvec) {
      V r;
#pragma unroll
      for (int e = 0; e < V::N; ++e) r.v[e] = f(a[u].v[e], b[u].v[e]);
      __builtin_nontemporal_store(r.raw, reinterpret_cast<u32x4*>(out) + i);
    }
  }
  if (blockIdx.x == gridDim.x - 1) {
    size_t i = nvec * V::N + threadIdx.x;
    if (i < count) out[i] = f(in0[i], in1[i]);
  }
}

template <typename T>
__device__ __forceinline__ T load_padded(const T* p, const int32_t* shape, const int32_t* strides,
                                         const int32_t* idx, int rank) {
  int64_t off = 0;
  for (int d = 0; d < rank; ++d) {
    if (idx[d] >= shape[d]) return T(0);
    off += (int64_t)idx[d] * strides[d];
  }
  return p[off];
}

// Walks every element of the tile this workgroup owns (blockIdx = tile index),
// calling body(idx[R], out_offset) for in-bounds output elements.
template <int R, typename P, typename F>
__device__ __forceinline__ void for_each_tile_elem(const P& out, F body) {
  int32_t pid[3] = {(int32_t)blockIdx.x, (int32_t)blockIdx.y, (int32_t)blockIdx.z};
  int64_t tile_elems = 1;
  for (int d = 0; d < R; ++d) tile_elems *= out.pshape[d];
  for (int64_t e = threadIdx.x; e < tile_elems; e += blockDim.x) {
    int32_t idx[R];
    int64_t rem = e;
    bool ok = true;
    int64_t off = 0;
    for (int d = R - 1; d >= 0; --d) {
      int32_t in_tile = (int32_t)(rem % out.pshape[d]);
      rem /= out.pshape[d];
      idx[d] = pid[d] * out.pshape[d] + in_tile;
      ok = ok && idx[d] < out.shape[d];
      off += (int64_t)idx[d] * out.strides[d];
    }
    if (ok) body(idx, off);
  }
}

// out[i * stride] = f(i) for i < count: 16 bytes per lane where the layout allows it
// (unit stride, 16-byte aligned base), element by element otherwise and for the tail.
template <typename T, typename F>
__device__ __forceinline__ void flat_generate(T* out, int64_t stride, size_t count, F f) {
  const size_t step = (size_t)gridDim.x * kThreads, gid = (size_t)blockIdx.x * kThreads + threadIdx.x;
  size_t done = 0;
  if (stride == 1 && ((uintptr_t)out & 15) == 0) {
    using V = Vec16<T>;
    const size_t nvec = count / V::N;
    for (size_t j = gid; j < nvec; j += step) {
      V r;
#pragma unroll
      for (int e = 0; e < V::N; ++e) r.v[e] = f(j * V::N + e);
      reinterpret_cast<u32x4*>(out)[j] = r.raw;
    }
    done = nvec * V::N;
  }
  for (size_t i = done + gid; i < count; i += step) out[(int64_t)i * stride] = f(i);
}

template <typename D, typename S>
__device__ __forceinline__ D convert_elem(S v) {
  return (D)v;
}
// The two 16-bit float formats convert through f32 (exact in that direction).
template <>
__device__ __forceinline__ __bf16 convert_elem<__bf16, _Float16>(_Float16 v) {
  return (__bf16)(float)v;
}
template <>
__device__ __forceinline__ _Float16 convert_elem<_Float16, __bf16>(__bf16 v) {
  return (_Float16)(float)v;
}

// dst[i] = convert(src[i]) for i < count, zero where src has no element i.  Streams of
// unit stride and 16-byte aligned bases move kElems elements per lane and pass (16 bytes of the
// narrower type, 16 to 64 of the wider), nontemporally; the rest goes element by element.
template <typename D, typename S>
__device__ __forceinline__ void flat_convert(const S* src, int64_t src_stride, size_t src_count, D* dst,
                                             int64_t dst_stride, size_t count) {
  constexpr int kElems = 16 / (sizeof(S) < sizeof(D) ? sizeof(S) : sizeof(D));
  constexpr int kSrcVecs = kElems * sizeof(S) / 16, kDstVecs = kElems * sizeof(D) / 16;
  const size_t step = (size_t)gridDim.x * kThreads, gid = (size_t)blockIdx.x * kThreads + threadIdx.x;
  size_t done = 0;
  if (src_stride == 1 && dst_stride == 1 && (((uintptr_t)src | (uintptr_t)dst) & 15) == 0) {
    // a workgroup takes kThreads * kGroups consecutive groups of kElems elements at a time and requests all of a
    // lane's loads before it converts the first value (at least 64 bytes in flight per lane)
    constexpr int kGroups = kSrcVecs >= 4 ? 1 : kSrcVecs == 2 ? 2 : 4;
    const size_t nvec = (count < src_count ? count : src_count) / kElems;
    for (size_t j0 = (size_t)blockIdx.x * (kThreads * kGroups) + threadIdx.x; j0 < nvec; j0 += step * kGroups) {
      union { u32x4 raw[kSrcVecs]; S v[kElems]; } in[kGroups];
#pragma unroll
      for (int u = 0; u < kGroups; ++u) {
        const size_t j = j0 + (size_t)u * kThreads;
        if (j < nvec) {
#pragma unroll
          for (int q = 0; q < kSrcVecs; ++q) in[u].raw[q] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src) + j * kSrcVecs + q);
        }
      }
#pragma unroll
      for (int u = 0; u < kGroups; ++u) {
        const size_t j = j0 + (size_t)u * kThreads;
        if (j < nvec) {
          union { u32x4 raw[kDstVecs]; D v[kElems]; } out;
#pragma unroll
          for (int e = 0; e < kElems; ++e) out.v[e] = convert_elem<D, S>(in[u].v[e]);
#pragma unroll
          for (int q = 0; q < kDstVecs; ++q) __builtin_nontemporal_store(out.raw[q], reinterpret_cast<u32x4*>(dst) + j * kDstVecs + q);
        }
      }
    }
    done = nvec * kElems;
  }
  for (size_t i = done + gid; i < count; i += step) {
    const S v = i < src_count ? src[(int64_t)i * src_stride] : S(0);
    dst[(int64_t)i * dst_stride] = convert_elem<D, S>(v);
  }
}

// dst[i] = f(src[i]) for i < count, with src read as 0 where it has no element i (a tile loaded "like" the output
// is zero-padded).  src may be dst (an update in place: every lane reads what it then writes).  Unit strides and
// 16-byte aligned bases move 16 bytes per lane and access; anything else goes element by element, like the tail.
template <typename T, typename F>
__device__ __forceinline__ void flat_map1(const T* src, int64_t src_stride, size_t src_count, T* dst, int64_t dst_stride,
                                          size_t count, F f) {
  using V = Vec16<T>;
  const size_t step = (size_t)gridDim.x * kThreads, gid = (size_t)blockIdx.x * kThreads + threadIdx.x;
  size_t done = 0;
  if (src_stride == 1 && dst_stride == 1 && (((uintptr_t)src | (uintptr_t)dst) & 15) == 0) {
    // a workgroup takes kThreads * kUnroll consecutive vectors at a time: kUnroll nontemporal loads in flight per
    // lane, then the stores (a stream touched once should not push other data out of the caches)
    const size_t nvec = (count < src_count ? count : src_count) / V::N;
    for (size_t j0 = (size_t)blockIdx.x * (kThreads * kUnroll) + threadIdx.x; j0 < nvec; j0 += step * kUnroll) {
      V in[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
        if (j0 + (size_t)u * kThreads < nvec) in[u].raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src) + j0 + (size_t)u * kThreads);
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
        if (j0 + (size_t)u * kThreads < nvec) {
          V out;
#pragma unroll
          for (int e = 0; e < V::N; ++e) out.v[e] = f(in[u].v[e]);
          __builtin_nontemporal_store(out.raw, reinterpret_cast<u32x4*>(dst) + j0 + (size_t)u * kThreads);
        }
    }
    done = nvec * V::N;
  }
  for (size_t i = done + gid; i < count; i += step) {
    const T v = i < src_count ? src[(int64_t)i * src_stride] : T(0);
    dst[(int64_t)i * dst_stride] = f(v);
  }
}

}  // namespace

// ---- saxpy: y <- a*x + y -------------------------------------------------------------------
#define SAXPY_KERNELS(T, NAME)                                                                      \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      saxpy_entry__##NAME##_r1_flat(PartitionArg<1> y, T a, TensorArg<1> x, TileGrid g) {          \
    size_t count = covered_1d(y.shape[0], y.pshape[0], g);                                         \
    flat_stream3<T>((T*)y.ptr, (const T*)x.ptr, (const T*)y.ptr, count,                            \
                    [a](T xv, T yv) { return fma_t<T>(a, xv, yv); });                              \
  }                                                                                                 \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      saxpy_entry__##NAME##_r2_flat(PartitionArg<2> y, T a, TensorArg<2> x, TileGrid g) {          \
    size_t count = (size_t)y.shape[0] * (size_t)y.shape[1];                                        \
    flat_stream3<T>((T*)y.ptr, (const T*)x.ptr, (const T*)y.ptr, count,                            \
                    [a](T xv, T yv) { return fma_t<T>(a, xv, yv); });                              \
  }                                                                                                 \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      saxpy_entry__##NAME##_r1_tiled(PartitionArg<1> y, T a, TensorArg<1> x, TileGrid g) {         \
    for_each_tile_elem<1>(y, [&](const int32_t* idx, int64_t off) {                                \
      T xv = load_padded<T>((const T*)x.ptr, x.shape, x.strides, idx, 1);                          \
      T* yp = (T*)y.ptr + off;                                                                     \
      *yp = fma_t<T>(a, xv, *yp);                                                                  \
    });                                                                                             \
  }                                                                                                 \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      saxpy_entry__##NAME##_r2_tiled(PartitionArg<2> y, T a, TensorArg<2> x, TileGrid g) {         \
    for_each_tile_elem<2>(y, [&](const int32_t* idx, int64_t off) {                                \
      T xv = load_padded<T>((const T*)x.ptr, x.shape, x.strides, idx, 2);                          \
      T* yp = (T*)y.ptr + off;                                                                     \
      *yp = fma_t<T>(a, xv, *yp);                                                                  \
    });                                                                                             \
  }                                                                                                 \
  /* z <- a*x + y with a separate output (rank 1) */                                               \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      axpy_entry__##NAME##_r1_flat(PartitionArg<1> z, T a, TensorArg<1> x, TensorArg<1> y,         \
                                   TileGrid g) {                                                    \
    size_t count = covered_1d(z.shape[0], z.pshape[0], g);                                         \
    flat_stream3<T>((T*)z.ptr, (const T*)x.ptr, (const T*)y.ptr, count,                            \
                    [a](T xv, T yv) { return fma_t<T>(a, xv, yv); });                              \
  }                                                                                                 \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      axpy_entry__##NAME##_r1_tiled(PartitionArg<1> z, T a, TensorArg<1> x, TensorArg<1> y,        \
                                    TileGrid g) {                                                   \
    for_each_tile_elem<1>(z, [&](const int32_t* idx, int64_t off) {                                \
      T xv = load_padded<T>((const T*)x.ptr, x.shape, x.strides, idx, 1);                          \
      T yv = load_padded<T>((const T*)y.ptr, y.shape, y.strides, idx, 1);                          \
      ((T*)z.ptr)[off] = fma_t<T>(a, xv, yv);                                                      \
    });                                                                                             \
  }

SAXPY_KERNELS(float, f32)
SAXPY_KERNELS(_Float16, f16)
SAXPY_KERNELS(double, f64)

// ---- add: z <- x + y -----------------------------------------------------------------------
#define ADD_KERNELS(T, NAME)                                                                        \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      add_entry__##NAME##_r1_flat(PartitionArg<1> z, TensorArg<1> x, TensorArg<1> y, TileGrid g) { \
    size_t count = covered_1d(z.shape[0], z.pshape[0], g);                                         \
    flat_stream3<T>((T*)z.ptr, (const T*)x.ptr, (const T*)y.ptr, count,                            \
                    [](T xv, T yv) { return (T)(xv + yv); });                                      \
  }                                                                                                 \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      add_entry__##NAME##_r1_tiled(PartitionArg<1> z, TensorArg<1> x, TensorArg<1> y,              \
                                   TileGrid g) {                                                    \
    for_each_tile_elem<1>(z, [&](const int32_t* idx, int64_t off) {                                \
      T xv = load_padded<T>((const T*)x.ptr, x.shape, x.strides, idx, 1);                          \
      T yv = load_padded<T>((const T*)y.ptr, y.shape, y.strides, idx, 1);                          \
      ((T*)z.ptr)[off] = (T)(xv + yv);                                                             \
    });                                                                                             \
  }                                                                                                 \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      add_entry__##NAME##_r2_tiled(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y,              \
                                   TileGrid g) {                                                    \
    for_each_tile_elem<2>(z, [&](const int32_t* idx, int64_t off) {                                \
      T xv = load_padded<T>((const T*)x.ptr, x.shape, x.strides, idx, 2);                          \
      T yv = load_padded<T>((const T*)y.ptr, y.shape, y.strides, idx, 2);                          \
      ((T*)z.ptr)[off] = (T)(xv + yv);                                                             \
    });                                                                                             \
  }

ADD_KERNELS(float, f32)
ADD_KERNELS(_Float16, f16)
ADD_KERNELS(__bf16, bf16)

// rank-2 flat form (add_2d_f16 of cutile-kernels/src/pointwise.rs:15-40 is add<f16> on [1, BLOCK] tiles)
#define ADD_R2_FLAT(T, NAME)                                                                        \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      add_entry__##NAME##_r2_flat(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y, TileGrid g) { \
    flat_stream3<T>((T*)z.ptr, (const T*)x.ptr, (const T*)y.ptr, (size_t)z.shape[0] * z.shape[1],  \
                    [](T xv, T yv) { return (T)(xv + yv); });                                      \
  }
ADD_R2_FLAT(float, f32)
ADD_R2_FLAT(_Float16, f16)
ADD_R2_FLAT(__bf16, bf16)

// ---- silu_mul_2d_f16: out <- sigmoid(gate) * gate * up, f32 math ---------------------------
// cutile-kernels/src/pointwise.rs:46-78: sigmoid = 1 / (1 + exp(0 - gate)).
__device__ __forceinline__ _Float16 silu_mul(_Float16 gate, _Float16 up) {
  const float g = (float)gate, u = (float)up;
  const float sig = 1.0f / (1.0f + __builtin_amdgcn_exp2f((0.0f - g) * 1.4426950408889634f));
  return (_Float16)(sig * g * u);
}
extern "C" __global__ void __launch_bounds__(kThreads)
    silu_mul_2d_f16_entry__f16_r2_flat(PartitionArg<2> out, TensorArg<2> gate, TensorArg<2> up, TileGrid g) {
  flat_stream3<_Float16>((_Float16*)out.ptr, (const _Float16*)gate.ptr, (const _Float16*)up.ptr,
                         (size_t)out.shape[0] * out.shape[1], [](_Float16 a, _Float16 b) { return silu_mul(a, b); });
}
extern "C" __global__ void __launch_bounds__(kThreads)
    silu_mul_2d_f16_entry__f16_r2_tiled(PartitionArg<2> out, TensorArg<2> gate, TensorArg<2> up, TileGrid g) {
  for_each_tile_elem<2>(out, [&](const int32_t* idx, int64_t off) {
    _Float16 gv = load_padded<_Float16>((const _Float16*)gate.ptr, gate.shape, gate.strides, idx, 2);
    _Float16 uv = load_padded<_Float16>((const _Float16*)up.ptr, up.shape, up.strides, idx, 2);
    ((_Float16*)out.ptr)[off] = silu_mul(gv, uv);
  });
}

// ---- KV cache update ------------------------------------------------------------------------
// kv_cache_update_seq_f16 / kv_cache_update_seq_dynpos_f16 (cutile-kernels/src/kv_cache.rs:15-49,
// 58-97): cache[h, position_start + s, :] = new[s, h, :] for s < seq_len, K and V together.
// new_* are [seq, heads, D], the caches [heads, max_seq, D].  Rows that would land
// beyond max_seq are dropped.  16 bytes per lane when the layout allows it.
extern "C" __global__ void __launch_bounds__(kThreads)
    kv_cache_update_entry__f16(TensorArg<3> new_k, TensorArg<3> new_v, PartitionArg<3> k_cache, PartitionArg<3> v_cache,
                               const uint32_t* pos_dev, int32_t position_start, int32_t seq_len, TileGrid g) {
  const int32_t d = new_k.shape[2], heads = min((int32_t)g.x, k_cache.shape[0]);
  const int32_t base = pos_dev ? (int32_t)pos_dev[0] : position_start;
  const int32_t max_seq = min(k_cache.shape[1], v_cache.shape[1]);
  auto vec_ok = [&](const void* p, const int32_t* st) {
    return st[2] == 1 && st[1] % 8 == 0 && st[0] % 8 == 0 && ((uintptr_t)p & 15) == 0;
  };
  const bool vec = d % 8 == 0 && vec_ok(new_k.ptr, new_k.strides) && vec_ok(new_v.ptr, new_v.strides) &&
                   vec_ok(k_cache.ptr, k_cache.strides) && vec_ok(v_cache.ptr, v_cache.strides);
  const int32_t per_row = vec ? d / 8 : d;
  const int64_t total = (int64_t)seq_len * heads * per_row;
  if (vec && (per_row & (per_row - 1)) == 0 && per_row <= kThreads && (int64_t)seq_len * heads < (1ll << 31)) {
    // Head rows of 8, 16 or 32 vectors (D = 64, 128, 256): a lane keeps its place in the row and groups of lanes walk
    // the (position, head) rows, so an item costs one 32-bit division.  The general walk below takes four 64-bit
    // divisions per item, which is more vector work than the copy is memory work.
    const uint32_t shift = (uint32_t)__builtin_ctz((uint32_t)per_row);
    const uint32_t c = threadIdx.x & (uint32_t)(per_row - 1), rows_per_wg = (uint32_t)kThreads >> shift;
    const uint32_t n_rows = (uint32_t)seq_len * (uint32_t)heads;
    for (uint32_t r = blockIdx.x * rows_per_wg + (threadIdx.x >> shift); r < n_rows; r += gridDim.x * rows_per_wg) {
      const uint32_t sidx = r / (uint32_t)heads, h = r - sidx * (uint32_t)heads;
      const int64_t pos = (int64_t)base + sidx;
      if (pos < 0 || pos >= max_seq) continue;
      const u32x4 kv = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(
          (const _Float16*)new_k.ptr + (int64_t)sidx * new_k.strides[0] + (int64_t)h * new_k.strides[1]) + c);
      const u32x4 vv = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(
          (const _Float16*)new_v.ptr + (int64_t)sidx * new_v.strides[0] + (int64_t)h * new_v.strides[1]) + c);
      __builtin_nontemporal_store(kv, reinterpret_cast<u32x4*>((_Float16*)k_cache.ptr + (int64_t)h * k_cache.strides[0] + pos * k_cache.strides[1]) + c);
      __builtin_nontemporal_store(vv, reinterpret_cast<u32x4*>((_Float16*)v_cache.ptr + (int64_t)h * v_cache.strides[0] + pos * v_cache.strides[1]) + c);
    }
    return;
  }
  for (int64_t t = (int64_t)blockIdx.x * kThreads + threadIdx.x; t < total; t += (int64_t)gridDim.x * kThreads) {
    const int32_t c = (int32_t)(t % per_row);
    const int64_t sh = t / per_row;
    const int32_t h = (int32_t)(sh % heads);
    const int64_t sidx = sh / heads;
    const int64_t pos = base + sidx;
    if (pos < 0 || pos >= max_seq) continue;
    const int64_t src_k = sidx * new_k.strides[0] + (int64_t)h * new_k.strides[1];
    const int64_t src_v = sidx * new_v.strides[0] + (int64_t)h * new_v.strides[1];
    const int64_t dst_k = (int64_t)h * k_cache.strides[0] + pos * k_cache.strides[1];
    const int64_t dst_v = (int64_t)h * v_cache.strides[0] + pos * v_cache.strides[1];
    if (vec) {
      // Streamed both ways: the new rows are read once, and a plain load or store would take a place in the
      // memory-side cache, pushing out whatever dirty lines the previous kernel left there at the cost of their
      // write-back.
      const u32x4 kv = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>((const _Float16*)new_k.ptr + src_k + c * 8));
      const u32x4 vv = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>((const _Float16*)new_v.ptr + src_v + c * 8));
      __builtin_nontemporal_store(kv, reinterpret_cast<u32x4*>((_Float16*)k_cache.ptr + dst_k + c * 8));
      __builtin_nontemporal_store(vv, reinterpret_cast<u32x4*>((_Float16*)v_cache.ptr + dst_v + c * 8));
    } else {
      ((_Float16*)k_cache.ptr)[dst_k + (int64_t)c * k_cache.strides[2]] = ((const _Float16*)new_k.ptr)[src_k + (int64_t)c * new_k.strides[2]];
      ((_Float16*)v_cache.ptr)[dst_v + (int64_t)c * v_cache.strides[2]] = ((const _Float16*)new_v.ptr)[src_v + (int64_t)c * new_v.strides[2]];
    }
  }
}

// ---- rotary position embedding -------------------------------------------------------------
// rope_seq_f16 / rope_seq_dynpos_f16 / qk_rope_dynpos_f16 (cutile-kernels/src/positional.rs:13-64,
// 70-130, 136-230): x [seq, heads, D] split in halves lo = [.., :D/2], hi = [.., D/2:];
// theta = f32(position_start + s) * inv_freq[i]; y_lo = x_lo cos - x_hi sin; y_hi = x_hi cos + x_lo sin.
// The reference launches one tile block per (s, head, half) and computes both halves
// in each; here a workgroup takes one position s: cos/sin of its D/2 angles are
// computed once into LDS (they do not depend on the head), then every lane
// rotates 8 pairs of one head (16-byte accesses).  In the q/k form heads >=
// num_q_heads of `out` come from `k`.  `pos_dev` (if not null) holds the start position.
extern "C" __global__ void __launch_bounds__(kThreads)
    rope_entry__f16(TensorArg<3> q, TensorArg<3> k, TensorArg<1> inv_freq, const uint32_t* pos_dev,
                    PartitionArg<3> out, int32_t position_start, int32_t num_q_heads, TileGrid g) {
  constexpr int kMaxHalf = 1024;                      // angles kept in LDS; longer heads recompute per lane
  __shared__ float cs_tab[kMaxHalf], sn_tab[kMaxHalf];
  const int32_t d = q.shape[2], half = d >> 1;
  const int64_t seq = min((int64_t)g.x, (int64_t)out.shape[0]);
  const int32_t heads = (int32_t)min((int64_t)g.y, (int64_t)out.shape[1]);
  const int32_t base = pos_dev ? (int32_t)pos_dev[0] : position_start;
  const float* freq = (const float*)inv_freq.ptr;
  const int32_t chunks = (half + 7) / 8;               // 8 rotation pairs per lane
  const bool tab = half <= kMaxHalf;
  const bool vec_out = (half % 8 == 0) && out.strides[2] == 1 && (out.strides[1] % 8 == 0) && (out.strides[0] % 8 == 0) &&
                       ((uintptr_t)out.ptr & 15) == 0;
  auto vec_in = [&](const TensorArg<3>& t) {
    return t.strides[2] == 1 && (t.strides[1] % 8 == 0) && (t.strides[0] % 8 == 0) && ((uintptr_t)t.ptr & 15) == 0;
  };
  const bool vec = vec_out && vec_in(q) && vec_in(k);
  for (int64_t s_idx = blockIdx.x; s_idx < seq; s_idx += gridDim.x) {
    const float pos = (float)(base + (int32_t)s_idx);
    if (tab) {
      __syncthreads();                                 // the previous position's table is no longer read
      for (int32_t i = threadIdx.x; i < half; i += kThreads)
        sincosf(pos * freq[(int64_t)i * inv_freq.strides[0]], &sn_tab[i], &cs_tab[i]);
      __syncthreads();
    }
    for (int32_t t = threadIdx.x; t < heads * chunks; t += kThreads) {
      const int32_t h = t / chunks, i0 = (t % chunks) * 8;
      const bool from_k = h >= num_q_heads;
      const TensorArg<3>& src = from_k ? k : q;
      const _Float16* xr = (const _Float16*)src.ptr + s_idx * src.strides[0] + (int64_t)(from_k ? h - num_q_heads : h) * src.strides[1];
      _Float16* orow = (_Float16*)out.ptr + s_idx * out.strides[0] + (int64_t)h * out.strides[1];
      auto angle = [&](int32_t i, float* sn, float* cs) {
        if (tab) {
          *sn = sn_tab[i];
          *cs = cs_tab[i];
        } else {
          sincosf(pos * freq[(int64_t)i * inv_freq.strides[0]], sn, cs);
        }
      };
      if (vec) {
        Vec16<_Float16> lo, hi, ylo, yhi;
        lo.raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xr + i0));
        hi.raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xr + half + i0));
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float sn, cs;
          angle(i0 + e, &sn, &cs);
          const float l = (float)lo.v[e], hv = (float)hi.v[e];
          ylo.v[e] = (_Float16)(l * cs - hv * sn);
          yhi.v[e] = (_Float16)(hv * cs + l * sn);
        }
        __builtin_nontemporal_store(ylo.raw, reinterpret_cast<u32x4*>(orow + i0));
        __builtin_nontemporal_store(yhi.raw, reinterpret_cast<u32x4*>(orow + half + i0));
      } else {
        for (int32_t i = i0; i < min(i0 + 8, half); ++i) {
          float sn, cs;
          angle(i, &sn, &cs);
          const float l = (float)xr[(int64_t)i * src.strides[2]], hv = (float)xr[(int64_t)(half + i) * src.strides[2]];
          orow[(int64_t)i * out.strides[2]] = (_Float16)(l * cs - hv * sn);
          orow[(int64_t)(half + i) * out.strides[2]] = (_Float16)(hv * cs + l * sn);
        }
      }
    }
  }
}

// ---- creation ------------------------------------------------------------------------------
#define CREATION_KERNELS(T, NAME)                                                                   \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      full_entry__##NAME(T value, PartitionArg<1> t, TileGrid g) {                                  \
    flat_generate<T>((T*)t.ptr, t.strides[0], covered_1d(t.shape[0], t.pshape[0], g),             \
                     [&](size_t) { return value; });                                               \
  }                                                                                                 \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      arange_entry__##NAME(PartitionArg<1> t, TileGrid g) {                                         \
    flat_generate<T>((T*)t.ptr, t.strides[0], covered_1d(t.shape[0], t.pshape[0], g),             \
                     [&](size_t i) { return (T)(int32_t)i; });                                     \
  }

CREATION_KERNELS(float, f32)
CREATION_KERNELS(double, f64)
CREATION_KERNELS(_Float16, f16)
CREATION_KERNELS(__bf16, bf16)
CREATION_KERNELS(int32_t, i32)
CREATION_KERNELS(int64_t, i64)
CREATION_KERNELS(uint8_t, u8)
CREATION_KERNELS(uint16_t, u16)
CREATION_KERNELS(uint32_t, u32)

extern "C" __global__ void __launch_bounds__(kThreads)
    linspace_entry__f32(PartitionArg<1> t, float start, float step, TileGrid g) {
  flat_generate<float>((float*)t.ptr, t.strides[0], covered_1d(t.shape[0], t.pshape[0], g),
                       [&](size_t i) { return start + (float)(int32_t)i * step; });
}

// eye<BR, BC>(tensor: [BR, BC] tiles of an f32 matrix): 1 where row == column, 0 elsewhere, over the
// region the tile grid covers (cutile/src/kernels/_creation.rs:110-138).  Flat over that region: the
// tile shape only decides how far the grid reaches, every element is written exactly once.
extern "C" __global__ void __launch_bounds__(kThreads) eye_entry__f32(PartitionArg<2> t, TileGrid g) {
  const int64_t rows = min((int64_t)t.shape[0], (int64_t)g.x * t.pshape[0]);
  const int64_t cols = min((int64_t)t.shape[1], (int64_t)g.y * t.pshape[1]);
  float* p = (float*)t.ptr;
  const int64_t total = rows * cols;
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < total; i += (int64_t)gridDim.x * kThreads) {
    const int64_t r = i / cols, c = i - r * cols;
    p[r * t.strides[0] + c * t.strides[1]] = r == c ? 1.0f : 0.0f;
  }
}

// ---- the example programs' small kernels --------------------------------------------------------
// relu<D>(input_output: [D] tiles of an f32 vector, updated in place): max(0, x) —
// cutile-examples/examples/async_mlp.rs:56-61.  A NaN becomes 0 (the maximum returns its other operand).
extern "C" __global__ void __launch_bounds__(kThreads) relu_entry__f32(PartitionArg<1> io, TileGrid g) {
  const size_t count = covered_1d(io.shape[0], io.pshape[0], g);
  flat_map1<float>((const float*)io.ptr, io.strides[0], count, (float*)io.ptr, io.strides[0], count,
                   [](float v) { return __builtin_fmaxf(0.0f, v); });
}

// dropout<S>(p, _x, x_keep, out: [S] tiles): out = select(x_keep > p, x_keep, 0) / (1 - p), x_keep loaded like the
// output tile (0 beyond its extent) — cutile-examples/examples/dropout.rs:17-32.  The first tensor is an argument the
// tile program never reads; it is marshalled and ignored here too.
extern "C" __global__ void __launch_bounds__(kThreads)
    dropout_entry__f32(float p, TensorArg<1> x, TensorArg<1> x_keep, PartitionArg<1> out, TileGrid g) {
  (void)x;
  const float keep_scale = 1.0f - p;
  flat_map1<float>((const float*)x_keep.ptr, x_keep.strides[0], (size_t)x_keep.shape[0], (float*)out.ptr, out.strides[0],
                   covered_1d(out.shape[0], out.pshape[0], g), [=](float v) { return (v > p ? v : 0.0f) / keep_scale; });
}

// scale_ptr(out_ptr, in_ptr, scale, len): out[i] = in[i] * scale for i < len, on raw pointers —
// cutile-examples/examples/scale_ptr.rs:26-80.  The tile program strides its 128-element blocks over the launch
// grid until len is covered, so every launch grid gives the same result; the walk here is over 16-byte vectors.
extern "C" __global__ void __launch_bounds__(kThreads)
    scale_ptr_entry__f32(float* out, const float* in, float scale, int32_t len) {
  const size_t count = len > 0 ? (size_t)len : 0;
  flat_map1<float>(in, 1, count, out, 1, count, [=](float v) { return v * scale; });
}

// matvec<BM, BK, K>(z: [BM] tiles, x: [M, K], y: [K]), all f32: z[r] <- z[r] + sum_k x[r, k] * y[k] over the
// K / BK whole K tiles (k_total) — cutile-examples/examples/async_mlp.rs:38-54.  Rows and K positions that x or y do
// not have read 0.  One wavefront per row: the row is the stream (x is read once, y stays in cache), lanes take
// 16-byte pieces 1 KiB apart, four accumulators per lane, then the wavefront's sum.
extern "C" __global__ void __launch_bounds__(kThreads)
    matvec_entry__f32(PartitionArg<1> z, TensorArg<2> x, TensorArg<1> y, int32_t k_total, TileGrid g) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  constexpr int kWaves = kThreads / 64;
  const int64_t rows = (int64_t)covered_1d(z.shape[0], z.pshape[0], g);
  const int32_t k_valid = min(min(x.shape[1], y.shape[0]), k_total);
  const float* yp = (const float*)y.ptr;
  const bool vectors = x.strides[1] == 1 && y.strides[0] == 1 && (x.strides[0] & 3) == 0 &&
                       (((uintptr_t)x.ptr | (uintptr_t)y.ptr) & 15) == 0;
  for (int64_t r = (int64_t)blockIdx.x * kWaves + wave; r < rows; r += (int64_t)gridDim.x * kWaves) {
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (r < x.shape[0]) {
      const float* xr = (const float*)x.ptr + r * x.strides[0];
      int32_t done = 0;
      if (vectors) {
        const int32_t nvec = k_valid / 4;
        for (int32_t j = lane; j < nvec; j += 64) {
          Vec16<float> a, b;
          a.raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xr) + j);
          b.raw = reinterpret_cast<const u32x4*>(yp)[j];
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[e] = __builtin_fmaf(a.v[e], b.v[e], acc[e]);
        }
        done = nvec * 4;
      }
      for (int32_t k = done + lane; k < k_valid; k += 64)
        acc[0] = __builtin_fmaf(xr[(int64_t)k * x.strides[1]], yp[(int64_t)k * y.strides[0]], acc[0]);
    }
    const float sum = lanes::across_wave<lanes::Sum>((acc[0] + acc[1]) + (acc[2] + acc[3]));
    if (lane == 0) {
      float* dst = (float*)z.ptr + r * z.strides[0];
      *dst = *dst + sum;
    }
  }
}

// ---- convert -------------------------------------------------------------------------------
#define CONVERT_KERNEL(S, SN, D, DN)                                                                \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      convert_entry__##SN##_##DN(TensorArg<1> src, PartitionArg<1> dst, TileGrid g) {               \
    flat_convert<D, S>((const S*)src.ptr, src.strides[0], (size_t)src.shape[0], (D*)dst.ptr,       \
                       dst.strides[0], covered_1d(dst.shape[0], dst.pshape[0], g));                \
  }

#define CONVERT_FROM(S, SN)            \
  CONVERT_KERNEL(S, SN, float, f32)    \
  CONVERT_KERNEL(S, SN, double, f64)   \
  CONVERT_KERNEL(S, SN, _Float16, f16) \
  CONVERT_KERNEL(S, SN, __bf16, bf16)  \
  CONVERT_KERNEL(S, SN, int32_t, i32)  \
  CONVERT_KERNEL(S, SN, int64_t, i64)

CONVERT_FROM(float, f32)
CONVERT_FROM(double, f64)
CONVERT_FROM(_Float16, f16)
CONVERT_FROM(__bf16, bf16)
CONVERT_FROM(int32_t, i32)
CONVERT_FROM(int64_t, i64)

// ---- mapped partitions: every tile receives its own logical index ----------------------------
// The reference checks its mapped schedules with kernels that store, into every tile a tile
// block visits, that tile's row-major index in the logical grid
// (cutile/tests/gpu/mapped_partition_schedule_matrix.rs:30-76): a dropped tile keeps
// the caller's fill, a duplicated one overwrites a neighbour.  Same kernel here, for
// i32 tensors of rank 1 to 3: workgroup b takes stream items b, b + gridDim.x, ...;
// an OWNED axis is walked in full by the workgroup that owns the item.
// With a sub-range (write_flat_index_subrange, the same file :75-106) the schedule runs over the range's lengths,
// the starts are added, and the index stored is the one in the whole grid.
template <int R>
__device__ __forceinline__ void mapped_tile_index(const PartitionArg<R>& z, const MappedArg& m, const MappedRangeArg& range) {
  int32_t* zp = (int32_t*)z.ptr;
  for (uint32_t item = blockIdx.x; item < m.total; item += gridDim.x) {
    uint32_t bid[3];
    mapped_index(m, item, bid);
    uint32_t lo[3] = {0, 0, 0}, hi[3] = {1, 1, 1};
    for (int a = 0; a < R; ++a) {
      lo[a] = m.map[a] == kOwnedAxis ? 0 : bid[a] + (uint32_t)range.start[a];
      hi[a] = m.map[a] == kOwnedAxis ? m.grid[a] : lo[a] + 1;
    }
    for (uint32_t c0 = lo[0]; c0 < hi[0]; ++c0)
      for (uint32_t c1 = lo[1]; c1 < hi[1]; ++c1)
        for (uint32_t c2 = lo[2]; c2 < hi[2]; ++c2) {
          const uint32_t c[3] = {c0, c1, c2};
          int32_t flat = 0;
          int64_t count = 1;
          for (int a = 0; a < R; ++a) {
            flat = flat * (int32_t)range.full_grid[a] + (int32_t)c[a];
            count *= z.pshape[a];
          }
          for (int64_t e = threadIdx.x; e < count; e += kThreads) {
            int64_t rest = e, off = 0;
            bool inside = true;
            for (int a = R - 1; a >= 0; --a) {
              const int64_t idx = (int64_t)c[a] * z.pshape[a] + rest % z.pshape[a];
              rest /= z.pshape[a];
              inside &= idx < z.shape[a];
              off += idx * z.strides[a];
            }
            if (inside) zp[off] = flat;
          }
        }
  }
}

#define MAPPED_TILE_INDEX_KERNEL(R)                                                                \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      mapped_tile_index_entry__i32_r##R(PartitionArg<R> z, MappedArg m) {                          \
    const MappedRangeArg whole = {{0, 0, 0}, {m.grid[0], m.grid[1], m.grid[2]}};                   \
    mapped_tile_index<R>(z, m, whole);                                                             \
  }                                                                                                \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      mapped_tile_index_within_entry__i32_r##R(PartitionArg<R> z, MappedArg m, MappedRangeArg range) { \
    mapped_tile_index<R>(z, m, range);                                                             \
  }
MAPPED_TILE_INDEX_KERNEL(1)
MAPPED_TILE_INDEX_KERNEL(2)
MAPPED_TILE_INDEX_KERNEL(3)

// Two mapped outputs sharing one index stream (`iter_indices_within_with`, cutile/src/_core.rs:932-941): the
// reference's dynpos_shared_rank3 / prefill_shared_rank3 kernels
// (cutile/tests/gpu/mapped_partition_schedule_matrix.rs:107-153).  k_cache and v_cache are [heads, max_seq, d] in
// tiles [B0, B1, B2]; the stream covers ranges [(0, -1), (start, n_tiles), (0, -1)], start by value or read from
// device memory; tile (h, s, c) of the source is taken at (h, s - start, c) for a [heads, seq, d] source and at
// (s - start, h, c) for a [seq, heads, d] one (out of range reads as zero), stored to k_cache and doubled to v_cache.
// A start that does not fit the grid writes nothing (the reference's range assert stops its kernel).
extern "C" __global__ void __launch_bounds__(kThreads)
    mapped_shared_cache_update_entry__f32(PartitionArg<3> k_cache, PartitionArg<3> v_cache, TensorArg<3> new_k, MappedArg m,
                                          MappedRangeArg range, const int32_t* pos_dev, int32_t seq_major) {
  const int32_t start = pos_dev ? pos_dev[0] : range.start[1];
  if (start < 0 || (uint32_t)start + m.grid[1] > range.full_grid[1]) return;
  float* kp = (float*)k_cache.ptr;
  float* vp = (float*)v_cache.ptr;
  const float* sp = (const float*)new_k.ptr;
  const int64_t count = (int64_t)k_cache.pshape[0] * k_cache.pshape[1] * k_cache.pshape[2];
  for (uint32_t item = blockIdx.x; item < m.total; item += gridDim.x) {
    uint32_t bid[3];
    mapped_index(m, item, bid);
    const int64_t dst_tile[3] = {(int64_t)bid[0] + range.start[0], (int64_t)bid[1] + start, (int64_t)bid[2] + range.start[2]};
    const int64_t src_tile[3] = {seq_major ? (int64_t)bid[1] : dst_tile[0], seq_major ? dst_tile[0] : (int64_t)bid[1], dst_tile[2]};
    for (int64_t e = threadIdx.x; e < count; e += kThreads) {
      int64_t rest = e, k_off = 0, v_off = 0, s_off = 0;
      bool dst_inside = true, src_inside = true;
      for (int a = 2; a >= 0; --a) {
        const int64_t in_tile = rest % k_cache.pshape[a];
        rest /= k_cache.pshape[a];
        const int64_t di = dst_tile[a] * k_cache.pshape[a] + in_tile, si = src_tile[a] * k_cache.pshape[a] + in_tile;
        dst_inside &= di < k_cache.shape[a] && di < v_cache.shape[a];
        src_inside &= si < new_k.shape[a];
        k_off += di * k_cache.strides[a];
        v_off += di * v_cache.strides[a];
        s_off += si * new_k.strides[a];
      }
      if (dst_inside) {
        const float x = src_inside ? sp[s_off] : 0.0f;
        kp[k_off] = x;
        vp[v_off] = x + x;
      }
    }
  }
}

// ---- greedy sampling and row gathers ---------------------------------------------------------
// argmax_blocks_f16 / lm_head_argmax_blocks_f16 / argmax_reduce_blocks_to_u32
// (cutile-kernels/src/argmax.rs:21-71, 88-158, 173-213), embedding_batch_f16
// (embeddings.rs:21-41), gather_row_f16 (pointwise.rs:86-99).
// A block's winner is its largest value and, among equal values, the smallest index; positions at or
// beyond `len` count as -1e30 at their own index, exactly as the tile programs mask them (argmax.rs:42-55).
namespace {

struct Best {
  float v;
  int32_t i;
};
__device__ __forceinline__ Best better(Best a, Best b) {
  return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a;
}
// Winner of the workgroup, valid in every lane.  `scratch`: kThreads / 64 entries of LDS.
__device__ __forceinline__ Best block_best(Best mine, Best* scratch) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    Best other = {__shfl_xor(mine.v, o, 64), __shfl_xor(mine.i, o, 64)};
    mine = better(mine, other);
  }
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) scratch[wave] = mine;
  __syncthreads();
  Best r = scratch[0];
#pragma unroll
  for (int w = 1; w < kThreads / 64; ++w) r = better(r, scratch[w]);
  return r;
}
constexpr float kMaskedLogit = -1.0e30f;

}  // namespace

// One workgroup per block of BLOCK_SIZE logits: block_max[b], block_idx[b].
extern "C" __global__ void __launch_bounds__(kThreads)
    argmax_blocks_entry__f16(TensorArg<1> logits, PartitionArg<1> block_max, PartitionArg<1> block_idx, int32_t len,
                             int32_t block_size, TileGrid g) {
  __shared__ Best scratch[kThreads / 64];
  const int32_t b = blockIdx.x;
  if (b >= (int32_t)g.x || b >= block_max.shape[0] || b >= block_idx.shape[0]) return;
  const int64_t base = (int64_t)b * block_size;
  const _Float16* lp = (const _Float16*)logits.ptr;
  Best mine = {-INFINITY, INT32_MAX};
  for (int32_t o = threadIdx.x; o < block_size; o += kThreads) {
    const int64_t idx = base + o;
    // beyond the tensor a tile load reads zero (cutile/src/_core.rs:651-657); beyond len the value is masked
    float v = idx < logits.shape[0] ? (float)lp[idx * logits.strides[0]] : 0.0f;
    if (idx >= len) v = kMaskedLogit;
    mine = better(mine, Best{v, (int32_t)idx});
  }
  const Best r = block_best(mine, scratch);
  if (threadIdx.x == 0) {
    ((float*)block_max.ptr)[(int64_t)b * block_max.strides[0]] = r.v;
    ((uint32_t*)block_idx.ptr)[(int64_t)b * block_idx.strides[0]] = (uint32_t)r.i;
  }
}

// logits[r] = sum_k f32(weights[r, k]) * f32(hidden[0, k]) for the 64 rows of block b, then the block's winner.
// The weights are read once, 16 bytes per lane and nontemporally (a [vocab, K] matrix streams through once per
// token); the hidden vector sits in LDS.  The launch holds two workgroups per compute unit, each taking a
// contiguous run of blocks (a stream of this kind reads fastest from few resident wavefronts); a wavefront takes
// 16 of a block's 64 rows, two at a time, 1024 columns per step, and requests the next step's weights before it
// multiplies the current ones.
namespace {

constexpr int kLmRows = 64, kLmRowsPerWave = kLmRows / (kThreads / 64), kLmChunksPerStep = 64 * 4;

struct LmHeadArgs {
  const _Float16* wp;
  const _Float16* hs;      // hidden in LDS
  float* row_logit;        // kLmRows entries of LDS
  Best* scratch;
  float* block_max;
  uint32_t* block_idx;
  int64_t w_stride0, max_stride, idx_stride;
  int32_t w_rows, chunks, steps_per_pair, steps_per_block, b_begin, vocab_size;
  int lane, wave;
};

typedef Vec16<_Float16> LmTile[2][4];

__device__ __forceinline__ void lm_head_issue(LmTile& w, const LmHeadArgs& a, int32_t step) {
  const int32_t b = a.b_begin + step / a.steps_per_block, in_block = step % a.steps_per_block;
  const int64_t r0 = (int64_t)b * kLmRows + (in_block / a.steps_per_pair * (kThreads / 64) + a.wave) * 2;
  const int32_t c0 = in_block % a.steps_per_pair * kLmChunksPerStep;
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int32_t c = c0 + u * 64 + a.lane;
      w[t][u].raw = u32x4{0, 0, 0, 0};   // a row beyond the matrix reads as zeros, like a padded tile load
      if (r0 + t < a.w_rows && c < a.chunks)
        w[t][u].raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(a.wp + (r0 + t) * a.w_stride0) + c);
    }
}

__device__ __forceinline__ void lm_head_consume(const LmTile& w, float (&acc)[2], const LmHeadArgs& a, int32_t step) {
  const int32_t b = a.b_begin + step / a.steps_per_block, in_block = step % a.steps_per_block;
  const int32_t pair = in_block / a.steps_per_pair, part = in_block % a.steps_per_pair;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int32_t c = part * kLmChunksPerStep + u * 64 + a.lane;
    if (c < a.chunks) {
      Vec16<_Float16> h;
      h.raw = *reinterpret_cast<const u32x4*>(a.hs + (int64_t)c * 8);
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[t] = __builtin_fmaf((float)w[t][u].v[e], (float)h.v[e], acc[t]);
    }
  }
  if (part + 1 < a.steps_per_pair) return;
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    acc[t] = lanes::across_wave<lanes::Sum>(acc[t]);
    if (a.lane == 0) a.row_logit[(pair * (kThreads / 64) + a.wave) * 2 + t] = acc[t];
    acc[t] = 0.0f;
  }
  if (in_block + 1 < a.steps_per_block) return;
  __syncthreads();
  Best mine = {-INFINITY, INT32_MAX};
  if (threadIdx.x < kLmRows) {
    const int64_t idx = (int64_t)b * kLmRows + threadIdx.x;
    mine = Best{idx < a.vocab_size ? a.row_logit[threadIdx.x] : kMaskedLogit, (int32_t)idx};
  }
  const Best r = block_best(mine, a.scratch);   // its barrier also orders these reads before the next block's writes
  if (threadIdx.x == 0) {
    a.block_max[(int64_t)b * a.max_stride] = r.v;
    a.block_idx[(int64_t)b * a.idx_stride] = (uint32_t)r.i;
  }
}

}  // namespace

extern "C" __global__ void __launch_bounds__(kThreads)
    lm_head_argmax_blocks_entry__f16(TensorArg<2> weights, TensorArg<2> hidden, PartitionArg<1> block_max,
                                     PartitionArg<1> block_idx, int32_t vocab_size, TileGrid g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  __shared__ float row_logit[kLmRows];
  __shared__ Best scratch[kThreads / 64];
  const int32_t n_blocks = min((int32_t)g.x, min(block_max.shape[0], block_idx.shape[0]));
  const int32_t b_begin = (int32_t)((int64_t)blockIdx.x * n_blocks / gridDim.x);
  const int32_t b_end = (int32_t)((int64_t)(blockIdx.x + 1) * n_blocks / gridDim.x);
  if (b_begin >= b_end) return;
  const int32_t k_len = min(weights.shape[1], hidden.shape[1]);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const _Float16* wp = (const _Float16*)weights.ptr;
  const _Float16* hp = (const _Float16*)hidden.ptr;
  _Float16* hs = (_Float16*)lds_raw;
  const bool vec = k_len % 8 == 0 && weights.strides[1] == 1 && weights.strides[0] % 8 == 0 && hidden.strides[1] == 1 &&
                   (((uintptr_t)wp | (uintptr_t)hp) & 15) == 0;
  for (int32_t k = threadIdx.x; k < k_len; k += kThreads) hs[k] = hp[(int64_t)k * hidden.strides[1]];
  __syncthreads();
  if (vec) {
    LmHeadArgs a;
    a.wp = wp, a.hs = hs, a.row_logit = row_logit, a.scratch = scratch;
    a.block_max = (float*)block_max.ptr, a.block_idx = (uint32_t*)block_idx.ptr;
    a.w_stride0 = weights.strides[0], a.max_stride = block_max.strides[0], a.idx_stride = block_idx.strides[0];
    a.w_rows = weights.shape[0], a.chunks = k_len / 8;
    a.steps_per_pair = max((a.chunks + kLmChunksPerStep - 1) / kLmChunksPerStep, 1);
    a.steps_per_block = a.steps_per_pair * (kLmRowsPerWave / 2);
    a.b_begin = b_begin, a.vocab_size = vocab_size, a.lane = lane, a.wave = wave;
    const int32_t steps = (b_end - b_begin) * a.steps_per_block;
    float acc[2] = {0.0f, 0.0f};
    LmTile even, odd;
    lm_head_issue(even, a, 0);
    for (int32_t s = 0; s < steps; s += 2) {
      if (s + 1 < steps) lm_head_issue(odd, a, s + 1);
      lm_head_consume(even, acc, a, s);
      if (s + 2 < steps) lm_head_issue(even, a, s + 2);
      if (s + 1 < steps) lm_head_consume(odd, acc, a, s + 1);
    }
    return;
  }
  for (int32_t b = b_begin; b < b_end; ++b) {
    const int64_t row0 = (int64_t)b * kLmRows + wave * kLmRowsPerWave;
    for (int rr = 0; rr < kLmRowsPerWave; ++rr) {
      const int64_t r = row0 + rr;
      float acc = 0.0f;
      if (r < weights.shape[0])
        for (int32_t k = lane; k < k_len; k += 64)
          acc = __builtin_fmaf((float)wp[r * weights.strides[0] + (int64_t)k * weights.strides[1]], (float)hs[k], acc);
      acc = lanes::across_wave<lanes::Sum>(acc);
      if (lane == 0) row_logit[wave * kLmRowsPerWave + rr] = acc;
    }
    __syncthreads();
    Best mine = {-INFINITY, INT32_MAX};
    if (threadIdx.x < kLmRows) {
      const int64_t idx = (int64_t)b * kLmRows + threadIdx.x;
      mine = Best{idx < vocab_size ? row_logit[threadIdx.x] : kMaskedLogit, (int32_t)idx};
    }
    const Best r = block_best(mine, scratch);
    if (threadIdx.x == 0) {
      ((float*)block_max.ptr)[(int64_t)b * block_max.strides[0]] = r.v;
      ((uint32_t*)block_idx.ptr)[(int64_t)b * block_idx.strides[0]] = (uint32_t)r.i;
    }
  }
}

// One workgroup: the winner among the first `block_size` (value, index) pairs, of which `num_blocks` count.
extern "C" __global__ void __launch_bounds__(kThreads)
    argmax_reduce_blocks_entry__u32(TensorArg<1> block_max, TensorArg<1> block_idx, PartitionArg<1> out,
                                    int32_t num_blocks, int32_t block_size, TileGrid g) {
  __shared__ Best scratch[kThreads / 64];
  if (blockIdx.x != 0 || g.x == 0) return;
  Best mine = {-INFINITY, INT32_MAX};
  for (int32_t o = threadIdx.x; o < block_size; o += kThreads) {
    float v = o < block_max.shape[0] ? ((const float*)block_max.ptr)[(int64_t)o * block_max.strides[0]] : 0.0f;
    const int32_t i = o < block_idx.shape[0] ? (int32_t)((const uint32_t*)block_idx.ptr)[(int64_t)o * block_idx.strides[0]] : 0;
    if (o >= num_blocks) v = kMaskedLogit;
    mine = better(mine, Best{v, i});
  }
  const Best r = block_best(mine, scratch);
  if (threadIdx.x == 0) ((uint32_t*)out.ptr)[0] = (uint32_t)r.i;
}

// out[row, :] = table[token_ids[row], :] (zeros for a token beyond the table, as a padded tile load gives);
// a workgroup copies whole rows, 16 bytes per lane when the layout allows it.
extern "C" __global__ void __launch_bounds__(kThreads)
    embedding_batch_entry__f16(TensorArg<1> token_ids, TensorArg<2> table, PartitionArg<2> out, TileGrid g) {
  const int32_t rows = min(min((int32_t)g.x, out.shape[0]), token_ids.shape[0]);
  const int64_t cover = (int64_t)g.y * out.pshape[1];
  const int32_t width = (int32_t)(cover < out.shape[1] ? cover : out.shape[1]);
  const _Float16* tp = (const _Float16*)table.ptr;
  _Float16* op = (_Float16*)out.ptr;
  const bool vec = width % 8 == 0 && table.strides[1] == 1 && out.strides[1] == 1 && table.strides[0] % 8 == 0 &&
                   out.strides[0] % 8 == 0 && (((uintptr_t)tp | (uintptr_t)op) & 15) == 0;
  for (int32_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const uint32_t token = ((const uint32_t*)token_ids.ptr)[(int64_t)row * token_ids.strides[0]];
    const bool known = token < (uint32_t)table.shape[0];
    const _Float16* src = tp + (int64_t)token * table.strides[0];
    _Float16* dst = op + (int64_t)row * out.strides[0];
    if (vec) {
      // up to four vectors per lane requested before the first is stored (a row of 4096 halves is two per lane)
      for (int32_t c0 = threadIdx.x; c0 < width / 8; c0 += kThreads * kUnroll) {
        u32x4 v[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          const int32_t c = c0 + u * kThreads;
          v[u] = u32x4{0, 0, 0, 0};
          if (known && c < width / 8 && c * 8 < table.shape[1]) v[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src) + c);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          const int32_t c = c0 + u * kThreads;
          if (c < width / 8) __builtin_nontemporal_store(v[u], reinterpret_cast<u32x4*>(dst) + c);
        }
      }
    } else {
      for (int32_t c = threadIdx.x; c < width; c += kThreads)
        dst[(int64_t)c * out.strides[1]] = known && c < table.shape[1] ? src[(int64_t)c * table.strides[1]] : (_Float16)0;
    }
  }
}

// out[c] = src[row_idx, c]; zeros where the source has no such element.
extern "C" __global__ void __launch_bounds__(kThreads)
    gather_row_entry__f16(TensorArg<2> src, PartitionArg<1> out, int32_t row_idx, TileGrid g) {
  const int64_t cover = (int64_t)g.x * out.pshape[0];
  const int32_t width = (int32_t)(cover < out.shape[0] ? cover : out.shape[0]);
  const bool known = row_idx >= 0 && row_idx < src.shape[0];
  const _Float16* sp = (const _Float16*)src.ptr + (int64_t)row_idx * src.strides[0];
  _Float16* op = (_Float16*)out.ptr;
  for (int64_t c = (int64_t)blockIdx.x * kThreads + threadIdx.x; c < width; c += (int64_t)gridDim.x * kThreads)
    op[c * out.strides[0]] = known && c < src.shape[1] ? sp[c * src.strides[1]] : (_Float16)0;
}

// ---- fused Q/K norm + rotary embedding + KV-cache update -------------------------------------
// qk_norm_rope_kv_prefill_raw_f16 / qk_norm_rope_kv_decode_raw_f16
// (cutile-kernels/src/experimental/fused_transformer.rs:22-345, 356-625), raw device pointers as there.
// For position s of the launch and head h: a q or k row [D] is RMS-normalised with its weight in f32
// (x * rsqrt(mean(x^2) + eps) * w, :182-240) and rotated, still in f32, by the angles
// (position_start + s) * inv_freq (:242-258); q rows go to q_out[s, h], k rows to
// k_cache[h, position_start + s], and the v row is copied to v_cache[h, position_start + s] (:263-341).
// q, q_out: rows of num_q_heads * D every q_row_stride elements; k, v: num_kv_heads * D every kv_row_stride;
// the caches are [num_kv_heads, max_seq, D].  The decode form is the same work for one position whose q, k
// and v rows sit back to back and whose position is read from device memory.
// One workgroup per position: the D/2 (cos, sin) pairs are computed once into LDS; a lane holds 8 rotation
// pairs of one row (two 16-byte accesses), D/16 neighbouring lanes hold a row and sum its squares.  The workgroup
// size (64 .. 256 lanes) is the launcher's: the one that leaves the fewest lanes idle in the last pass over the rows.
namespace {
struct FusedRowsArgs {
  const _Float16 *q, *k, *v, *q_weight, *k_weight;
  _Float16 *q_out, *k_cache, *v_cache;
  float eps;
  int32_t num_q_heads, num_kv_heads, d, half, chunks, chunk_shift, max_seq, rows;
  int64_t q_row_stride, kv_row_stride;
};
// where row r of position s_idx comes from
__device__ __forceinline__ const _Float16* fused_source(const FusedRowsArgs& a, int64_t s_idx, int32_t r) {
  if (r < a.num_q_heads) return a.q + s_idx * a.q_row_stride + (int64_t)r * a.d;
  if (r < a.num_q_heads + a.num_kv_heads) return a.k + s_idx * a.kv_row_stride + (int64_t)(r - a.num_q_heads) * a.d;
  return a.v + s_idx * a.kv_row_stride + (int64_t)(r - a.num_q_heads - a.num_kv_heads) * a.d;
}
// norm + rotation (q, k rows) or copy (v rows) of the 16 elements this lane holds of lane slot t
__device__ __forceinline__ void fused_finish(const FusedRowsArgs& a, int64_t s_idx, int32_t pos_i, int32_t t, u32x4 lo_raw,
                                             u32x4 hi_raw, const float* cs_tab, const float* sn_tab) {
  Vec16<_Float16> lo, hi;
  lo.raw = lo_raw;
  hi.raw = hi_raw;
  const int32_t r = t >> a.chunk_shift, c = t & (a.chunks - 1);
  const bool is_q = r < a.num_q_heads, is_k = !is_q && r < a.num_q_heads + a.num_kv_heads;
  float ss = 0.0f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float l = (float)lo.v[e], h = (float)hi.v[e];
    ss += l * l + h * h;
  }
  // the row's lanes are `chunks` neighbours (D / 16, a power of two; the same for every lane): quad steps, the mirrored
  // halves of a row of 16 lanes, then whole rows
  if (a.chunks >= 2) ss += lanes::dpp<lanes::kQuadXor1>(ss);
  if (a.chunks >= 4) ss += lanes::dpp<lanes::kQuadXor2>(ss);
  if (a.chunks >= 8) ss += lanes::dpp<lanes::kHalfMirror>(ss);
  if (a.chunks >= 16) ss += lanes::dpp<lanes::kRowMirror>(ss);
  if (a.chunks >= 32) {
    float e, o;
    lanes::split_row_pairs(ss, &e, &o);
    ss = e + o;
  }
  if (a.chunks >= 64) ss = lanes::across_halves<lanes::Sum>(ss);
  if (r >= a.rows || (!is_q && (pos_i < 0 || pos_i >= a.max_seq))) return;
  _Float16* dst;
  if (is_q) {
    dst = a.q_out + s_idx * a.q_row_stride + (int64_t)r * a.d;
  } else {
    const int32_t kv_head = is_k ? r - a.num_q_heads : r - a.num_q_heads - a.num_kv_heads;
    dst = (is_k ? a.k_cache : a.v_cache) + ((int64_t)kv_head * a.max_seq + pos_i) * a.d;
  }
  if (is_q || is_k) {
    const float inv = __builtin_amdgcn_rsqf(ss / (float)a.d + a.eps);
    const _Float16* w = is_q ? a.q_weight : a.k_weight;
    Vec16<_Float16> wlo, whi, ylo, yhi;
    wlo.raw = reinterpret_cast<const u32x4*>(w)[c];
    whi.raw = reinterpret_cast<const u32x4*>(w + a.half)[c];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float nl = ((float)lo.v[e] * inv) * (float)wlo.v[e], nh = ((float)hi.v[e] * inv) * (float)whi.v[e];
      const float cs = cs_tab[c * 8 + e], sn = sn_tab[c * 8 + e];
      ylo.v[e] = (_Float16)(nl * cs - nh * sn);
      yhi.v[e] = (_Float16)(nh * cs + nl * sn);
    }
    lo.raw = ylo.raw;
    hi.raw = yhi.raw;
  }
  if (is_q) {   // the rotated queries go to the attention kernel of a later launch: past the caches
    asm volatile("");
    __builtin_nontemporal_store(lo.raw, reinterpret_cast<u32x4*>(dst) + c);
    __builtin_nontemporal_store(hi.raw, reinterpret_cast<u32x4*>(dst + a.half) + c);
    asm volatile("");
  } else {
    reinterpret_cast<u32x4*>(dst)[c] = lo.raw;
    reinterpret_cast<u32x4*>(dst + a.half)[c] = hi.raw;
  }
}
}  // namespace

extern "C" __global__ void __launch_bounds__(kThreads)
    qk_norm_rope_kv_entry__f16(const _Float16* q, const _Float16* k, const _Float16* v, const _Float16* q_weight,
                               const _Float16* k_weight, const float* inv_freq, _Float16* q_out, _Float16* k_cache,
                               _Float16* v_cache, const uint32_t* pos_dev, float eps, int32_t position_start,
                               int32_t seq_len, int32_t num_q_heads, int32_t num_kv_heads, int32_t d, int32_t max_seq,
                               int64_t q_row_stride, int64_t kv_row_stride) {
  constexpr int kTable = 1024;                           // (cos, sin) pairs kept in LDS
  __shared__ float cs_tab[kTable], sn_tab[kTable];
  FusedRowsArgs a;
  a.q = q, a.k = k, a.v = v, a.q_weight = q_weight, a.k_weight = k_weight;
  a.q_out = q_out, a.k_cache = k_cache, a.v_cache = v_cache;
  a.eps = eps, a.num_q_heads = num_q_heads, a.num_kv_heads = num_kv_heads, a.d = d, a.max_seq = max_seq;
  a.half = d >> 1, a.chunks = d >> 4;                    // a lane: elements [8c, 8c+8) of both halves
  a.chunk_shift = 31 - __builtin_clz((uint32_t)a.chunks);   // D/16 is a power of two
  a.rows = num_q_heads + 2 * num_kv_heads;
  a.q_row_stride = q_row_stride, a.kv_row_stride = kv_row_stride;
  const int32_t base = pos_dev ? (int32_t)pos_dev[0] : position_start;
  const int32_t threads = (int32_t)blockDim.x;          // chosen by the launcher so that the lane slots fill whole passes
  const int32_t slots = (a.rows * a.chunks + threads - 1) / threads * threads;   // whole lane groups stay together
  for (int64_t s_idx = blockIdx.x; s_idx < seq_len; s_idx += gridDim.x) {
    const int32_t pos_i = base + (int32_t)s_idx;
    __syncthreads();                                   // the previous position's table is no longer read
    for (int32_t i = threadIdx.x; i < a.half; i += threads) sincosf((float)pos_i * inv_freq[i], &sn_tab[i], &cs_tab[i]);
    __syncthreads();
    // (requesting rows before the table is computed costs registers, hence residency: measured 4.9 - 5.3 against 5.4 TB/s)
    for (int32_t t = (int32_t)threadIdx.x; t < slots; t += threads) {
      const int32_t r = t >> a.chunk_shift, c = t & (a.chunks - 1);
      u32x4 lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
      if (r < a.rows) {
        const _Float16* src = fused_source(a, s_idx, r);
        lo = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src) + c);
        hi = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src + a.half) + c);
      }
      fused_finish(a, s_idx, pos_i, t, lo, hi, cs_tab, sn_tab);
    }
  }
}

// ---- KV block layout conversion ---------------------------------------------------------------
// copy_stacked_to_contiguous_f16 / copy_contiguous_to_stacked_f16
// (cutile-kernels/src/experimental/kvbm.rs:112-187, 283-352; layouts :358-400).  A cache block is nh heads x nl
// layers x no offsets (K, V) x nt tokens x hd values.  Stacked form: one tensor per (block, layer, offset) — table
// entry (block * nl + layer) * no + offset — laid out [nt, nh, hd] (NHD) or [nh, nt, hd] (HND).  Contiguous form: one
// tensor per block, [nl, no, nt, nh, hd] (operational NHD), [nl, no, nh, nt, hd] (operational HND) or
// [nh, nl, no, nt, hd] (universal).  Every element is copied once; a lane moves 16 bytes along hd.
namespace {

struct KvbmArgs {
  const int64_t* stacked_tensors;
  const int64_t* contiguous_tensors;
  int32_t to_stacked, stacked_hnd, contiguous_layout, nh, nl, no, nt, hd, per_row;
};

// Source and destination of 16-byte vector (or element) i.  The copy is walked chunk by chunk — a chunk is one
// (block, layer, offset) tensor of the stacked side, nh * nt rows, contiguous there — and inside a chunk in the order
// of the contiguous side, where the chunk is one run (operational layouts) or nh runs of nt rows (universal):
// neighbouring workgroups stay inside one 64 KiB-class region on both sides (walking whole blocks in contiguous
// order instead left 256-byte pieces 2 KiB apart on the stacked side and measured 5.4 TB/s).
// I is the integer type of the index arithmetic: 32 bits whenever the whole copy has fewer than 2^31 vectors.
template <typename I>
__device__ __forceinline__ void kvbm_locate(const KvbmArgs& a, I i, I rows_per_chunk, const _Float16** src, _Float16** dst) {
  const I c = i % (I)a.per_row, row = i / (I)a.per_row;
  const I chunk = row / rows_per_chunk, in_chunk = row % rows_per_chunk;
  const I o = chunk % (I)a.no, bl = chunk / (I)a.no;
  const I l = bl % (I)a.nl, b = bl / (I)a.nl;
  I h, t;
  if (a.contiguous_layout == 0) {            // operational NHD [nl, no, nt, nh]: tokens outside heads
    h = in_chunk % (I)a.nh, t = in_chunk / (I)a.nh;
  } else {                                   // operational HND [nl, no, nh, nt], universal [nh, nl, no, nt]
    t = in_chunk % (I)a.nt, h = in_chunk / (I)a.nt;
  }
  int64_t cont_row;
  if (a.contiguous_layout == 2) cont_row = (((int64_t)h * a.nl + (int64_t)l) * a.no + (int64_t)o) * a.nt + (int64_t)t;
  else cont_row = (int64_t)(l * (I)a.no + o) * rows_per_chunk + (int64_t)in_chunk;
  const int64_t stacked_row = a.stacked_hnd ? (int64_t)h * a.nt + (int64_t)t : (int64_t)t * a.nh + (int64_t)h;
  const int64_t step = a.per_row == a.hd ? 1 : 8;      // elements per index unit
  _Float16* sp = reinterpret_cast<_Float16*>(a.stacked_tensors[(int64_t)chunk]) + stacked_row * a.hd + (int64_t)c * step;
  _Float16* cp = reinterpret_cast<_Float16*>(a.contiguous_tensors[(int64_t)b]) + cont_row * a.hd + (int64_t)c * step;
  *src = a.to_stacked ? cp : sp;
  *dst = a.to_stacked ? sp : cp;
}

template <typename I>
__device__ __forceinline__ void kvbm_copy_body(const KvbmArgs& a, int64_t total, int64_t rows_per_chunk) {
  constexpr int kPerLane = 1;                 // vectors in flight per lane
  const bool vec = a.per_row != a.hd;
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  for (int64_t i0 = (int64_t)blockIdx.x * kThreads + threadIdx.x; i0 < total; i0 += stride * kPerLane) {
    const _Float16* src[kPerLane];
    _Float16* dst[kPerLane];
    u32x4 v[kPerLane];
#pragma unroll
    for (int u = 0; u < kPerLane; ++u) {
      const int64_t i = i0 + u * stride;
      if (i < total) {
        kvbm_locate<I>(a, (I)i, (I)rows_per_chunk, &src[u], &dst[u]);
        if (vec) v[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src[u]));
      }
    }
    // a block changes layout on its way to another tier or to a later launch: read once, written once, past the caches
#pragma unroll
    for (int u = 0; u < kPerLane; ++u) {
      const int64_t i = i0 + u * stride;
      if (i < total) {
        if (vec) __builtin_nontemporal_store(v[u], reinterpret_cast<u32x4*>(dst[u]));
        else *dst[u] = *src[u];
      }
    }
  }
}

}  // namespace

extern "C" __global__ void __launch_bounds__(kThreads)
    kvbm_copy_entry__f16(const int64_t* stacked_tensors, const int64_t* contiguous_tensors, int32_t to_stacked,
                         int32_t stacked_hnd, int32_t contiguous_layout, int32_t num_blocks, int32_t nh, int32_t nl,
                         int32_t no, int32_t nt, int32_t hd) {
  KvbmArgs a;
  a.stacked_tensors = stacked_tensors, a.contiguous_tensors = contiguous_tensors;
  a.to_stacked = to_stacked, a.stacked_hnd = stacked_hnd, a.contiguous_layout = contiguous_layout;
  a.nh = nh, a.nl = nl, a.no = no, a.nt = nt, a.hd = hd;
  a.per_row = hd % 8 == 0 ? hd / 8 : hd;      // 16-byte vectors per (head, token) row, else elements
  const int64_t rows_per_chunk = (int64_t)nh * nt;
  const int64_t total = (int64_t)num_blocks * nl * no * rows_per_chunk * a.per_row;
  if (total < (1ll << 31)) kvbm_copy_body<uint32_t>(a, total, rows_per_chunk);
  else kvbm_copy_body<int64_t>(a, total, rows_per_chunk);
}
