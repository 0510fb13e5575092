// Elementwise and creation kernels for gfx950: saxpy, axpy with a separate
// output, add, full, arange, linspace, convert.
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

// ---- creation ------------------------------------------------------------------------------
#define CREATION_KERNELS(T, NAME)                                                                   \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      full_entry__##NAME(T value, PartitionArg<1> t, TileGrid g) {                                  \
    size_t count = covered_1d(t.shape[0], t.pshape[0], g);                                         \
    size_t stride = (size_t)gridDim.x * kThreads;                                                  \
    for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < count; i += stride)          \
      ((T*)t.ptr)[i * t.strides[0]] = value;                                                       \
  }                                                                                                 \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      arange_entry__##NAME(PartitionArg<1> t, TileGrid g) {                                         \
    size_t count = covered_1d(t.shape[0], t.pshape[0], g);                                         \
    size_t stride = (size_t)gridDim.x * kThreads;                                                  \
    for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < count; i += stride)          \
      ((T*)t.ptr)[i * t.strides[0]] = (T)(int32_t)i;                                               \
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
  size_t count = covered_1d(t.shape[0], t.pshape[0], g);
  size_t stride = (size_t)gridDim.x * kThreads;
  for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < count; i += stride)
    ((float*)t.ptr)[i * t.strides[0]] = start + (float)(int32_t)i * step;
}

// ---- convert -------------------------------------------------------------------------------
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

#define CONVERT_KERNEL(S, SN, D, DN)                                                                \
  extern "C" __global__ void __launch_bounds__(kThreads)                                           \
      convert_entry__##SN##_##DN(TensorArg<1> src, PartitionArg<1> dst, TileGrid g) {               \
    size_t count = covered_1d(dst.shape[0], dst.pshape[0], g);                                     \
    size_t stride = (size_t)gridDim.x * kThreads;                                                  \
    for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < count; i += stride) {        \
      S v = i < (size_t)src.shape[0] ? ((const S*)src.ptr)[i * src.strides[0]] : S(0);            \
      ((D*)dst.ptr)[i * dst.strides[0]] = convert_elem<D, S>(v);                                   \
    }                                                                                               \
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
