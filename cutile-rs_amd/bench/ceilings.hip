// Ceiling probes for bench.py: what one MI355X sustains on the bare resources the
// tile kernels are priced against.  They are not tile kernels and are not part of
// the host library: the build writes them to their own code object
// (lib/probes.hsaco), which bench.py loads through the C ABI's module calls
// (cutile_module_load_data / cutile_module_get_function / cutile_launch_kernel).
//
//   probe_mfma_bf16    nothing but v_mfma_f32_32x32x16_bf16 on register operands,
//                      eight independent accumulators per wavefront, two wavefronts
//                      per SIMD.  `mode` 0: operands are ones (few bits toggle);
//                      1: operands are hashed values with random signs and
//                      mantissas in [0.5, 2), the bit activity of real GEMM data.
//                      The gap between the two is the power cap at work.
//   probe_mfma_bf16_lds  the same loop with the GEMM kernel's operand traffic: six
//                      16-byte LDS fragment reads per eight MFMAs.
//   probe_mfma16_bf16 / probe_mfma16_bf16_lds   the two loops on v_mfma_f32_16x16x32_bf16
//                      (64 MFMAs, twice the flops, per iteration).
//   probe_valu_exp2    v_exp_f32 against the multiply-adds of a software exp2, alone and interleaved
//   probe_stream_read / _write / _copy   16-byte nontemporal accesses over a
//                      buffer, the access pattern of the row kernels.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

namespace {

__device__ __forceinline__ uint32_t hash32(uint32_t x) {
  x *= 2654435761u; x ^= x >> 15; x *= 2246822519u; x ^= x >> 13; x *= 3266489917u; x ^= x >> 16;
  return x;
}
// two bf16 values: random sign, exponent 126..127 (|v| in [0.5, 2)), random mantissa
__device__ __forceinline__ uint32_t random_bf16_pair(uint32_t h) { return (h & 0x80ff80ffu) | 0x3f003f00u; }

template <bool USE_LDS>
__device__ __forceinline__ void mfma_loop(float* sink, int32_t iters, int32_t mode) {
  constexpr int TM = 4, TN = 2;
  __shared__ __attribute__((aligned(1024))) unsigned char lds[USE_LDS ? 65536 : 16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (USE_LDS) {
    for (int i = tid; i < 65536 / 4; i += blockDim.x)
      ((uint32_t*)lds)[i] = mode ? random_bf16_pair(hash32(i + blockIdx.x * 7919u)) : 0x3f803f80u;
    __syncthreads();
  }
  bf16x8 a[2][TM], b[2][TN];
  const int r = (wave & 3) * 32 + (lane & 31), u = (lane >> 5) ^ ((r >> 1) & 7);
  const uint32_t addr = r * 128 + u * 16;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
#pragma unroll
    for (int i = 0; i < TM + TN; ++i) {
      u32x4 v;
#pragma unroll
      for (int c = 0; c < 4; ++c)
        v[c] = mode ? random_bf16_pair(hash32((uint32_t)(blockIdx.x * blockDim.x + tid) * 64u + h * 32 + i * 4 + c)) : 0x3f803f80u;
      if (i < TM) a[h][i] = __builtin_bit_cast(bf16x8, v);
      else b[h][i - TM] = __builtin_bit_cast(bf16x8, v);
    }
  }
  f32x16 acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      if (USE_LDS) {
        const uint32_t o = ((it * 2 + half) & 3) * 512;
#pragma unroll
        for (int i = 0; i < TM; ++i) a[half ^ 1][i] = *(const bf16x8*)(lds + addr + i * 4096 + o);
#pragma unroll
        for (int i = 0; i < TN; ++i) b[half ^ 1][i] = *(const bf16x8*)(lds + addr + 32768 + i * 4096 + o);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
          acc[tn][tm] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[half][tn], a[half][tm], acc[tn][tm], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) s += acc[i][j][v];
  sink[(size_t)blockIdx.x * blockDim.x + tid] = s;
}

// The same two loops on v_mfma_f32_16x16x32_bf16: per iteration 64 MFMAs on a 8 x 4 grid of 16 x 16 accumulator
// blocks (two 32-wide K steps; twice the flops of an iteration of the loops above), with the GemmRing16 kernel's operand traffic in the LDS
// form (eight 16-byte x fragment reads and four y fragment reads per 32 MFMAs).  Per flop this form writes half as
// many accumulator values, and on random operands that shows at the power limit.
template <bool USE_LDS>
__device__ __forceinline__ void mfma16_loop(float* sink, int32_t iters, int32_t mode) {
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  constexpr int TM = 8, TN = 4;
  __shared__ __attribute__((aligned(1024))) unsigned char lds[USE_LDS ? 65536 : 16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (USE_LDS) {
    for (int i = tid; i < 65536 / 4; i += blockDim.x)
      ((uint32_t*)lds)[i] = mode ? random_bf16_pair(hash32(i + blockIdx.x * 7919u)) : 0x3f803f80u;
    __syncthreads();
  }
  bf16x8 a[TM / 2], b[2][TN];
  const int r = (wave & 3) * 32 + (lane & 15), u = (lane >> 4) ^ ((r >> 1) & 7);
  const uint32_t addr = r * 128 + u * 16;
#pragma unroll
  for (int i = 0; i < TM / 2 + 2 * TN; ++i) {
    u32x4 v;
#pragma unroll
    for (int c = 0; c < 4; ++c)
      v[c] = mode ? random_bf16_pair(hash32((uint32_t)(blockIdx.x * blockDim.x + tid) * 64u + i * 4 + c)) : 0x3f803f80u;
    if (i < TM / 2) a[i] = __builtin_bit_cast(bf16x8, v);
    else b[(i - TM / 2) / TN][(i - TM / 2) % TN] = __builtin_bit_cast(bf16x8, v);
  }
  f32x4 acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {       // one 32-wide K step: 32 MFMAs in two blocks of 16
#pragma unroll
      for (int mh = 0; mh < 2; ++mh) {
        const uint32_t o = ((it * 4 + half * 2 + mh) & 3) * 512;
        if (USE_LDS && mh == 1) {
#pragma unroll
          for (int i = 0; i < TN; ++i) b[half ^ 1][i] = *(const bf16x8*)(lds + addr + 32768 + i * 4096 + o);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int tm = 0; tm < TM / 2; ++tm) {
#pragma unroll
          for (int tn = 0; tn < TN; ++tn)
            acc[tn][mh * (TM / 2) + tm] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[half][tn], a[tm], acc[tn][mh * (TM / 2) + tm], 0, 0, 0);
          if (USE_LDS) a[tm] = *(const bf16x8*)(lds + addr + tm * 4096 + o);   // the fragment of the next block
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) s += acc[i][j][v];
  sink[(size_t)blockIdx.x * blockDim.x + tid] = s;
}
}  // namespace
extern "C" __global__ void __launch_bounds__(512) probe_mfma16_bf16(float* sink, int32_t iters, int32_t mode) {
  mfma16_loop<false>(sink, iters, mode);
}
extern "C" __global__ void __launch_bounds__(512) probe_mfma16_bf16_lds(float* sink, int32_t iters, int32_t mode) {
  mfma16_loop<true>(sink, iters, mode);
}
// What an exponential costs the vector ALU next to multiply-adds: per iteration and lane 16 independent chains of
// mode 0: v_exp_f32 and one add; mode 1: seven fused multiply-adds (a range reduction plus a cubic, the least a
// software exp2 takes); mode 2: both interleaved.  Mode 2 taking the sum of modes 0 and 1 says the two share one
// issue port; mode 1 taking longer than mode 0 says a polynomial does not relieve it.
template <int MODE>
__device__ __forceinline__ void valu_exp2_loop(float* sink, int32_t iters, float seed) {
  float v[16], w[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    v[i] = seed + 0.001f * (float)(threadIdx.x + i);
    w[i] = seed * 0.5f + (float)i;
  }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      if (MODE != 1) v[i] = __builtin_amdgcn_exp2f(v[i]) - 1.0f;
      if (MODE != 0) {
#pragma unroll
        for (int f = 0; f < 7; ++f) w[i] = __builtin_fmaf(w[i], 0.999f, 0.001f);
      }
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) s += v[i] + w[i];
  sink[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}
extern "C" __global__ void __launch_bounds__(512) probe_valu_exp2(float* sink, int32_t iters, int32_t mode) {
  if (mode == 0) valu_exp2_loop<0>(sink, iters, 0.3f);
  else if (mode == 1) valu_exp2_loop<1>(sink, iters, 0.3f);
  else valu_exp2_loop<2>(sink, iters, 0.3f);
}
// flops per launch = gridDim.x * (blockDim.x / 64) * iters * 2 * 8 * (2 * 32 * 32 * 16); twice that for the mfma16 probes
extern "C" __global__ void __launch_bounds__(512) probe_mfma_bf16(float* sink, int32_t iters, int32_t mode) {
  mfma_loop<false>(sink, iters, mode);
}
extern "C" __global__ void __launch_bounds__(512) probe_mfma_bf16_lds(float* sink, int32_t iters, int32_t mode) {
  mfma_loop<true>(sink, iters, mode);
}

// Each workgroup walks chunks of 256 lanes x VEC vectors, chunk c, c + gridDim.x, ...; n_vec is a multiple of 256 * VEC.
// Store policies: 0 plain, 1 nontemporal, 2 sc1, 3 sc0 sc1 (the cache-scope bits of gfx950 stores).
namespace {
template <int POLICY>
__device__ __forceinline__ void store_vec(u32x4* p, u32x4 v) {
  if (POLICY == 0) *p = v;
  else if (POLICY == 1) __builtin_nontemporal_store(v, p);
  else if (POLICY == 2) asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
  else asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" ::"v"(p), "v"(v) : "memory");
}
template <int POLICY, int VEC>
__device__ __forceinline__ void write_stream(u32x4* dst, uint64_t n_vec) {
  const u32x4 x = {threadIdx.x, blockIdx.x, 0x3c003c00u, 0xbc00bc00u};
  for (uint64_t base = (uint64_t)blockIdx.x * 256 * VEC; base < n_vec; base += (uint64_t)gridDim.x * 256 * VEC) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) store_vec<POLICY>(dst + base + i * 256 + threadIdx.x, x);
  }
}
template <int POLICY, int VEC>
__device__ __forceinline__ void copy_stream(const u32x4* src, u32x4* dst, uint64_t n_vec) {
  for (uint64_t base = (uint64_t)blockIdx.x * 256 * VEC; base < n_vec; base += (uint64_t)gridDim.x * 256 * VEC) {
    u32x4 v[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = __builtin_nontemporal_load(src + base + i * 256 + threadIdx.x);
#pragma unroll
    for (int i = 0; i < VEC; ++i) store_vec<POLICY>(dst + base + i * 256 + threadIdx.x, v[i]);
  }
}
}  // namespace

constexpr int kVec = 8;
extern "C" __global__ void __launch_bounds__(256) probe_stream_read(const u32x4* src, u32x4* sink, uint64_t n_vec) {
  u32x4 x = {0, 0, 0, 0};
  for (uint64_t base = (uint64_t)blockIdx.x * 256 * kVec; base < n_vec; base += (uint64_t)gridDim.x * 256 * kVec) {
    u32x4 v[kVec];
#pragma unroll
    for (int i = 0; i < kVec; ++i) v[i] = __builtin_nontemporal_load(src + base + i * 256 + threadIdx.x);
#pragma unroll
    for (int i = 0; i < kVec; ++i) x ^= v[i];
  }
  if ((x[0] ^ x[1] ^ x[2] ^ x[3]) == 0x9e3779b9u) sink[threadIdx.x] = x;   // keeps the loads alive; practically never taken
}
#define WRITE_PROBE(NAME, POLICY) \
  extern "C" __global__ void __launch_bounds__(256) probe_stream_write_##NAME(u32x4* dst, uint64_t n_vec) { write_stream<POLICY, 8>(dst, n_vec); }
WRITE_PROBE(plain, 0)
WRITE_PROBE(nt, 1)
WRITE_PROBE(sc1, 2)
WRITE_PROBE(sc0sc1, 3)
#define COPY_PROBE(NAME, POLICY, VEC) \
  extern "C" __global__ void __launch_bounds__(256) probe_stream_copy_##NAME(const u32x4* src, u32x4* dst, uint64_t n_vec) { copy_stream<POLICY, VEC>(src, dst, n_vec); }
COPY_PROBE(plain_v8, 0, 8)
COPY_PROBE(nt_v8, 1, 8)
COPY_PROBE(nt_v4, 1, 4)
COPY_PROBE(sc0sc1_v8, 3, 8)
