// Device random fills behind the RNG entries of the C ABI (the reference binds cuRAND's generator for
// api::randn / api::rand: cuda-core/src/api.rs:214-293, cutile/src/api.rs:683-719).
//
// Generator: Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3",
// SC'11), counter based: block b of a stream is philox(key = seed, counter = (b, 0)), four 32-bit words.
// An element never depends on which lane or launch produced it, only on (seed, stream position):
//   f32: element e uses word e % 4 of block (offset + e / 4)
//   f64: element e uses words 2 (e % 2), 2 (e % 2) + 1 of block (offset + e / 2)
// uniform f32 = (word >> 8) * 2^-24 in [0, 1); uniform f64 = ((hi << 21) ^ (lo >> 11)) * 2^-53 in [0, 1);
// normal: Box-Muller on the two uniforms of a pair (u1 moved to (0, 1]): elements 2i, 2i + 1 are
// r cos(t), r sin(t) with r = sqrt(-2 ln u1), t = 2 pi u2.
// HBM-bound: 16-byte stores, one Philox block per four f32 (two f64) values.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

struct u4 { uint32_t x, y, z, w; };

__device__ __forceinline__ u4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1) {
  constexpr uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u, W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint32_t hi0 = __umulhi(M0, c0), lo0 = M0 * c0;
    const uint32_t hi1 = __umulhi(M1, c2), lo1 = M1 * c2;
    const uint32_t n0 = hi1 ^ c1 ^ k0, n2 = hi0 ^ c3 ^ k1;
    c0 = n0; c1 = lo1; c2 = n2; c3 = lo0;
    k0 += W0; k1 += W1;
  }
  return u4{c0, c1, c2, c3};
}

__device__ __forceinline__ float uniform_f32(uint32_t w) { return (float)(w >> 8) * 5.9604644775390625e-8f; }          // 2^-24
__device__ __forceinline__ float uniform_f32_open0(uint32_t w) { return (float)((w >> 8) + 1u) * 5.9604644775390625e-8f; }
__device__ __forceinline__ double uniform_f64(uint32_t lo, uint32_t hi) {
  return (double)((((uint64_t)hi) << 21) ^ (uint64_t)(lo >> 11)) * 1.1102230246251565e-16;                                  // 2^-53
}

}  // namespace

// kind 0: uniform [0, 1); kind 1: normal(mean, std).  Each lane walks blocks lane, lane + total lanes, ...
extern "C" __global__ void __launch_bounds__(256) rng_fill_entry__f32(float* out, uint64_t n, uint64_t seed, uint64_t offset,
                                                                       int32_t kind, float mean, float std) {
  const uint64_t blocks = (n + 3) / 4, stride = (uint64_t)gridDim.x * blockDim.x;
  const uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
  for (uint64_t b = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; b < blocks; b += stride) {
    const uint64_t ctr = offset + b;
    const u4 r = philox4x32_10((uint32_t)ctr, (uint32_t)(ctr >> 32), 0u, 0u, k0, k1);
    float v[4];
    if (kind == 0) {
      v[0] = uniform_f32(r.x); v[1] = uniform_f32(r.y); v[2] = uniform_f32(r.z); v[3] = uniform_f32(r.w);
    } else {
      const float r0 = sqrtf(-2.0f * logf(uniform_f32_open0(r.x))), r1 = sqrtf(-2.0f * logf(uniform_f32_open0(r.z)));
      float s0, c0, s1, c1;
      sincosf(6.283185307179586f * uniform_f32(r.y), &s0, &c0);
      sincosf(6.283185307179586f * uniform_f32(r.w), &s1, &c1);
      v[0] = fmaf(std, r0 * c0, mean); v[1] = fmaf(std, r0 * s0, mean);
      v[2] = fmaf(std, r1 * c1, mean); v[3] = fmaf(std, r1 * s1, mean);
    }
    const uint64_t e = b * 4;
    if (e + 4 <= n && (((uintptr_t)out) & 15) == 0) {
      *reinterpret_cast<float4*>(out + e) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
      for (int i = 0; i < 4; ++i)
        if (e + i < n) out[e + i] = v[i];
    }
  }
}

extern "C" __global__ void __launch_bounds__(256) rng_fill_entry__f64(double* out, uint64_t n, uint64_t seed, uint64_t offset,
                                                                       int32_t kind, double mean, double std) {
  const uint64_t blocks = (n + 1) / 2, stride = (uint64_t)gridDim.x * blockDim.x;
  const uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
  for (uint64_t b = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; b < blocks; b += stride) {
    const uint64_t ctr = offset + b;
    const u4 r = philox4x32_10((uint32_t)ctr, (uint32_t)(ctr >> 32), 0u, 0u, k0, k1);
    double v0 = uniform_f64(r.x, r.y), v1 = uniform_f64(r.z, r.w);
    if (kind != 0) {
      const double u1 = v0 + 1.1102230246251565e-16;   // (0, 1]
      const double rad = sqrt(-2.0 * log(u1));
      double s, c;
      sincos(6.283185307179586476925 * v1, &s, &c);
      v0 = fma(std, rad * c, mean);
      v1 = fma(std, rad * s, mean);
    }
    const uint64_t e = b * 2;
    if (e + 2 <= n && (((uintptr_t)out) & 15) == 0) {
      *reinterpret_cast<double2*>(out + e) = make_double2(v0, v1);
    } else {
      if (e < n) out[e] = v0;
      if (e + 1 < n) out[e + 1] = v1;
    }
  }
}
