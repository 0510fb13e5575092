// MX block-scaled fp8 GEMM for gfx950:
//   z[M,N] = alpha * sum_k (x[i,k] * sx[i,k/32]) * (y[j,k] * sy[j,k/32])
// x [M,K] and y [N,K] are fp8 e4m3fn bytes (both K-contiguous), sx [M,K/32] and
// sy [N,K/32] are e8m0 scale bytes (2^(b-127)), accumulation is f32.
//
// Tile program being implemented (cutile-examples/examples/mxfp8.rs:34-64): per
// [BM,BN] output tile, for each K tile: tile_z = mmaf_scaled(x, yᵀ, tile_z, sx, syᵀ);
// then z.store(tile_z * alpha).  The op contract is cutile/src/_core.rs:2283-2311.
//
// Mapping to CDNA4: v_mfma_scale_f32_32x32x64_f8f6f4 multiplies a 32x64 by a
// 64x32 fp8 block and scales each 32-wide K block of every row by an e8m0 byte,
// so the scales never touch the data path: no dequantisation, no extra
// multiplies.  Operand layout (measured on gfx950): a lane (row r = lane%32,
// half h = lane/32) holds 32 bytes; its first 16 belong to the instruction's K
// block 0 (bytes 16h..16h+15 of it) and its last 16 to K block 1; lanes with
// h = 0 supply the scale of block 0 for their row and lanes with h = 1 the scale
// of block 1, as byte 0 of the scale VGPR.  The
// four scale bytes a row needs for a 128-wide K tile are fetched as one aligned
// dword straight from global memory (they are 1/32 of the data) and shifted so
// that the lane's own block sits in the byte the instruction reads.
// Data tiles go through LDS exactly like the bf16 GEMM's x tile (both operands
// are K-contiguous here, so there is no transpose at all): double buffered,
// XOR-swizzled 16-byte units, one barrier per K tile, buffer-descriptor loads
// for branch-free zero padding, transposed MFMA issue for 4-column-per-lane
// stores, XCD-aware grouped tile order.
#include <hip/hip_runtime.h>

#include "kernel_args.h"

using namespace cutile;

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kNumXcd = 8;
constexpr int kGroupM = 8;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  uint32_t a = __builtin_bit_cast(uint32_t, lo), b = __builtin_bit_cast(uint32_t, hi);
  a += 0x7fffu + ((a >> 16) & 1u);
  b += 0x7fffu + ((b >> 16) & 1u);
  return (a >> 16) | (b & 0xffff0000u);
}

__device__ __forceinline__ void tile_coords(uint32_t tiles_m, uint32_t tiles_n, uint32_t* pm,
                                            uint32_t* pn) {
  const uint32_t total = tiles_m * tiles_n;
  uint32_t id = blockIdx.x;
  if (total % kNumXcd == 0) id = (id % kNumXcd) * (total / kNumXcd) + id / kNumXcd;
  const uint32_t per_group = kGroupM * tiles_n;
  const uint32_t group = id / per_group;
  const uint32_t first_m = group * kGroupM;
  const uint32_t rows = min(tiles_m - first_m, (uint32_t)kGroupM);
  const uint32_t in_group = id % per_group;
  *pm = first_m + in_group % rows;
  *pn = in_group / rows;
}

template <int BM, int BN, int WAVES_M, int WAVES_N, typename OutT>
struct MxGemm {
  static constexpr int BK = 128;  // fp8 elements (= bytes) per K tile: four MX blocks
  static constexpr int kWaves = WAVES_M * WAVES_N;
  static constexpr int kThreads = kWaves * 64;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int kUnitsPerRow = BK / 16;
  static constexpr int kALoads = BM * kUnitsPerRow / kThreads;
  static constexpr int kBLoads = BN * kUnitsPerRow / kThreads;
  static constexpr int kABytes = BM * BK, kBBytes = BN * BK;
  static constexpr int kStageBytes = kABytes + kBBytes;
  static constexpr int kLdsBytes = 2 * kStageBytes;
  static_assert((BM * kUnitsPerRow) % kThreads == 0 && (BN * kUnitsPerRow) % kThreads == 0, "split");

  __device__ static __forceinline__ int lds_off(int r, int u) {
    return r * BK + ((u ^ ((r >> 1) & 7)) << 4);
  }

  __device__ static void run(const PartitionArg<2>& z, const TensorArg<2>& x, const TensorArg<2>& y,
                             const TensorArg<2>& xs, const TensorArg<2>& ys, float alpha,
                             const TileGrid& g) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[kLdsBytes];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int l32 = lane & 31, khalf = lane >> 5;
    uint32_t pm, pn;
    tile_coords(g.x, g.y, &pm, &pn);
    const int32_t M = x.shape[0], N = y.shape[0], K = min(x.shape[1], y.shape[1]);
    const int32_t lda = x.strides[0], ldb = y.strides[0];
    const int32_t ldsa = xs.strides[0], ldsb = ys.strides[0];
    const int32_t row0 = pm * BM, col0 = pn * BN;

    const __amdgpu_buffer_rsrc_t ra = make_rsrc(x.ptr, (uint32_t)((int64_t)(M - 1) * lda + x.shape[1]));
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(y.ptr, (uint32_t)((int64_t)(N - 1) * ldb + y.shape[1]));
    const __amdgpu_buffer_rsrc_t rsa = make_rsrc(xs.ptr, (uint32_t)((int64_t)(xs.shape[0] - 1) * ldsa + xs.shape[1]));
    const __amdgpu_buffer_rsrc_t rsb = make_rsrc(ys.ptr, (uint32_t)((int64_t)(ys.shape[0] - 1) * ldsb + ys.shape[1]));
    constexpr uint32_t kOob = 0x80000000u;

    int a_row[kALoads], a_unit[kALoads], b_row[kBLoads], b_unit[kBLoads];
#pragma unroll
    for (int i = 0; i < kALoads; ++i) {
      int c = tid + i * kThreads;
      a_row[i] = c / kUnitsPerRow;
      a_unit[i] = c % kUnitsPerRow;
    }
#pragma unroll
    for (int i = 0; i < kBLoads; ++i) {
      int c = tid + i * kThreads;
      b_row[i] = c / kUnitsPerRow;
      b_unit[i] = c % kUnitsPerRow;
    }
    u32x4 a_reg[kALoads], b_reg[kBLoads];
    uint32_t sa_reg[TM], sb_reg[TN];  // one dword = the 4 scale bytes of this lane's row for a K tile
    auto load_global = [&](int32_t k0) {
#pragma unroll
      for (int i = 0; i < kALoads; ++i) {
        int32_t r = row0 + a_row[i], kk = k0 + a_unit[i] * 16;
        uint32_t off = (r < M && kk < K) ? (uint32_t)((int64_t)r * lda + kk) : kOob;
        a_reg[i] = __builtin_amdgcn_raw_buffer_load_b128(ra, off, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < kBLoads; ++i) {
        int32_t r = col0 + b_row[i], kk = k0 + b_unit[i] * 16;
        uint32_t off = (r < N && kk < K) ? (uint32_t)((int64_t)r * ldb + kk) : kOob;
        b_reg[i] = __builtin_amdgcn_raw_buffer_load_b128(rb, off, 0, 0);
      }
    };
    auto load_scales = [&](int32_t k0) {
      // Rows beyond the tensor read scale byte 0 (2^-127) against all-zero data: contributes 0.
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) {
        int32_t r = row0 + wm * WM + tm * 32 + l32;
        uint32_t off = r < M ? (uint32_t)((int64_t)r * ldsa + k0 / 32) : kOob;
        sa_reg[tm] = __builtin_amdgcn_raw_buffer_load_b32(rsa, off, 0, 0);
      }
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
        int32_t r = col0 + wn * WN + tn * 32 + l32;
        uint32_t off = r < N ? (uint32_t)((int64_t)r * ldsb + k0 / 32) : kOob;
        sb_reg[tn] = __builtin_amdgcn_raw_buffer_load_b32(rsb, off, 0, 0);
      }
    };
    auto store_lds = [&](int stage) {
      unsigned char* sa = lds + stage * kStageBytes;
      unsigned char* sb = sa + kABytes;
#pragma unroll
      for (int i = 0; i < kALoads; ++i) *reinterpret_cast<u32x4*>(sa + lds_off(a_row[i], a_unit[i])) = a_reg[i];
#pragma unroll
      for (int i = 0; i < kBLoads; ++i) *reinterpret_cast<u32x4*>(sb + lds_off(b_row[i], b_unit[i])) = b_reg[i];
    };

    f32x16 acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[tn][tm][v] = 0.0f;

    const int k_tiles = K / BK;
    uint32_t sa_cur[TM], sb_cur[TN];
    if (k_tiles > 0) {
      load_global(0);
      load_scales(0);
      store_lds(0);
    }
    __syncthreads();

    for (int kt = 0; kt < k_tiles; ++kt) {
      const int cur = kt & 1;
      // This lane's four scale bytes for the current K tile (MX blocks 4kt..4kt+3).
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) sa_cur[tm] = sa_reg[tm];
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) sb_cur[tn] = sb_reg[tn];
      if (kt + 1 < k_tiles) {
        load_global((kt + 1) * BK);
        load_scales((kt + 1) * BK);
      }
      const unsigned char* sa = lds + cur * kStageBytes;
      const unsigned char* sb = sa + kABytes;
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        i32x8 af[TM], bfr[TN];
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
          int r = wm * WM + tm * 32 + l32;
          u32x4 lo = *reinterpret_cast<const u32x4*>(sa + lds_off(r, ks * 4 + khalf));
          u32x4 hi = *reinterpret_cast<const u32x4*>(sa + lds_off(r, ks * 4 + 2 + khalf));
          af[tm] = i32x8{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
        }
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
          int r = wn * WN + tn * 32 + l32;
          u32x4 lo = *reinterpret_cast<const u32x4*>(sb + lds_off(r, ks * 4 + khalf));
          u32x4 hi = *reinterpret_cast<const u32x4*>(sb + lds_off(r, ks * 4 + 2 + khalf));
          bfr[tn] = i32x8{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
        }
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
          for (int tm = 0; tm < TM; ++tm) {
            // MFMA step ks covers MX blocks 2ks and 2ks+1 of the K tile; lanes 0-31 supply
            // the scale of the first, lanes 32-63 of the second, moved to byte 0.
            acc[tn][tm] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                bfr[tn], af[tm], acc[tn][tm], 0, 0, 0, (int)(sb_cur[tn] >> (8 * (2 * ks + khalf))), 0,
                (int)(sa_cur[tm] >> (8 * (2 * ks + khalf))));
          }
      }
      if (kt + 1 < k_tiles) store_lds(cur ^ 1);
      __syncthreads();
    }

    OutT* zp = (OutT*)z.ptr;
    const int32_t ldz = z.strides[0];
    const int32_t zM = z.shape[0], zN = z.shape[1];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      const int32_t r = row0 + wm * WM + tm * 32 + l32;
      if (r >= zM) continue;
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int32_t c = col0 + wn * WN + tn * 32 + q * 8 + khalf * 4;
          if (c >= zN) continue;
          OutT* dst = zp + (int64_t)r * ldz + c;
          float v0 = acc[tn][tm][q * 4 + 0] * alpha, v1 = acc[tn][tm][q * 4 + 1] * alpha;
          float v2 = acc[tn][tm][q * 4 + 2] * alpha, v3 = acc[tn][tm][q * 4 + 3] * alpha;
          if constexpr (sizeof(OutT) == 2) {
            u32x2 o;
            o.x = pack_bf16x2(v0, v1);
            o.y = pack_bf16x2(v2, v3);
            *reinterpret_cast<u32x2*>(dst) = o;
          } else {
            f32x4 o = {v0, v1, v2, v3};
            *reinterpret_cast<f32x4*>(dst) = o;
          }
        }
    }
  }
};

}  // namespace

#define MX_KERNEL(NAME, BM, BN, WVM, WVN, OUT_T)                                                   \
  extern "C" __global__ void __launch_bounds__(WVM* WVN * 64)                                     \
      linear_tile_entry__##NAME(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y, TensorArg<2> xs, \
                                TensorArg<2> ys, float alpha, TileGrid g) {                        \
    MxGemm<BM, BN, WVM, WVN, OUT_T>::run(z, x, y, xs, ys, alpha, g);                               \
  }

MX_KERNEL(mxfp8_bf16_256x256x128_w2x2, 256, 256, 2, 2, __bf16)
MX_KERNEL(mxfp8_bf16_256x256x128_w2x4, 256, 256, 2, 4, __bf16)
MX_KERNEL(mxfp8_bf16_128x128x128_w2x2, 128, 128, 2, 2, __bf16)
MX_KERNEL(mxfp8_f32_256x256x128_w2x2, 256, 256, 2, 2, float)
MX_KERNEL(mxfp8_f32_128x128x128_w2x2, 128, 128, 2, 2, float)
MX_KERNEL(mxfp8_f32_32x32x128_w1x1, 32, 32, 1, 1, float)
MX_KERNEL(mxfp8_f32_64x64x128_w1x1, 64, 64, 1, 1, float)
