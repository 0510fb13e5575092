// Tiled bf16 GEMM for gfx950: z[M,N] (+)= x[M,K] · y[K,N], f32 accumulation on
// the matrix cores, bf16 (or f32) output.
//
// Tile program being implemented (cutile-benchmarks/benches/gemm.rs:20-41,
// cutile-examples/examples/gemm.rs:20-36): one tile block per [BM,BN] output
// tile; acc = z.load() (or 0); for i in 0..K/BK: acc = mma(x[pid0,i], y[i,pid1], acc);
// z.store(acc).  Loads outside a tensor read 0, stores outside z are dropped.
//
// Mapping to CDNA4:
//  * one workgroup per output tile, WAVES_M x WAVES_N wavefronts, each owning a
//    WM x WN sub-tile built from v_mfma_f32_32x32x16_bf16 (64-lane wavefronts,
//    8 K-values per lane per operand);
//  * x and y tiles are staged through LDS, double buffered, one barrier per
//    K-step; the next tile's global loads are issued before the current tile's
//    MFMAs so HBM/L2 latency hides under matrix work;
//  * x is K-contiguous, which is what an MFMA operand wants (ds_read_b128 per
//    lane).  y is N-contiguous; its operand is formed with ds_read_b64_tr_b16,
//    the LDS transpose read of gfx950, so no transposed copy of y is ever made;
//  * both LDS tiles are XOR-swizzled in 16-byte units so operand reads spread
//    over the banks;
//  * the MFMA is issued with y's fragment as its first operand and x's as the
//    second, i.e. it produces the transposed tile: each lane then holds 4
//    consecutive N-columns of one output row, which turns the epilogue into
//    8-byte stores instead of 2-byte ones;
//  * global reads go through buffer descriptors, whose out-of-range reads return
//    0 — exactly the tile program's zero padding, with no branches;
//  * workgroup ids are remapped so that each XCD (own L2) works on a compact
//    band of output tiles, walked in groups of GROUP_M tile rows.
#include <hip/hip_runtime.h>

#include "kernel_args.h"

using namespace cutile;

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define LDS_PTR(T) __attribute__((address_space(3))) T*

constexpr int kNumXcd = 8;
constexpr int kGroupM = 8;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  // round-to-nearest-even; inputs are finite products/sums (NaN keeps a NaN pattern)
  uint32_t a = __builtin_bit_cast(uint32_t, lo), b = __builtin_bit_cast(uint32_t, hi);
  a += 0x7fffu + ((a >> 16) & 1u);
  b += 0x7fffu + ((b >> 16) & 1u);
  return (a >> 16) | (b & 0xffff0000u);
}

// Tile index for this workgroup: XCD-contiguous, then grouped along M.
__device__ __forceinline__ void tile_coords(uint32_t tiles_m, uint32_t tiles_n, uint32_t* pm,
                                            uint32_t* pn) {
  const uint32_t total = tiles_m * tiles_n;
  uint32_t id = blockIdx.x;
  // Workgroups are dealt round-robin to the XCDs; give each XCD a contiguous
  // range of logical tile ids (only when the count divides evenly, otherwise the
  // plain order is kept so every tile is still covered exactly once).
  if (total % kNumXcd == 0) id = (id % kNumXcd) * (total / kNumXcd) + id / kNumXcd;
  const uint32_t per_group = kGroupM * tiles_n;
  const uint32_t group = id / per_group;
  const uint32_t first_m = group * kGroupM;
  const uint32_t rows = min(tiles_m - first_m, (uint32_t)kGroupM);
  const uint32_t in_group = id % per_group;
  *pm = first_m + in_group % rows;
  *pn = in_group / rows;
}

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, typename OutT>
struct Gemm {
  static constexpr int kWaves = WAVES_M * WAVES_N;
  static constexpr int kThreads = kWaves * 64;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int kAChunksPerRow = BK / 8;          // 16-byte units per x-tile row
  static constexpr int kBChunksPerRow = BN / 8;          // 16-byte units per y-tile row
  static constexpr int kAChunks = BM * kAChunksPerRow;
  static constexpr int kBChunks = BK * kBChunksPerRow;
  static constexpr int kALoads = kAChunks / kThreads;
  static constexpr int kBLoads = kBChunks / kThreads;
  static constexpr int kABytes = BM * BK * 2, kBBytes = BK * BN * 2;
  static constexpr int kStageBytes = kABytes + kBBytes;
  static constexpr int kLdsBytes = 2 * kStageBytes;
  static_assert(BK == 64, "the x-tile swizzle assumes 8 sixteen-byte units per row");
  static_assert(kAChunks % kThreads == 0 && kBChunks % kThreads == 0, "tile must split evenly");
  static_assert(kBChunksPerRow >= 16, "the y-tile swizzle needs at least 16 units per row");

  // x tile: row-major [BM][BK]; unit u of row r lives at unit (u ^ ((r >> 1) & 7)).
  __device__ static __forceinline__ int a_lds_off(int r, int u) {
    return r * (BK * 2) + ((u ^ ((r >> 1) & 7)) << 4);
  }
  // y tile: row-major [BK][BN]; unit u of k-row r lives at unit (u ^ ((r & 3) << 2)).
  __device__ static __forceinline__ int b_lds_off(int r, int u) {
    return r * (BN * 2) + ((u ^ ((r & 3) << 2)) << 4);
  }

  __device__ static void run(const PartitionArg<2>& z, const TensorArg<2>& x, const TensorArg<2>& y,
                             int32_t k_total, const TileGrid& g, int32_t accumulate) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[kLdsBytes];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    uint32_t pm, pn;
    tile_coords(g.x, g.y, &pm, &pn);
    const int32_t M = x.shape[0], N = y.shape[1];
    const int32_t lda = x.strides[0], ldb = y.strides[0];
    const int32_t row0 = pm * BM, col0 = pn * BN;
    // K actually readable from both operands and asked for; beyond it tiles read 0.
    const int32_t k_valid = min(min(x.shape[1], y.shape[0]), k_total);

    const __amdgpu_buffer_rsrc_t ra = make_rsrc(x.ptr, (uint32_t)(((int64_t)(M - 1) * lda + x.shape[1]) * 2));
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(y.ptr, (uint32_t)(((int64_t)(y.shape[0] - 1) * ldb + N) * 2));
    constexpr uint32_t kOob = 0x80000000u;  // beyond any descriptor -> reads 0

    // Per-thread global -> LDS assignments (fixed over the K loop except for k0).
    int a_row[kALoads], a_unit[kALoads], b_row[kBLoads], b_unit[kBLoads];
#pragma unroll
    for (int i = 0; i < kALoads; ++i) {
      int c = tid + i * kThreads;
      a_row[i] = c / kAChunksPerRow;
      a_unit[i] = c % kAChunksPerRow;
    }
#pragma unroll
    for (int i = 0; i < kBLoads; ++i) {
      int c = tid + i * kThreads;
      b_row[i] = c / kBChunksPerRow;
      b_unit[i] = c % kBChunksPerRow;
    }

    u32x4 a_reg[kALoads], b_reg[kBLoads];
    auto load_global = [&](int32_t k0) {
#pragma unroll
      for (int i = 0; i < kALoads; ++i) {
        int32_t r = row0 + a_row[i], kk = k0 + a_unit[i] * 8;
        uint32_t off = (r < M && kk < k_valid) ? (uint32_t)(((int64_t)r * lda + kk) * 2) : kOob;
        a_reg[i] = __builtin_amdgcn_raw_buffer_load_b128(ra, off, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < kBLoads; ++i) {
        int32_t kk = k0 + b_row[i], c = col0 + b_unit[i] * 8;
        uint32_t off = (kk < k_valid && c < N) ? (uint32_t)(((int64_t)kk * ldb + c) * 2) : kOob;
        b_reg[i] = __builtin_amdgcn_raw_buffer_load_b128(rb, off, 0, 0);
      }
    };
    auto store_lds = [&](int stage) {
      unsigned char* sa = lds + stage * kStageBytes;
      unsigned char* sb = sa + kABytes;
#pragma unroll
      for (int i = 0; i < kALoads; ++i) *reinterpret_cast<u32x4*>(sa + a_lds_off(a_row[i], a_unit[i])) = a_reg[i];
#pragma unroll
      for (int i = 0; i < kBLoads; ++i) *reinterpret_cast<u32x4*>(sb + b_lds_off(b_row[i], b_unit[i])) = b_reg[i];
    };

    f32x16 acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[tn][tm][v] = 0.0f;

    // Lane roles inside the operand reads.
    const int l32 = lane & 31, khalf = lane >> 5;          // x operand: row l32, k-units khalf
    const int grp = lane >> 4, l16 = lane & 15;            // y operand: transpose-read groups
    const int tr_row = l16 >> 2, tr_col = (l16 & 3) * 4;   // address role inside a 4x16 block
    const int b_n_half = (grp & 1) * 16, b_k_half = (grp >> 1) * 8;

    const int k_tiles = (k_total + BK - 1) / BK;
    if (k_tiles > 0) {
      load_global(0);
      store_lds(0);
    }
    __syncthreads();

    for (int kt = 0; kt < k_tiles; ++kt) {
      const int cur = kt & 1;
      if (kt + 1 < k_tiles) load_global((kt + 1) * BK);
      const unsigned char* sa = lds + cur * kStageBytes;
      const unsigned char* sb = sa + kABytes;
#pragma unroll
      for (int ks = 0; ks < BK / 16; ++ks) {
        bf16x8 af[TM], bfr[TN];
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
          int r = wm * WM + tm * 32 + l32;
          af[tm] = *reinterpret_cast<const bf16x8*>(sa + a_lds_off(r, ks * 2 + khalf));
        }
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
          int n = wn * WN + tn * 32 + b_n_half + tr_col;  // first of the 4 columns this lane addresses
          int kr = ks * 16 + b_k_half + tr_row;
          const unsigned char* p0 = sb + b_lds_off(kr, n >> 3) + (n & 7) * 2;
          const unsigned char* p1 = sb + b_lds_off(kr + 4, n >> 3) + (n & 7) * 2;
          s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))p0);
          s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))p1);
          typedef short s16x8 __attribute__((ext_vector_type(8)));
          s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
          bfr[tn] = __builtin_bit_cast(bf16x8, both);
        }
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
          for (int tm = 0; tm < TM; ++tm)
            acc[tn][tm] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[tn], af[tm], acc[tn][tm], 0, 0, 0);
      }
      if (kt + 1 < k_tiles) store_lds(cur ^ 1);
      __syncthreads();
    }

    // Epilogue.  acc[tn][tm][v]: output row = tm*32 + l32, columns
    // tn*32 + (v/4)*8 + khalf*4 + (v%4): four consecutive columns per v-quad.
    OutT* zp = (OutT*)z.ptr;
    const int32_t ldz = z.strides[0];
    const int32_t zM = z.shape[0], zN = z.shape[1];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      const int32_t r = row0 + wm * WM + tm * 32 + l32;
      if (r >= zM) continue;
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int32_t c = col0 + wn * WN + tn * 32 + q * 8 + khalf * 4;
          if (c >= zN) continue;
          OutT* dst = zp + (int64_t)r * ldz + c;
          float v0 = acc[tn][tm][q * 4 + 0], v1 = acc[tn][tm][q * 4 + 1];
          float v2 = acc[tn][tm][q * 4 + 2], v3 = acc[tn][tm][q * 4 + 3];
          if constexpr (sizeof(OutT) == 2) {
            if (accumulate) {
              u32x2 old = *reinterpret_cast<const u32x2*>(dst);
              v0 += __builtin_bit_cast(float, old.x << 16);
              v1 += __builtin_bit_cast(float, old.x & 0xffff0000u);
              v2 += __builtin_bit_cast(float, old.y << 16);
              v3 += __builtin_bit_cast(float, old.y & 0xffff0000u);
            }
            u32x2 o;
            o.x = pack_bf16x2(v0, v1);
            o.y = pack_bf16x2(v2, v3);
            *reinterpret_cast<u32x2*>(dst) = o;
          } else {
            f32x4 o = {v0, v1, v2, v3};
            if (accumulate) o += *reinterpret_cast<const f32x4*>(dst);
            *reinterpret_cast<f32x4*>(dst) = o;
          }
        }
      }
    }
  }
};

}  // namespace

// gemm<bf16, BM, BN, BK>(z, x, y, k) with trailing launch metadata.
#define GEMM_KERNEL(NAME, BM, BN, BK, WVM, WVN, OUT_T)                                          \
  extern "C" __global__ void __launch_bounds__(WVM* WVN * 64)                                  \
      gemm_entry__##NAME(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y, int32_t k, TileGrid g, \
                         int32_t accumulate) {                                                  \
    Gemm<BM, BN, BK, WVM, WVN, OUT_T>::run(z, x, y, k, g, accumulate);                          \
  }

GEMM_KERNEL(bf16_256x256x64_w2x2, 256, 256, 64, 2, 2, __bf16)
GEMM_KERNEL(bf16_256x256x64_w2x4, 256, 256, 64, 2, 4, __bf16)
GEMM_KERNEL(bf16_256x256x64_w4x2, 256, 256, 64, 4, 2, __bf16)
GEMM_KERNEL(bf16_256x128x64_w2x2, 256, 128, 64, 2, 2, __bf16)
GEMM_KERNEL(bf16_128x256x64_w2x2, 128, 256, 64, 2, 2, __bf16)
GEMM_KERNEL(bf16_128x128x64_w2x2, 128, 128, 64, 2, 2, __bf16)
GEMM_KERNEL(bf16_64x128x64_w2x2, 64, 128, 64, 2, 2, __bf16)
GEMM_KERNEL(bf16f32_128x128x64_w2x2, 128, 128, 64, 2, 2, float)
GEMM_KERNEL(bf16f32_256x256x64_w2x2, 256, 256, 64, 2, 2, float)
