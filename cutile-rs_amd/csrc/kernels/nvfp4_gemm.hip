// NVFP4 block-scaled GEMM for gfx950 (CDNA4).
//
// linear_tile of cutile-examples/examples/nvfp4.rs:24-78:
//   z[M, N] = alpha * sum_k  x[i, k] * sx[i, k / 16]  *  y[j, k] * sy[j, k / 16]
// x [M, K/2] and y [N, K/2] hold two e2m1 values per byte (low nibble first,
// cuda-core/src/dtype.rs:60-99), x_scales [M, K/16] and y_scales [N, K/16] are e4m3fn
// bytes, accumulation and z are f32.
//
// CDNA4's scaled matrix instruction takes fp4 operands, but only with one power-of-two
// (e8m0) scale per 32 values: a 3-bit-mantissa scale per 16 values cannot be expressed
// in it.  The product e2m1 * e4m3 however has at most six significant bits and lies in
// [2^-10, 2688], so it is EXACTLY representable in f16.  The kernel therefore expands the
// operands to f16 on their way into LDS and multiplies with v_mfma_f32_32x32x16_f16:
// every partial product is exact in f32 and the result differs from the definition above
// only by the order of the f32 additions.  HBM sees the packed operands (a quarter of the
// bf16 GEMM's bytes); the matrix pipe runs at its 16-bit rate.  The variants of record ("_q") use
// v_mfma_f32_16x16x32_f16: 1241 against 1141 TFLOP/s at 8192^3 on random operands (see Nvfp4Gemm).
//
// Pipeline: register-staged.  For K tile kt+1 every lane fetches 16 bytes (32 values of
// one row) of x and of y plus the two scale bytes that belong to them; while the MFMAs of
// tile kt run from the current LDS stage, the fetched values are expanded
// (v_cvt_scalef32_pk_f16_fp4: two values per instruction; v_pk_mul_f16 by the block's
// scale) and written to the other stage as four 16-byte units.  Rows are 128 bytes of f16
// with 16-byte unit u stored at unit u ^ ((row >> 1) & 7), so the operand reads of 32 rows
// fall on distinct banks.
//
// A fully dealt-out schedule (fragments read one K step ahead, expansion units and fetches placed
// between individual MFMAs, hand-over before the last K step, fetches two tiles ahead) was built
// and measured equal to this form (1138 vs 1127-1140 TFLOP/s at 8192^3), so the simple form stays.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "gemm_common.h"
#include "kernel_args.h"

using namespace cutile;
using namespace cutile::gemm;

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// 8 packed e2m1 values (one dword, low nibble first) times one f16 scale -> 8 f16 (one LDS unit)
__device__ __forceinline__ u32x4 expand_fp4x8(uint32_t packed, _Float16 scale) {
  const f16x2 s = {scale, scale};
  u32x4 out;
  out.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(packed, 1.0f, 0) * s);
  out.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(packed, 1.0f, 1) * s);
  out.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(packed, 1.0f, 2) * s);
  out.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(packed, 1.0f, 3) * s);
  return out;
}

// SHAPE16: v_mfma_f32_16x16x32_f16 instead of v_mfma_f32_32x32x16_f16 — half as many accumulator values written per
// flop, which is worth a few per cent at the chip's power limit (see gemm_bf16.hip, GemmRing16).  Both operands are
// K-contiguous rows here, so only the fragment addresses (row lane % 16, K group lane / 16 of a 32-wide step) and the
// accumulator layout (a lane: row lane % 16, columns 4 (lane / 16) .. + 3 of each 16 x 16 block) change.
template <int BM, int BN, int WAVES_M, int WAVES_N, typename OutT, bool SHAPE16 = false>
struct Nvfp4Gemm {
  static constexpr int BK = 64;                      // values per K tile: four scale blocks of 16
  static constexpr int kRowBytes = BK * 2;           // a stage row in f16: eight 16-byte units
  static constexpr int kWaves = WAVES_M * WAVES_N;
  static constexpr int kThreads = kWaves * 64;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int BLK = SHAPE16 ? 16 : 32;      // rows / columns of one accumulator block
  static constexpr int TM = WM / BLK, TN = WN / BLK;
  // a piece = 32 values of one row = 16 packed bytes = two scale blocks; two pieces per row and K tile
  static constexpr int kAPieces = BM * 2 / kThreads, kBPieces = BN * 2 / kThreads;
  static constexpr int kABytes = BM * kRowBytes, kBBytes = BN * kRowBytes;
  static constexpr int kStageBytes = kABytes + kBBytes;
  static constexpr int kLdsBytes = 2 * kStageBytes;
  static_assert((BM * 2) % kThreads == 0 && (BN * 2) % kThreads == 0 && WM % 32 == 0 && WN % 32 == 0, "split");

  __device__ static __forceinline__ int lds_off(int r, int u) { return r * kRowBytes + ((u ^ ((r >> 1) & 7)) << 4); }

  __device__ static void run(const PartitionArg<2>& z, const TensorArg<2>& x, const TensorArg<2>& y,
                             const TensorArg<2>& xs, const TensorArg<2>& ys, float alpha, const TileGrid& g) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[kLdsBytes];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int l32 = lane & 31, khalf = lane >> 5;
    const int l16 = lane & 15, grp = lane >> 4;
    uint32_t pm, pn;
    tile_coords(g.x, g.y, &pm, &pn);
    const int32_t M = x.shape[0], N = y.shape[0];
    const int32_t k_bytes = min(x.shape[1], y.shape[1]);           // packed bytes per row
    const int32_t lda = x.strides[0], ldb = y.strides[0];
    const int32_t ldsa = xs.strides[0], ldsb = ys.strides[0];
    const int32_t row0 = pm * BM, col0 = pn * BN;

    const __amdgpu_buffer_rsrc_t ra = make_rsrc(x.ptr, (uint32_t)((int64_t)(M - 1) * lda + x.shape[1]));
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(y.ptr, (uint32_t)((int64_t)(N - 1) * ldb + y.shape[1]));
    const __amdgpu_buffer_rsrc_t rsa = make_rsrc(xs.ptr, (uint32_t)((int64_t)(xs.shape[0] - 1) * ldsa + xs.shape[1]));
    const __amdgpu_buffer_rsrc_t rsb = make_rsrc(ys.ptr, (uint32_t)((int64_t)(ys.shape[0] - 1) * ldsb + ys.shape[1]));
    constexpr uint32_t kOob = 0x80000000u;

    // Rows past the tensor fetch zeros: data 0 and scale 0, so they add nothing.
    int a_row[kAPieces], a_half[kAPieces], b_row[kBPieces], b_half[kBPieces];
    uint32_t a_goff[kAPieces], a_soff[kAPieces], b_goff[kBPieces], b_soff[kBPieces];
#pragma unroll
    for (int i = 0; i < kAPieces; ++i) {
      const int c = tid + i * kThreads;
      a_row[i] = c >> 1;
      a_half[i] = c & 1;
      const int32_t r = row0 + a_row[i];
      a_goff[i] = r < M ? (uint32_t)((int64_t)r * lda + a_half[i] * 16) : kOob;
      a_soff[i] = r < M ? (uint32_t)((int64_t)r * ldsa + a_half[i] * 2) : kOob;
    }
#pragma unroll
    for (int i = 0; i < kBPieces; ++i) {
      const int c = tid + i * kThreads;
      b_row[i] = c >> 1;
      b_half[i] = c & 1;
      const int32_t r = col0 + b_row[i];
      b_goff[i] = r < N ? (uint32_t)((int64_t)r * ldb + b_half[i] * 16) : kOob;
      b_soff[i] = r < N ? (uint32_t)((int64_t)r * ldsb + b_half[i] * 2) : kOob;
    }
    u32x4 a_reg[kAPieces], b_reg[kBPieces];
    uint32_t a_sc[kAPieces], b_sc[kBPieces];      // two e4m3 scale bytes in the low half
    auto load_global = [&](int32_t kt) {          // K tile kt: packed bytes 32 kt .., scale bytes 4 kt ..
#pragma unroll
      for (int i = 0; i < kAPieces; ++i) {
        a_reg[i] = __builtin_amdgcn_raw_buffer_load_b128(ra, a_goff[i], kt * 32, 0);
        a_sc[i] = __builtin_amdgcn_raw_buffer_load_b16(rsa, a_soff[i], kt * 4, 0);
      }
#pragma unroll
      for (int i = 0; i < kBPieces; ++i) {
        b_reg[i] = __builtin_amdgcn_raw_buffer_load_b128(rb, b_goff[i], kt * 32, 0);
        b_sc[i] = __builtin_amdgcn_raw_buffer_load_b16(rsb, b_soff[i], kt * 4, 0);
      }
    };
    // LDS takes a 16-byte write from 8 lanes per cycle (128 bytes): lanes 0-7 are 4 rows x 2 halves, and rows
    // 2j, 2j+1 share their swizzle term, so writing unit d of every row in step d would put both on the same
    // banks.  Odd rows therefore walk their four units in the order 2, 3, 0, 1.
    auto expand_piece = [&](unsigned char* tile, int row, int half, const u32x4& q, uint32_t sc) {
      const bool odd = row & 1;
      const _Float16 s0 = (_Float16)__builtin_amdgcn_cvt_f32_fp8((int)sc, 0);   // e4m3fn -> f32 -> f16: exact
      const _Float16 s1 = (_Float16)__builtin_amdgcn_cvt_f32_fp8((int)sc, 1);
      const _Float16 sa = odd ? s1 : s0, sb = odd ? s0 : s1;
      const uint32_t q0 = odd ? q.z : q.x, q1 = odd ? q.w : q.y, q2 = odd ? q.x : q.z, q3 = odd ? q.y : q.w;
      const int flip = odd ? 2 : 0;
      *reinterpret_cast<u32x4*>(tile + lds_off(row, half * 4 + (0 ^ flip))) = expand_fp4x8(q0, sa);
      *reinterpret_cast<u32x4*>(tile + lds_off(row, half * 4 + (1 ^ flip))) = expand_fp4x8(q1, sa);
      *reinterpret_cast<u32x4*>(tile + lds_off(row, half * 4 + (2 ^ flip))) = expand_fp4x8(q2, sb);
      *reinterpret_cast<u32x4*>(tile + lds_off(row, half * 4 + (3 ^ flip))) = expand_fp4x8(q3, sb);
    };
    auto store_lds = [&](int stage) {
      unsigned char* sa = lds + stage * kStageBytes;
      unsigned char* sb = sa + kABytes;
#pragma unroll
      for (int i = 0; i < kAPieces; ++i) expand_piece(sa, a_row[i], a_half[i], a_reg[i], a_sc[i]);
#pragma unroll
      for (int i = 0; i < kBPieces; ++i) expand_piece(sb, b_row[i], b_half[i], b_reg[i], b_sc[i]);
    };

    typedef float f32x4v __attribute__((ext_vector_type(4)));
    using Acc = std::conditional_t<SHAPE16, f32x4v, f32x16>;
    constexpr int kAccRegs = SHAPE16 ? 4 : 16;
    Acc acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int v = 0; v < kAccRegs; ++v) acc[tn][tm][v] = 0.0f;

    const int k_tiles = k_bytes / 32;
    if (k_tiles > 0) {
      load_global(0);
      store_lds(0);
    }
    __syncthreads();

    constexpr int kSteps = SHAPE16 ? 2 : 4;     // K steps of 32 or 16 values per tile
    for (int kt = 0; kt < k_tiles; ++kt) {
      const int cur = kt & 1;
      if (kt + 1 < k_tiles) load_global(kt + 1);
      const unsigned char* sa = lds + cur * kStageBytes;
      const unsigned char* sb = sa + kABytes;
#pragma unroll
      for (int ks = 0; ks < kSteps; ++ks) {
        f16x8 af[TM], bfr[TN];
        const int frow = SHAPE16 ? l16 : l32, funit = SHAPE16 ? ks * 4 + grp : ks * 2 + khalf;
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) af[tm] = *reinterpret_cast<const f16x8*>(sa + lds_off(wm * WM + tm * BLK + frow, funit));
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) bfr[tn] = *reinterpret_cast<const f16x8*>(sb + lds_off(wn * WN + tn * BLK + frow, funit));
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
          for (int tm = 0; tm < TM; ++tm) {
            if constexpr (SHAPE16)
              acc[tn][tm] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bfr[tn], af[tm], acc[tn][tm], 0, 0, 0);
            else
              acc[tn][tm] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bfr[tn], af[tm], acc[tn][tm], 0, 0, 0);
          }
        // the expansion of the next tile rides between the matrix instructions of the later K steps
        if (ks == (SHAPE16 ? 0 : 1) && kt + 1 < k_tiles) store_lds(cur ^ 1);
      }
      __syncthreads();
    }

    OutT* zp = (OutT*)z.ptr;
    const int32_t ldz = z.strides[0];
    const int32_t zM = z.shape[0], zN = z.shape[1];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      const int32_t r = row0 + wm * WM + tm * BLK + (SHAPE16 ? l16 : l32);
      if (r >= zM) continue;
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int q = 0; q < (SHAPE16 ? 1 : 4); ++q) {
          // the lane's 4 consecutive columns of this block: 8 q + 4 (lane / 32) of 32, or 4 (lane / 16) of 16
          const int32_t c = col0 + wn * WN + tn * BLK + (SHAPE16 ? grp * 4 : q * 8 + khalf * 4);
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

// linear_tile<BM, BN, BK, BK_PACKED, BK_SCALES>(z: [BM,BN] tiles, x, y, x_scales, y_scales, alpha) with trailing launch metadata.
#define NVFP4_KERNEL(NAME, BM, BN, WVM, WVN, OUT_T)                                                \
  extern "C" __global__ void __launch_bounds__(WVM* WVN * 64)                                     \
      linear_tile_nvfp4_entry__##NAME(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y, TensorArg<2> xs, \
                                      TensorArg<2> ys, float alpha, TileGrid g) {                  \
    Nvfp4Gemm<BM, BN, WVM, WVN, OUT_T>::run(z, x, y, xs, ys, alpha, g);                            \
  }

#define NVFP4_KERNEL16(NAME, BM, BN, WVM, WVN, OUT_T)                                              \
  extern "C" __global__ void __launch_bounds__(WVM* WVN * 64)                                     \
      linear_tile_nvfp4_entry__##NAME(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y, TensorArg<2> xs, \
                                      TensorArg<2> ys, float alpha, TileGrid g) {                  \
    Nvfp4Gemm<BM, BN, WVM, WVN, OUT_T, true>::run(z, x, y, xs, ys, alpha, g);                      \
  }
NVFP4_KERNEL16(f32_256x256x64_q4x2, 256, 256, 4, 2, float)
NVFP4_KERNEL16(f32_256x256x64_q2x4, 256, 256, 2, 4, float)
NVFP4_KERNEL16(bf16_256x256x64_q4x2, 256, 256, 4, 2, __bf16)
NVFP4_KERNEL16(bf16_256x256x64_q2x4, 256, 256, 2, 4, __bf16)
NVFP4_KERNEL(f32_256x256x64_w4x2, 256, 256, 4, 2, float)
NVFP4_KERNEL(f32_256x256x64_w2x4, 256, 256, 2, 4, float)
NVFP4_KERNEL(f32_128x128x64_w2x2, 128, 128, 2, 2, float)
NVFP4_KERNEL(f32_64x64x64_w1x1, 64, 64, 1, 1, float)
NVFP4_KERNEL(f32_32x32x64_w1x1, 32, 32, 1, 1, float)
NVFP4_KERNEL(bf16_256x256x64_w2x4, 256, 256, 2, 4, __bf16)
NVFP4_KERNEL(bf16_256x256x64_w4x2, 256, 256, 4, 2, __bf16)
NVFP4_KERNEL(bf16_128x128x64_w2x2, 128, 128, 2, 2, __bf16)
