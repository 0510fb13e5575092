// Pieces shared by the GEMM kernels for gfx950 (bf16 and MX fp8): vector types,
// buffer descriptors, the workgroup -> tile mapping and the LDS-staged epilogue.
#pragma once
#include <hip/hip_runtime.h>

#include "kernel_args.h"

namespace cutile {
namespace gemm {

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
  typedef __bf16 b2 __attribute__((ext_vector_type(2)));
  typedef float f2 __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f2{lo, hi}, b2));  // v_cvt_pk_bf16_f32, round to nearest even
}

// 16-bit outputs: two f32 rounded to nearest even into one register, and a stored pair widened again.
template <typename OutT>
__device__ __forceinline__ uint32_t pack_out2(float lo, float hi) {
  if constexpr (__is_same(OutT, _Float16)) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f2{lo, hi}, h2));   // v_cvt_pk_f16_f32
  } else {
    return pack_bf16x2(lo, hi);
  }
}
template <typename OutT>
__device__ __forceinline__ float stored_lo(uint32_t bits) {
  if constexpr (__is_same(OutT, _Float16)) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    return (float)__builtin_bit_cast(h2, bits)[0];
  } else {
    return __builtin_bit_cast(float, bits << 16);
  }
}
template <typename OutT>
__device__ __forceinline__ float stored_hi(uint32_t bits) {
  if constexpr (__is_same(OutT, _Float16)) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    return (float)__builtin_bit_cast(h2, bits)[1];
  } else {
    return __builtin_bit_cast(float, bits & 0xffff0000u);
  }
}
// v_mfma_f32_32x32x16 on 16-byte operand fragments of bf16 or f16 (the fragments travel as raw bits).
template <typename InT>
__device__ __forceinline__ f32x16 mfma_32x32x16(bf16x8 a, bf16x8 b, f32x16 c) {
  if constexpr (__is_same(InT, _Float16)) {
    typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
}

// v_mfma_f32_16x16x32 on the same fragments: half as many accumulator values written per flop.
typedef float f32x4_acc __attribute__((ext_vector_type(4)));
template <typename InT>
__device__ __forceinline__ f32x4_acc mfma_16x16x32(bf16x8 a, bf16x8 b, f32x4_acc c) {
  if constexpr (__is_same(InT, _Float16)) {
    typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
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

// The same order for a workgroup that walks several tiles: item `id` of a launch of `stride` workgroups (workgroup b
// takes b, b + stride, ...).  Workgroups are dealt round-robin to the XCDs, so with stride a multiple of 8 all items of
// a workgroup lie on its XCD, which covers one contiguous eighth of the M-grouped order round by round.
__device__ __forceinline__ void tile_of_id(uint32_t id, uint32_t tiles_m, uint32_t tiles_n, uint32_t stride, uint32_t* pm,
                                           uint32_t* pn) {
  const uint32_t total = tiles_m * tiles_n;
  if (total % kNumXcd == 0 && stride % kNumXcd == 0) id = (id % kNumXcd) * (total / kNumXcd) + id / kNumXcd;
  const uint32_t per_group = kGroupM * tiles_n;
  const uint32_t group = id / per_group;
  const uint32_t first_m = group * kGroupM;
  const uint32_t rows = min(tiles_m - first_m, (uint32_t)kGroupM);
  const uint32_t in_group = id % per_group;
  *pm = first_m + in_group % rows;
  *pn = in_group / rows;
}

// Epilogue shared by the pipelined variants: accumulators -> z through LDS.
// In the MFMA layout a lane owns 4 consecutive columns of one row, so a direct
// store touches 32 rows with 8 or 16 bytes each and every 128-byte line of z is
// written in 8 pieces.  Staged through LDS (f32, one 32-row band of the
// wavefront's sub-tile at a time, wavefront-private so no barrier is needed), the
// same data leaves as 16-byte stores with consecutive lanes on consecutive
// columns: whole lines.  `accumulate` adds the old z in f32 before the single
// rounding, as the tile program does (acc = z.load(); ...; z.store(acc)).
// `stage` is this wavefront's private region of kEpilogueBytesPerWave<WN> bytes.
// Rows are WN*4 bytes; 16-byte chunk c of row r sits at chunk c ^ (r & 15), so the 16
// rows of one write pass fall on distinct banks.
template <int WN>
constexpr int kEpilogueBytesPerWave = 32 * WN * 4;

// An output too large to still be cached when its consumer runs is read and stored past the caches
// (nontemporal), which leaves them to the operand panels: measured +1.8 % at 8192^3 (128 MiB of bf16),
// -3 % at 4096^3 (32 MiB, which a following launch finds in the memory-side cache).
constexpr int64_t kStreamedOutputBytes = 64ll << 20;
template <typename V>
__device__ __forceinline__ V load_z(const V* p, bool stream) {
  V v;
  if (stream) {
    asm volatile("");   // as in store_z
    v = __builtin_nontemporal_load(p);
    asm volatile("");
  } else {
    v = *p;
  }
  return v;
}
template <typename V>
__device__ __forceinline__ void store_z(V v, V* p, bool stream) {
  if (stream) {
    asm volatile("");   // empty statements on both sides keep the optimiser from merging the two
    __builtin_nontemporal_store(v, p);   // stores of this branch and the next into one plain store
    asm volatile("");
  } else {
    *p = v;
  }
}

// `write_band(tm)` puts rows [32 tm, 32 tm + 32) of the wavefront's sub-tile into `stage` (f32, row r at r * WN * 4,
// 16-byte chunk c of row r at chunk c ^ (r & 15)); TM = 32-row bands, WN = columns of the sub-tile.
template <int TM, int WN, typename OutT, typename BandWriter>
__device__ __forceinline__ void store_bands_staged(BandWriter write_band, unsigned char* stage, OutT* zp, int32_t ldz,
                                                   int32_t zM, int32_t zN, int32_t wave_row0, int32_t wave_col0,
                                                   int lane, int32_t accumulate) {
  constexpr int PITCH = WN * 4;
  constexpr int COLS_PER_LANE = sizeof(OutT) == 2 ? 8 : 4;      // 16 bytes of output per lane
  constexpr int LANES_PER_ROW = WN / COLS_PER_LANE;
  constexpr int ROWS_PER_PASS = 64 / LANES_PER_ROW;
  constexpr int PASSES = 32 / ROWS_PER_PASS;
  const int rd_row = lane / LANES_PER_ROW, rd_col = (lane % LANES_PER_ROW) * COLS_PER_LANE;
  const int32_t gc = wave_col0 + rd_col;
  const bool col_ok = gc < zN;
  const bool stream = (int64_t)zM * zN * (int64_t)sizeof(OutT) >= kStreamedOutputBytes;
  const bool full = gc + COLS_PER_LANE <= zN;  // zN is a multiple of 4: otherwise exactly the first 4 columns are inside
  // Old z, all of it requested before anything is waited for.
  u32x4 old[TM][PASSES];
  if (accumulate) {
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
      for (int pass = 0; pass < PASSES; ++pass) {
        const int32_t gr = wave_row0 + tm * 32 + pass * ROWS_PER_PASS + rd_row;
        old[tm][pass] = u32x4{0, 0, 0, 0};
        if (gr < zM && col_ok) {
          const OutT* src = zp + (int64_t)gr * ldz + gc;
          if (full) {
            old[tm][pass] = load_z(reinterpret_cast<const u32x4*>(src), stream);
          } else {
            u32x2 h = load_z(reinterpret_cast<const u32x2*>(src), stream);
            old[tm][pass].x = h.x;
            old[tm][pass].y = h.y;
          }
        }
      }
  }
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) {
    // write this band in the MFMA layout
    write_band(tm);
    // read it back row-contiguous and store
#pragma unroll
    for (int pass = 0; pass < PASSES; ++pass) {
      const int r = pass * ROWS_PER_PASS + rd_row;
      const int32_t gr = wave_row0 + tm * 32 + r;
      const unsigned char* src = stage + r * PITCH;
      f32x4 lo = *reinterpret_cast<const f32x4*>(src + (((rd_col >> 2) ^ (r & 15)) << 4));
      const u32x4 o = old[tm][pass];
      if constexpr (sizeof(OutT) == 2) {
        f32x4 hi = *reinterpret_cast<const f32x4*>(src + ((((rd_col >> 2) + 1) ^ (r & 15)) << 4));
        if (accumulate) {
          lo[0] += stored_lo<OutT>(o.x);
          lo[1] += stored_hi<OutT>(o.x);
          lo[2] += stored_lo<OutT>(o.y);
          lo[3] += stored_hi<OutT>(o.y);
          hi[0] += stored_lo<OutT>(o.z);
          hi[1] += stored_hi<OutT>(o.z);
          hi[2] += stored_lo<OutT>(o.w);
          hi[3] += stored_hi<OutT>(o.w);
        }
        if (gr < zM && col_ok) {
          OutT* dst = zp + (int64_t)gr * ldz + gc;
          if (full) {
            u32x4 w = {pack_out2<OutT>(lo[0], lo[1]), pack_out2<OutT>(lo[2], lo[3]), pack_out2<OutT>(hi[0], hi[1]),
                       pack_out2<OutT>(hi[2], hi[3])};
            store_z(w, reinterpret_cast<u32x4*>(dst), stream);
          } else {
            u32x2 w = {pack_out2<OutT>(lo[0], lo[1]), pack_out2<OutT>(lo[2], lo[3])};
            store_z(w, reinterpret_cast<u32x2*>(dst), stream);
          }
        }
      } else {
        if (accumulate) lo += __builtin_bit_cast(f32x4, o);
        if (gr < zM && col_ok) store_z(lo, reinterpret_cast<f32x4*>(zp + (int64_t)gr * ldz + gc), stream);
      }
    }
  }
}

// accumulators of v_mfma_f32_32x32x16: a lane holds row lane % 32 and, per 32-column block, the column quadruples
// 2 q + lane / 32 (q = 0..3)
template <int TM, int TN, typename OutT>
__device__ __forceinline__ void store_tile_staged(f32x16 (&acc)[TN][TM], unsigned char* stage, OutT* zp, int32_t ldz,
                                                  int32_t zM, int32_t zN, int32_t wave_row0, int32_t wave_col0,
                                                  int lane, int32_t accumulate) {
  constexpr int PITCH = TN * 32 * 4;
  const int l32 = lane & 31, khalf = lane >> 5;
  store_bands_staged<TM, TN * 32, OutT>(
      [&](int tm) {
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            f32x4 v = {acc[tn][tm][q * 4 + 0], acc[tn][tm][q * 4 + 1], acc[tn][tm][q * 4 + 2], acc[tn][tm][q * 4 + 3]};
            *reinterpret_cast<f32x4*>(stage + l32 * PITCH + (((tn * 8 + q * 2 + khalf) ^ (l32 & 15)) << 4)) = v;
          }
      },
      stage, zp, ldz, zM, zN, wave_row0, wave_col0, lane, accumulate);
}
// accumulators of v_mfma_f32_16x16x32 (TM, TN count 16 x 16 blocks): a lane holds row lane % 16 and the column
// quadruple lane / 16 of each block; two row blocks make one 32-row band
template <int TM, int TN, typename OutT>
__device__ __forceinline__ void store_tile_staged16(f32x4_acc (&acc)[TN][TM], unsigned char* stage, OutT* zp, int32_t ldz,
                                                    int32_t zM, int32_t zN, int32_t wave_row0, int32_t wave_col0,
                                                    int lane, int32_t accumulate) {
  static_assert(TM % 2 == 0, "two 16-row blocks per band");
  constexpr int PITCH = TN * 16 * 4;
  const int l16 = lane & 15, grp = lane >> 4;
  store_bands_staged<TM / 2, TN * 16, OutT>(
      [&](int band) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int tn = 0; tn < TN; ++tn) {
            const int r = h * 16 + l16;
            const f32x4 v = {acc[tn][band * 2 + h][0], acc[tn][band * 2 + h][1], acc[tn][band * 2 + h][2], acc[tn][band * 2 + h][3]};
            *reinterpret_cast<f32x4*>(stage + r * PITCH + (((tn * 4 + grp) ^ (r & 15)) << 4)) = v;
          }
      },
      stage, zp, ldz, zM, zN, wave_row0, wave_col0, lane, accumulate);
}

}  // namespace gemm
}  // namespace cutile
