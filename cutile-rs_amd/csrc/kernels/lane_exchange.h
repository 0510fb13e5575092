// Cross-lane exchanges that stay inside the vector ALU (gfx950).
//
// A lane-indexed permute (ds_bpermute, what __shfl_xor compiles to) travels through the LDS crossbar and back: about a
// hundred cycles, with a wait of its own, per step.  Reductions over a wavefront need none of that:
//  * inside a row of 16 lanes, DPP operand modifiers pair lanes for free: quad neighbours (lane ^ 1, lane ^ 2), then
//    the mirrored halves of 8 and of 16 lanes.  After the quad steps every lane of a quad holds the same value, so
//    the mirror steps pair groups that already agree and the result is the full sum / maximum in every lane;
//  * across rows, v_permlane16_swap exchanges the odd rows of its first operand with the even rows of its second,
//    and v_permlane32_swap the upper 32 lanes of the first with the lower 32 of the second.  Given two copies of v they
//    leave (row 0, row 0, row 2, row 2) / (row 1, row 1, row 3, row 3), respectively the lower half's and the upper
//    half's values in every lane; a commutative combine of the two registers is the exchange-and-combine step.
//    Both instructions need two idle issue cycles after a vector write of their operands (the s_nop in front).
#pragma once
#include <hip/hip_runtime.h>

namespace cutile {
namespace lanes {

template <int CTRL>
__device__ __forceinline__ float dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
template <int CTRL>
__device__ __forceinline__ int32_t dpp(int32_t v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, false);
}
constexpr int kQuadXor1 = 0xB1;       // quad_perm [1,0,3,2]
constexpr int kQuadXor2 = 0x4E;       // quad_perm [2,3,0,1]
constexpr int kHalfMirror = 0x141;    // row_half_mirror: lane i of 8 <-> 7 - i
constexpr int kRowMirror = 0x140;     // row_mirror: lane i of 16 <-> 15 - i

// Two copies of v -> (even rows' values in every lane, odd rows' values in every lane), rows of 16 lanes.
template <typename T>
__device__ __forceinline__ void split_row_pairs(T v, T* even, T* odd) {
  static_assert(sizeof(T) == 4, "32-bit values");
  T a = v, b = v;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 0" : "+v"(a), "+v"(b));
  *even = a;
  *odd = b;
}
// Two copies of v -> (lower 32 lanes' values in every lane, upper 32 lanes' values in every lane).
template <typename T>
__device__ __forceinline__ void split_halves(T v, T* lower, T* upper) {
  static_assert(sizeof(T) == 4, "32-bit values");
  T a = v, b = v;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 0" : "+v"(a), "+v"(b));
  *lower = a;
  *upper = b;
}

struct Sum {
  __device__ static __forceinline__ float of(float a, float b) { return a + b; }
};
struct Max {
  __device__ static __forceinline__ float of(float a, float b) { return fmaxf(a, b); }
};

// Combine over the lanes l, l ^ 32.
template <class Op>
__device__ __forceinline__ float across_halves(float v) {
  float lo, hi;
  split_halves(v, &lo, &hi);
  return Op::of(lo, hi);
}
// Combine over the lanes l, l ^ 16, l ^ 32, l ^ 48.
template <class Op>
__device__ __forceinline__ float across_rows(float v) {
  float e, o;
  split_row_pairs(v, &e, &o);
  return across_halves<Op>(Op::of(e, o));
}
// Combine over groups of LANES consecutive lanes (a power of two up to 64), the result in every lane of the group.
template <class Op, int LANES>
__device__ __forceinline__ float across_group(float v) {
  static_assert(LANES >= 1 && LANES <= 64 && (LANES & (LANES - 1)) == 0, "group width");
  if constexpr (LANES >= 2) v = Op::of(v, dpp<kQuadXor1>(v));
  if constexpr (LANES >= 4) v = Op::of(v, dpp<kQuadXor2>(v));
  if constexpr (LANES >= 8) v = Op::of(v, dpp<kHalfMirror>(v));
  if constexpr (LANES >= 16) v = Op::of(v, dpp<kRowMirror>(v));
  if constexpr (LANES >= 32) {
    float e, o;
    split_row_pairs(v, &e, &o);
    v = Op::of(e, o);
  }
  if constexpr (LANES >= 64) v = across_halves<Op>(v);
  return v;
}
template <class Op>
__device__ __forceinline__ float across_wave(float v) {
  return across_group<Op, 64>(v);
}

}  // namespace lanes
}  // namespace cutile
