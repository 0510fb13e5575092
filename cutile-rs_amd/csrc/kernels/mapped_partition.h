// Mapped partitions: the schedule that turns a stream item into a tile index.
//
// The reference separates the logical tile grid of an output partition from the
// physical launch grid: `partition.map(map_shape, num_tile_blocks)` launches
// `num_tile_blocks` tile blocks, and tile block b walks the stream items
// b, b + num_tile_blocks, ... (cutile/src/tensor.rs:314-401; loop lowering in
// cutile-compiler/src/compiler/compile_expression.rs: lower = pid.0, step = grid.0,
// upper = product of the streamed axes).  An item is decomposed into one block id per
// streamed axis by emit_mapped_partition_schedule / emit_swizzle_2d
// (cutile-compiler/src/compiler/compile_intrinsic.rs:2438-2900):
//   * leading axes (all but the last two) row-major, their map dims must be 1;
//   * the trailing two axes (m, n) by the map dims (GM, GN):
//       (1, 1)   row-major;
//       (GM, 1)  bands of GM tile rows, column by column inside a band (the last band
//                may be shorter: `min(num_m - first_m, GM)`);
//       (GM, GN) the same bands cut into groups of GN columns, each group walked
//                column by column.
//   * an axis whose map dim is OWNED (0) is not streamed: its coordinate is 0 and the
//     kernel walks that axis itself.
// This header is shared by the device kernels and the host library (which exposes the
// same function so a caller can inspect the order).
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define CUTILE_SCHED_FN __host__ __device__ inline
#else
#define CUTILE_SCHED_FN inline
#endif

namespace cutile {

constexpr int32_t kOwnedAxis = 0;

// The record a mapped kernel receives after its partition argument.
struct MappedArg {
  int32_t map[3];      // map dims of the partition's axes (unused axes 1)
  int32_t rank;        // rank of the map = rank of the logical grid
  uint32_t grid[3];    // logical tile grid of the partition (unused axes 1)
  uint32_t total;      // number of stream items = product of the streamed axes
};
static_assert(sizeof(MappedArg) == 32, "mapped records must stay a flat i32 sequence");

// A sub-range of the logical grid (`iter_indices_within`, cutile/src/_core.rs:912-930; lowering in
// cutile-compiler/src/compiler/compile_expression.rs:1403-1420): the schedule runs over the per-axis lengths
// (MappedArg::grid holds them) and the axis starts are added to the block ids it yields.
struct MappedRangeArg {
  int32_t start[3];        // first tile per axis
  uint32_t full_grid[3];   // the partition's whole logical grid
};

CUTILE_SCHED_FN void swizzle_2d(uint32_t t, uint32_t num_m, uint32_t num_n, uint32_t gm, uint32_t gn, uint32_t* bid_m,
                                uint32_t* bid_n) {
  if (gm == 1 && gn == 1) {
    *bid_m = t / num_n;
    *bid_n = t % num_n;
    return;
  }
  const uint32_t in_band_cap = gm * num_n;
  const uint32_t band = t / in_band_cap;
  const uint32_t first_m = band * gm;
  const uint32_t rows = num_m - first_m < gm ? num_m - first_m : gm;
  const uint32_t in_band = t - band * in_band_cap;
  if (gn == 1) {
    *bid_m = first_m + in_band % rows;
    *bid_n = in_band / rows;
    return;
  }
  const uint32_t group_cap = rows * gn;
  const uint32_t first_n = (in_band / group_cap) * gn;
  const uint32_t in_group = in_band % group_cap;
  *bid_m = first_m + in_group % rows;
  *bid_n = first_n + in_group / rows;
}

// Block ids (one per axis of the partition, owned axes 0) of stream item t.
CUTILE_SCHED_FN void mapped_index(const MappedArg& m, uint32_t t, uint32_t bid[3]) {
  uint32_t lens[3], maps[3];
  int axes[3], n = 0;
  for (int a = 0; a < m.rank; ++a) {
    bid[a] = 0;
    if (m.map[a] != kOwnedAxis) {
      lens[n] = m.grid[a];
      maps[n] = (uint32_t)m.map[a];
      axes[n++] = a;
    }
  }
  for (int a = m.rank; a < 3; ++a) bid[a] = 0;
  if (n == 1) {
    bid[axes[0]] = t;
  } else if (n == 2) {
    swizzle_2d(t, lens[0], lens[1], maps[0], maps[1], &bid[axes[0]], &bid[axes[1]]);
  } else if (n == 3) {
    const uint32_t inner = lens[1] * lens[2];
    bid[axes[0]] = t / inner;
    swizzle_2d(t % inner, lens[1], lens[2], maps[1], maps[2], &bid[axes[1]], &bid[axes[2]]);
  }
}

}  // namespace cutile
