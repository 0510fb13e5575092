// Kernel-argument records shared by device code and the host launcher.
//
// A tensor argument is marshalled exactly as the reference's launcher pushes it
// (cutile/src/tensor.rs:2005-2016): device pointer, then shape[rank] and
// strides[rank] as i32 (strides in elements).  An output partition appends
// partition_shape[rank] and partition_strides[rank] (cutile/src/tensor.rs:1723-1739).
// Passing the record by value gives the same kernarg bytes as pushing the scalars
// one by one, because every record is a multiple of 8 bytes.
//
// The reference launches one CUDA block per tile and lets its assembler pick the
// thread count.  Here every kernel fixes its own workgroup shape, and the host
// launcher translates the tile grid into a HIP grid; the tile grid itself is
// handed to the kernel as a trailing TileGrid argument so that kernels which
// cover several tiles per workgroup (or remap workgroups for L2 locality) still
// honour partial-coverage launches.
#pragma once
#include <stdint.h>

namespace cutile {

template <int R>
struct TensorArg {
  void* ptr;
  int32_t shape[R];
  int32_t strides[R];
};

template <int R>
struct PartitionArg {
  void* ptr;
  int32_t shape[R];
  int32_t strides[R];
  int32_t pshape[R];
  int32_t pstrides[R];
};

struct TileGrid {
  uint32_t x, y, z, pad;
};

static_assert(sizeof(TensorArg<1>) == 16 && sizeof(TensorArg<2>) == 24 && sizeof(TensorArg<3>) == 32 &&
                  sizeof(TensorArg<4>) == 40,
              "tensor records must stay a flat (ptr, i32...) sequence");
static_assert(sizeof(PartitionArg<1>) == 24 && sizeof(PartitionArg<2>) == 40 && sizeof(PartitionArg<3>) == 56,
              "partition records must stay a flat (ptr, i32...) sequence");

}  // namespace cutile
