// The precompiled-kernel table: what stands where the reference has its JIT and
// kernel cache (cutile/src/tile_kernel.rs:96-114,371-399,675-756).  A key that the
// reference would compile on first launch is here resolved to a gfx950 code
// object embedded in the library plus the launch metadata the HIP kernel needs
// (workgroup shape, LDS bytes, the tile shape it implements).
#pragma once
#include <string>
#include <vector>

#include "runtime_state.h"

namespace cutile {

enum Image : int { IMG_ELEMENTWISE = 0, IMG_ROWWISE, IMG_GEMM, IMG_FMHA, IMG_MXGEMM, IMG_NVFP4, IMG_RNG, IMG_COUNT };

struct KernelEntry {
  const char* function;  // entry name in the reference, e.g. "gemm"
  const char* variant;   // name of this implementation inside the family
  const char* symbol;    // symbol in the code object
  Image image;
  uint32_t block[3];
  uint32_t lds_bytes;
  int32_t tile[4];       // (BM, BN, BK, extra); 0 = not tile-specific
  const char* dtype;     // element type the variant is written for, or ""
  int64_t capacity;      // row-wise kernels: longest segment held in registers; 0 = n/a
  int32_t rank;          // elementwise kernels: tensor rank; 0 = n/a
};

const std::vector<KernelEntry>& kernel_table();

// Finds the entry (function, variant); nullptr if absent.
const KernelEntry* find_entry(const char* function, const std::string& variant);
// Resolves the entry's hipFunction_t on `device`, loading its code object on
// first use (single flight per device).
cutile_status_t load_entry(cutile_device_t device, const KernelEntry* entry, hipFunction_t* fn);
// Preferred variant set through cutile_kernel_set_preferred_variant, or "".
std::string preferred_variant(const char* function);
// Winner a tuning record names for (function, shape-class bucket), or "".
std::string preferred_variant_for(const char* function, const std::string& bucket);
void clear_bucket_preferences();
// Loads the tuning records once per process (tuning.cpp); cheap afterwards.
void ensure_tuning_records_loaded();
// Human-readable list of variants of `function`, for error messages.
std::string list_variants(const char* function);

}  // namespace cutile
