// Size of the device-resident scratch array (scratch.hip) and the one function the
// side library libcutile_hip_scratch.so exports.
#pragma once
#include <stddef.h>

// 8 MiB per GPU, held from the first call on that GPU until the process ends.
#define CUTILE_SCRATCH_BYTES (8u << 20)

#define CUTILE_SCRATCH_LIBRARY "libcutile_hip_scratch.so"
#define CUTILE_SCRATCH_LOOKUP_SYMBOL "cutile_scratch_lookup"

#ifdef __cplusplus
extern "C"
#endif
int cutile_scratch_lookup(void** device_ptr, size_t* bytes, int* device_ordinal);
