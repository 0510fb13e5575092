/*
 * cutile_hip_testing.h — test doubles for the host side of the library.
 *
 * The reference tests its host logic without a GPU by substituting fakes for the
 * device (FakeAlloc in cutile/src/tensor.rs:2146-2159, MockFlags in
 * cuda-async/src/slot_table.rs:182-190, meta tensors in cutile/src/api.rs:450-462).
 * This header is the same idea one level lower: a recording stand-in for the HIP
 * runtime.  It executes NO kernels and computes nothing: launches are recorded
 * (symbol, grid, workgroup, kernel-argument bytes) so that validation, variant
 * selection, grid translation and argument marshalling can be asserted on a
 * machine without a GPU.  "Device" memory is host memory, copies are memcpy,
 * streams complete immediately, host callbacks run inline.
 *
 * These entry points are exported by libcutile_hip_testing.so only (the product
 * library's objects plus the stand-in); libcutile_hip.so, the library that ships,
 * exports none of them.  Never enabled implicitly.
 */
#ifndef CUTILE_HIP_TESTING_H
#define CUTILE_HIP_TESTING_H

#include "cutile_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Routes every runtime call of this library to the recording fake exposing
 * `n_devices` devices.  Drops cached device state. */
cutile_status_t cutile_testing_use_fake_hip(int32_t n_devices);
/* Restores the real runtime (bound on next use).  Drops cached device state. */
cutile_status_t cutile_testing_use_real_hip(void);

typedef struct {
  const char* symbol;          /* kernel symbol the function handle was resolved from */
  uint32_t grid[3];
  uint32_t block[3];
  uint32_t shared_mem_bytes;
  void* stream;
  const unsigned char* args;   /* copy of the kernel-argument buffer */
  size_t args_size;
  int32_t in_capture;          /* recorded while the stream was capturing */
  int32_t from_graph_replay;   /* emitted by a graph launch */
} cutile_testing_launch_record_t;

int32_t cutile_testing_launch_count(void);
cutile_status_t cutile_testing_get_launch(int32_t index, cutile_testing_launch_record_t* record);
void cutile_testing_clear_log(void);
/* Makes the next `count` calls of the named runtime entry point (e.g.
 * "hipModuleLaunchKernel", "hipStreamEndCapture") fail with `hip_error`. */
cutile_status_t cutile_testing_inject_failure(const char* hip_function, int32_t hip_error, int32_t count);
/* Counters of the fake: streams created, modules loaded, bytes currently allocated. */
uint64_t cutile_testing_streams_created(void);
uint64_t cutile_testing_bytes_allocated(void);

#ifdef __cplusplus
}
#endif
#endif /* CUTILE_HIP_TESTING_H */
