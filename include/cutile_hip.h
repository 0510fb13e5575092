/*
 * cutile_hip.h — C ABI of the MI355X (gfx950) tile-kernel path.
 *
 * This is the drop-in boundary: the entry points a Rust FFI crate binds in place
 * of the reference's cuda-bindings / cuda-core / cuda-async crates and of its
 * Tile-IR JIT.  Plain pointers, integers and POD records only.
 *
 *   Part A  driver layer      replaces cuda-bindings + cuda-core
 *   Part B  kernel table      replaces the JIT: (module, function, generics) ->
 *                             precompiled gfx950 code object + launch metadata
 *   Part C  launch builder    replaces cuda-async AsyncKernelLaunch
 *   Part D  entry launchers   one per #[cutile::entry] kernel on the path; they
 *                             do what the macro-generated launcher's execute()
 *                             does: infer generics, validate, infer the grid,
 *                             pick the kernel, push arguments, launch
 *   Part E  async runtime     replaces cuda-async: stream pools, completion
 *                             reactor, graph capture / replay
 *
 * Conventions.  Every function returns cutile_status_t: 0 = success, > 0 = the
 * hipError_t the HIP runtime returned (the reference's DriverError(code),
 * cuda-core/src/error.rs:17,61-93), < 0 = an error raised by this library before
 * any GPU work (the reference's Launch / KernelLaunch / Tensor errors,
 * cutile/src/error.rs:43-56).  cutile_last_error_message() returns the calling
 * thread's message for the most recent non-zero status; the wording of
 * validation errors follows the reference where its tests assert on it.
 * Handles are opaque pointers owned by the library unless stated otherwise.
 * Nothing here falls back to a CPU implementation: without a HIP runtime and a
 * gfx950 device every compute entry point fails with CUTILE_ERR_LIBRARY_INIT or
 * the driver's error.
 */
#ifndef CUTILE_HIP_H
#define CUTILE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef int32_t cutile_status_t;

enum {
  CUTILE_SUCCESS = 0,
  /* libamdhip64 could not be loaded or a symbol is missing — the reference's
   * "shared object init failed" (cuda-bindings/src/dyn_load.rs:19-51). */
  CUTILE_ERR_LIBRARY_INIT = -1,
  CUTILE_ERR_INVALID_ARGUMENT = -2,
  /* no precompiled variant for the requested (function, generics) key */
  CUTILE_ERR_KERNEL_NOT_FOUND = -3,
  /* launch validation failed (shape / partition / grid / precondition) */
  CUTILE_ERR_KERNEL_LAUNCH = -4,
  /* tensor / partition construction error */
  CUTILE_ERR_TENSOR = -5,
  /* nested execution, capture misuse and other runtime-state errors */
  CUTILE_ERR_STATE = -6,
  CUTILE_ERR_OUT_OF_SLOTS = -7
};

const char* cutile_last_error_message(void);
const char* cutile_status_name(cutile_status_t status);
const char* cutile_version(void);

/* ======================================================================== */
/* Part A — driver layer                                                     */
/* ======================================================================== */
typedef struct cutile_device* cutile_device_t;   /* cuda-core/src/runtime.rs:82-88 Device */
typedef void* cutile_stream_t;                    /* a hipStream_t; runtime.rs:489-494 Stream */
typedef void* cutile_event_t;                     /* a hipEvent_t; runtime.rs:534-537 Event */
typedef struct cutile_module* cutile_module_t;    /* runtime.rs:782-786 Module */
typedef void* cutile_function_t;                  /* a hipFunction_t; runtime.rs:839-843 Function */
typedef void* cutile_mempool_t;                   /* a hipMemPool_t; runtime.rs:374-465 MemPool */
typedef void* cutile_graph_t;                     /* hipGraph_t */
typedef void* cutile_graph_exec_t;                /* hipGraphExec_t */

/* Loads libamdhip64 (reusing a copy already mapped into the process) and calls
 * hipInit.  Idempotent; every other entry point calls it lazily.
 * cuda-bindings/src/dyn_load.rs:121-143. */
cutile_status_t cutile_init(void);
/* Device::device_count — runtime.rs:196 */
cutile_status_t cutile_device_count(int32_t* count);
/* Device::new(ordinal): process-global handle per ordinal — runtime.rs:126-139 */
cutile_status_t cutile_device_get(int32_t ordinal, cutile_device_t* device);
/* Device::name — runtime.rs:214 */
cutile_status_t cutile_device_name(cutile_device_t device, char* buf, size_t buf_len);
/* gcnArchName of the device, e.g. "gfx950:sramecc+:xnack-" */
cutile_status_t cutile_device_arch(cutile_device_t device, char* buf, size_t buf_len);
/* Device::bind_to_thread — runtime.rs:229 */
cutile_status_t cutile_device_bind_to_thread(cutile_device_t device);
/* Device::synchronize — runtime.rs:244 */
cutile_status_t cutile_device_synchronize(cutile_device_t device);
/* Device::l2_cache_size_bytes — runtime.rs:597 */
cutile_status_t cutile_device_l2_cache_size(cutile_device_t device, size_t* bytes);
typedef struct {
  int32_t compute_units;
  int32_t clock_khz;
  int32_t memory_clock_khz;
  int32_t memory_bus_bits;
  int32_t l2_bytes;
  int32_t lds_bytes_per_block;
  int32_t wavefront_size;
  int32_t reserved;
  uint64_t total_memory_bytes;
} cutile_device_props_t;
cutile_status_t cutile_device_props(cutile_device_t device, cutile_device_props_t* props);

/* Device::new_stream: non-blocking stream, taken from a per-device pool and
 * never destroyed (runtime.rs:249-266,504-509,613-631).  cutile_stream_release
 * returns it to the pool. */
cutile_status_t cutile_stream_create(cutile_device_t device, cutile_stream_t* stream);
cutile_status_t cutile_stream_release(cutile_device_t device, cutile_stream_t stream);
/* Stream::synchronize / query — runtime.rs:696,706.  *done = 1 when idle. */
cutile_status_t cutile_stream_synchronize(cutile_stream_t stream);
cutile_status_t cutile_stream_query(cutile_stream_t stream, int32_t* done);
/* Stream::launch_host_function — runtime.rs:715-758 */
typedef void (*cutile_host_fn_t)(void* user);
cutile_status_t cutile_stream_launch_host_func(cutile_stream_t stream, cutile_host_fn_t fn, void* user);
/* Stream::begin_capture (relaxed mode) / end_capture — runtime.rs:760-780 */
cutile_status_t cutile_stream_begin_capture(cutile_stream_t stream);
cutile_status_t cutile_stream_end_capture(cutile_stream_t stream, cutile_graph_t* graph);
/* reactor flag write: cuStreamWriteValue32 — cuda-async/src/reactor.rs:154-179 */
cutile_status_t cutile_stream_write_value32(cutile_stream_t stream, void* device_ptr, uint32_t value);

/* Event — runtime.rs:534-594 */
cutile_status_t cutile_event_create(cutile_event_t* event);
cutile_status_t cutile_event_record(cutile_event_t event, cutile_stream_t stream);
cutile_status_t cutile_event_synchronize(cutile_event_t event);
cutile_status_t cutile_event_elapsed_ms(cutile_event_t start, cutile_event_t end, float* ms);
cutile_status_t cutile_event_destroy(cutile_event_t event);

/* Device::load_module_from_bytes: checks the ELF magic first — runtime.rs:309-328 */
cutile_status_t cutile_module_load_data(cutile_device_t device, const void* image, size_t size,
                                        cutile_module_t* module);
cutile_status_t cutile_module_unload(cutile_module_t module);
/* Module::load_function — runtime.rs:828-835 */
cutile_status_t cutile_module_get_function(cutile_module_t module, const char* name,
                                           cutile_function_t* function);
/* launch_kernel: cuLaunchKernel with a void** parameter array — cuda-core/src/api.rs:48-70 */
cutile_status_t cutile_launch_kernel(cutile_function_t function, const uint32_t grid[3],
                                     const uint32_t block[3], uint32_t shared_mem_bytes,
                                     cutile_stream_t stream, void** kernel_params);

/* malloc_async / malloc_from_pool_async / free_async — cuda-core/src/api.rs:76-119 */
cutile_status_t cutile_malloc_async(size_t bytes, cutile_stream_t stream, void** device_ptr);
cutile_status_t cutile_malloc_from_pool_async(size_t bytes, cutile_mempool_t pool,
                                              cutile_stream_t stream, void** device_ptr);
cutile_status_t cutile_free_async(void* device_ptr, cutile_stream_t stream);
/* memset_d8_async / memcpy_{htod,dtoh,dtod}_async — cuda-core/src/api.rs:102-166 */
cutile_status_t cutile_memset_d8_async(void* device_ptr, uint8_t value, size_t bytes, cutile_stream_t stream);
cutile_status_t cutile_memcpy_htod_async(void* dst, const void* src, size_t bytes, cutile_stream_t stream);
cutile_status_t cutile_memcpy_dtoh_async(void* dst, const void* src, size_t bytes, cutile_stream_t stream);
cutile_status_t cutile_memcpy_dtod_async(void* dst, const void* src, size_t bytes, cutile_stream_t stream);
/* pinned, mapped host memory for the reactor's completion flags —
 * cuda-async/src/slot_table.rs (cuMemHostAlloc portable|devicemap) */
cutile_status_t cutile_host_alloc_mapped(size_t bytes, void** host_ptr, void** device_ptr);
cutile_status_t cutile_host_free(void* host_ptr);

/* MemPool — runtime.rs:335-465 */
cutile_status_t cutile_mempool_create(cutile_device_t device, cutile_mempool_t* pool);
cutile_status_t cutile_mempool_default(cutile_device_t device, cutile_mempool_t* pool);
cutile_status_t cutile_mempool_destroy(cutile_mempool_t pool);
cutile_status_t cutile_mempool_set_release_threshold(cutile_mempool_t pool, uint64_t bytes);
typedef struct {
  uint64_t reserved_current, reserved_high, used_current, used_high;
} cutile_pool_mem_stats_t;
cutile_status_t cutile_mempool_stats(cutile_mempool_t pool, cutile_pool_mem_stats_t* stats);
cutile_status_t cutile_mempool_reset_used_high(cutile_mempool_t pool);
cutile_status_t cutile_mempool_reset_reserved_high(cutile_mempool_t pool);

/* graph instantiate / upload / launch / destroy — cuda-async/src/cuda_graph.rs:61-137,179-244 */
cutile_status_t cutile_graph_instantiate(cutile_graph_t graph, cutile_graph_exec_t* exec);
cutile_status_t cutile_graph_upload(cutile_graph_exec_t exec, cutile_stream_t stream);
cutile_status_t cutile_graph_launch(cutile_graph_exec_t exec, cutile_stream_t stream);
cutile_status_t cutile_graph_exec_destroy(cutile_graph_exec_t exec);
cutile_status_t cutile_graph_destroy(cutile_graph_t graph);

/* RNG: create / seed / normal(f32, f64) / uniform(f32, f64) / destroy — cuda-core/src/api.rs:214-293 (the reference
 * binds cuRAND's default generator).  Here the generator is Philox4x32-10, counter based, evaluated by a fill kernel of
 * this library: element e of a stream depends only on (seed, position), so a fill is reproducible whatever the launch
 * shape, and consecutive fills continue the stream (each fill advances the position by the Philox blocks it used:
 * 4 f32 or 2 f64 values per block).  The value stream is this library's own, not cuRAND's.  uniform: [0, 1);
 * normal: Box-Muller.  Fills are enqueued on `stream` (the reference's generator runs on its own stream setting);
 * a generator is not thread safe (one fill at a time), like a curandGenerator_t. */
typedef struct cutile_rng* cutile_rng_t;
cutile_status_t cutile_rng_create(cutile_rng_t* rng);
cutile_status_t cutile_rng_set_seed(cutile_rng_t rng, uint64_t seed);      /* also rewinds the stream position to 0 */
cutile_status_t cutile_rng_set_offset(cutile_rng_t rng, uint64_t offset);  /* stream position in Philox blocks */
cutile_status_t cutile_rng_get_offset(cutile_rng_t rng, uint64_t* offset);
cutile_status_t cutile_rng_normal_f32(cutile_rng_t rng, void* device_ptr, size_t num_elements, float mean, float std,
                                      cutile_stream_t stream);
cutile_status_t cutile_rng_normal_f64(cutile_rng_t rng, void* device_ptr, size_t num_elements, double mean, double std,
                                      cutile_stream_t stream);
cutile_status_t cutile_rng_uniform_f32(cutile_rng_t rng, void* device_ptr, size_t num_elements, cutile_stream_t stream);
cutile_status_t cutile_rng_uniform_f64(cutile_rng_t rng, void* device_ptr, size_t num_elements, cutile_stream_t stream);
cutile_status_t cutile_rng_destroy(cutile_rng_t rng);

/* ======================================================================== */
/* Part B — kernel table                                                     */
/* ======================================================================== */
/* What the reference obtains from compile_from_context (cutile/src/tile_kernel.rs:675-756):
 * a loaded function plus what is needed to launch and validate it.  Here the
 * function comes from a precompiled gfx950 code object embedded in this library. */
typedef struct {
  cutile_function_t function;   /* loaded on the device passed to the lookup */
  const char* symbol;           /* "<fn>_entry__<variant>" */
  const char* variant;          /* variant name inside the function family */
  uint32_t block[3];            /* workgroup shape the kernel was written for */
  uint32_t lds_bytes;           /* LDS the kernel uses; it is static (carried by the code object), launches pass 0 */
  int32_t tile[4];              /* tile shape (BM, BN, BK, -) the variant implements; 0 = any */
} cutile_kernel_info_t;

/* Looks up `function` (e.g. "gemm") with reference-style generics strings
 * (e.g. {"bf16","256","256","64"}) and a variant hint (NULL = the library's
 * choice for this key).  Unknown keys fail with CUTILE_ERR_KERNEL_NOT_FOUND and a
 * message listing the variants that exist.  Loads the code object on first use
 * (single-flight per device), like the reference's kernel cache
 * (tile_kernel.rs:371-399,705-733). */
cutile_status_t cutile_kernel_lookup(cutile_device_t device, const char* function,
                                     const char* const* generics, int32_t n_generics,
                                     const char* variant, cutile_kernel_info_t* info);
/* Number of code-object loads performed so far (the analogue of
 * jit_compile_count, tile_kernel.rs:45-62). */
uint64_t cutile_module_load_count(void);
/* Enumerates the table: returns the number of entries; writes up to `cap`
 * "function<generics>:variant" C strings (owned by the library). */
int32_t cutile_kernel_list(const char** names, int32_t cap);
/* Pins the variant that cutile_launch_* entry points use for `function` when
 * several fit (the autotuner's output).  variant == NULL restores the default. */
cutile_status_t cutile_kernel_set_preferred_variant(const char* function, const char* variant);

/* The same per shape class: `bucket` names the class a launcher derives from its arguments (what
 * cutile_last_resolved_bucket reports after a launch, e.g. "bf16_256x256|tiles>256" for gemm).  This is how the winners of
 * verified tuning records reach the launchers; order of precedence at a launch: the caller's variant, the function-wide
 * pin (an explicit run-time choice beats a file on disk), the bucket's winner, the table's order. */
cutile_status_t cutile_kernel_set_preferred_variant_for(const char* function, const char* bucket, const char* variant);
/* Tuning records (cutile/src/tune.rs:762-1016): JSON records of autotuner winners, one file per kernel, in the directory
 * `tuned` beside the library (or $CUTILE_TUNING_RECORDS; empty = none), loaded on the first launcher call.  A record is
 * applied only if Record::load_verified accepts it against the running library (schema, kernel, architecture,
 * code-object fingerprint, every winner's variant fingerprint, same device toolchain); anything else is refused as a
 * whole and said so in the report.  cutile_tuning_reload(dir) drops what was applied and loads `dir` (NULL = default). */
cutile_status_t cutile_tuning_reload(const char* directory);
const char* cutile_tuning_report(void);           /* one line per file: applied / refused / warning; valid until the thread's next call */
int32_t cutile_tuning_applied_count(void);        /* buckets with a winner from a record */
/* Where the calling thread's last launcher call took its variant from: "caller", "record:<bucket>", "pinned" or "table";
 * and the shape class that call was filed under ("" for launchers without classes). */
const char* cutile_last_resolved_source(void);
const char* cutile_last_resolved_bucket(void);

/* Provenance of the running library, for records of tuning winners (cutile/src/tune.rs:762-832 keeps
 * source_hash, toolchain fingerprint, arch and crate version; here they come from the kernel table):
 * the library version, the device compiler's version text captured at build time, the one target
 * architecture, and a 16-hex-digit fingerprint of the code object that holds `function` (variant == NULL)
 * or of that code object plus one variant's symbol. */
const char* cutile_library_version(void);
const char* cutile_toolchain_fingerprint(void);
const char* cutile_target_arch(void);
cutile_status_t cutile_kernel_fingerprint(const char* function, const char* variant, char out[17]);

/* ======================================================================== */
/* Part C — launch builder                                                   */
/* ======================================================================== */
/* AsyncKernelLaunch — cuda-async/src/launch.rs:23-146.  Arguments are pushed in
 * kernel-signature order; the builder owns copies of the values. */
typedef struct cutile_launch* cutile_launch_t;
cutile_status_t cutile_launch_create(cutile_function_t function, cutile_launch_t* launch);
cutile_status_t cutile_launch_destroy(cutile_launch_t launch);
/* launch.rs:131-138 push_arg: any POD scalar, by value */
cutile_status_t cutile_launch_push_arg(cutile_launch_t launch, const void* value, size_t size, size_t align);
/* launch.rs:117-124 push_device_ptr */
cutile_status_t cutile_launch_push_device_ptr(cutile_launch_t launch, void* device_ptr);
/* launch.rs:63-74 LaunchConfig */
cutile_status_t cutile_launch_set_config(cutile_launch_t launch, const uint32_t grid[3],
                                         const uint32_t block[3], uint32_t shared_mem_bytes);
/* launch.rs:95-113 launch on a stream; may be called repeatedly */
cutile_status_t cutile_launch_execute(cutile_launch_t launch, cutile_stream_t stream);

/* ======================================================================== */
/* Part D — entry launchers                                                  */
/* ======================================================================== */
#define CUTILE_MAX_RANK 4

/* dtype names are the strings the reference passes in .generics
 * (cuda-core/src/dtype.rs:189-229). */
typedef enum {
  CUTILE_DTYPE_F32 = 0, CUTILE_DTYPE_F64, CUTILE_DTYPE_F16, CUTILE_DTYPE_BF16,
  CUTILE_DTYPE_I8, CUTILE_DTYPE_I16, CUTILE_DTYPE_I32, CUTILE_DTYPE_I64,
  CUTILE_DTYPE_U8, CUTILE_DTYPE_U16, CUTILE_DTYPE_U32, CUTILE_DTYPE_U64,
  CUTILE_DTYPE_BOOL, CUTILE_DTYPE_F8E4M3FN, CUTILE_DTYPE_F8E5M2, CUTILE_DTYPE_F8E8M0FNU,
  CUTILE_DTYPE_F4E2M1FNX2,          /* one byte = two e2m1 values, low nibble first (cuda-core/src/dtype.rs:60-99) */
  CUTILE_DTYPE_COUNT
} cutile_dtype_t;
const char* cutile_dtype_name(cutile_dtype_t dtype);
size_t cutile_dtype_size(cutile_dtype_t dtype);
/* returns CUTILE_DTYPE_COUNT for an unknown name */
cutile_dtype_t cutile_dtype_from_name(const char* name);

/* A tensor argument: what KernelInput pushes (cutile/src/tensor.rs:2005-2016). */
typedef struct {
  void* ptr;                        /* device pointer (already offset for views) */
  cutile_dtype_t dtype;
  int32_t rank;
  int32_t shape[CUTILE_MAX_RANK];
  int32_t strides[CUTILE_MAX_RANK]; /* in elements */
} cutile_tensor_arg_t;

/* An output partition: what KernelOutput pushes (cutile/src/tensor.rs:1723-1739),
 * plus its coverage mode (GridBound::Exact / AtMost, tensor.rs:1677-1685). */
typedef struct {
  cutile_tensor_arg_t tensor;
  int32_t partition_shape[CUTILE_MAX_RANK];
  int32_t partition_strides[CUTILE_MAX_RANK];
  int32_t prefix_coverage;          /* 0 = exact cover, 1 = partition_prefix (at most) */
} cutile_partition_arg_t;

/* Builder options of the generated launcher (cutile-macro/src/_module.rs:901-923):
 * .grid(), .generics(), plus the variant hint this build adds. */
typedef struct {
  uint32_t grid[3];                 /* (0,0,0) = infer from the partition */
  const char* const* generics;      /* NULL = infer from argument dtypes / partition shapes */
  int32_t n_generics;
  const char* variant;              /* NULL = library's choice */
} cutile_launch_opts_t;

/* Launch modes of the generated launcher — cutile-macro/src/_module.rs:852-900.  `.compile()` / `.compile_on()` run a
 * launcher with its launch block skipped (_compile_only): arguments are validated, the kernel is resolved and its code
 * object loaded on the device, nothing is enqueued.  `.specialize()` resolves the launch's identity without compiling
 * or launching.  Here a mode is a property of the calling thread: 0 = launch, 1 = compile only (validate, resolve,
 * load), 2 = specialize only (validate, resolve; nothing is loaded).  The C++ surface sets it around one launcher call
 * and restores 0. */
cutile_status_t cutile_set_launch_mode(int32_t mode);
cutile_status_t cutile_get_launch_mode(int32_t* mode);
/* The kernel the calling thread's last launcher call resolved: its table name and the same record cutile_kernel_lookup
 * fills (`function` is NULL after a specialize-only call: nothing was loaded). */
cutile_status_t cutile_last_resolved_kernel(const char** function, cutile_kernel_info_t* info);

/* Partition::grid — cutile/src/tensor.rs:447-468 */
cutile_status_t cutile_partition_grid(const cutile_partition_arg_t* p, uint32_t grid[3]);
/* infer_launch_grid over the bounds of all partition arguments —
 * cutile/src/tile_kernel.rs:934-967.  `explicit_grid` (0,0,0) = infer. */
cutile_status_t cutile_infer_launch_grid(const uint32_t explicit_grid[3],
                                         const cutile_partition_arg_t* const* partitions,
                                         int32_t n_partitions, uint32_t grid[3]);
/* Partition::map(map_shape, num_tile_blocks) -> MappedLaunchPartition — cutile/src/tensor.rs:314-350.
 * The logical tile grid of `partition` is walked by `num_tile_blocks` tile blocks; a map dimension of
 * CUTILE_MAP_OWNED marks an axis that is not streamed (each stream item owns its full extent). */
#define CUTILE_MAP_OWNED 0
typedef struct {
  cutile_partition_arg_t partition;   /* must not be a prefix (partial-coverage) partition */
  int32_t map_rank;                   /* 1..3, must equal the rank of the logical grid */
  int32_t map_shape[3];
  uint32_t num_tile_blocks;
} cutile_mapped_partition_arg_t;
/* MappedLaunchPartition::validate — cutile/src/tensor.rs:352-400: the launch grid (num_tile_blocks, 1, 1), or
 * the reference's error ("rank-1 through rank-3 map shape", "at least one streamed (non-OWNED) map axis",
 * "non-empty logical partition grid", "map rank must match the logical partition grid rank",
 * "num_tile_blocks > 0", "num_tile_blocks cannot exceed the streamed logical tile count"). */
cutile_status_t cutile_mapped_partition_grid(const cutile_mapped_partition_arg_t* p, uint32_t grid[3]);
/* The schedule of `for index in z.iter_indices()` as a host-visible map: the block id per partition axis (owned
 * axes 0) of stream item `item`, and the number of stream items.  Tile block b visits items b, b + num_tile_blocks, ...
 * — cutile-compiler/src/compiler/compile_intrinsic.rs:2438-2900 (emit_swizzle_2d, emit_mapped_partition_schedule). */
cutile_status_t cutile_mapped_partition_index(const cutile_mapped_partition_arg_t* p, uint32_t item, uint32_t index[3],
                                              uint32_t* n_items);
/* `for index in z.iter_indices_within(ranges)` — cutile/src/_core.rs:912-930: the same schedule over a sub-range of
 * the logical grid.  `ranges` holds one (start_tile, num_tiles) pair per map axis (2 * map_rank values); num_tiles
 * -1 is the rest of the axis.  The schedule runs over the lengths and the starts are added to the block ids
 * (cutile-compiler/src/compiler/compile_expression.rs:1403-1420).  Errors as the reference's checks: negative
 * start or length, a range beyond the grid, OWNED axes (:1279-1284, :1447-1470).  `index` may be NULL to ask for
 * the item count alone (an empty range has none). */
cutile_status_t cutile_mapped_partition_index_within(const cutile_mapped_partition_arg_t* p, const int32_t* ranges,
                                                     uint32_t item, uint32_t index[3], uint32_t* n_items);
/* write_flat_index_subrange / write_flat_index_subrange_rest<BM, BN, MAP_SHAPE>(z: MappedPartitionMut<i32>, start_tile,
 * n_tiles): only the tiles inside the ranges receive their row-major index in the whole logical grid —
 * cutile/tests/gpu/mapped_partition_schedule_matrix.rs:75-106 (any rank 1..3, a pair per axis as above) */
cutile_status_t cutile_launch_mapped_tile_index_within(cutile_stream_t stream, const cutile_mapped_partition_arg_t* z,
                                                       const int32_t* ranges, const cutile_launch_opts_t* opts);
/* `a.iter_indices_with(&b)` — cutile/src/_core.rs:904-911: two mapped outputs written at the same indices must share
 * tile shape, map shape and logical grid (cutile-compiler/src/compiler/compile_expression.rs:1318-1397: "iter_indices_with
 * requires both mapped partitions to share tile and map shapes", "shared mapped partitions require equal logical
 * partition grids: axis N"). */
cutile_status_t cutile_mapped_partitions_shared(const cutile_mapped_partition_arg_t* a, const cutile_mapped_partition_arg_t* b);
/* dynpos_shared_rank3 / prefill_shared_rank3<BS, BD, MAP_SHAPE>(k_cache, v_cache: MappedPartitionMut<f32, [1,BS,BD]>, new_k,
 * pos | seq_len, n_tiles) — cutile/tests/gpu/mapped_partition_schedule_matrix.rs:107-153: one stream over
 * [(0,-1), (start, n_tiles), (0,-1)] of two caches [heads, max_seq, d]; cache tile (h, s, c) <- source tile
 * (h, s - start, c) of a [heads, seq, d] source (source_seq_major 0) or (s - start, h, c) of a [seq, heads, d] one (1);
 * v_cache receives twice the value.  `position` (one i32 in device memory) replaces start_tile when given. */
cutile_status_t cutile_launch_mapped_shared_cache_update_f32(cutile_stream_t stream, const cutile_mapped_partition_arg_t* k_cache,
                                                             const cutile_mapped_partition_arg_t* v_cache,
                                                             const cutile_tensor_arg_t* new_k, int32_t source_seq_major,
                                                             const cutile_tensor_arg_t* position, int32_t start_tile,
                                                             int32_t n_tiles, const cutile_launch_opts_t* opts);
/* gemm_persistent<T, BM, BN, BK, MAP_SHAPE>(z: MappedPartitionMut [BM,BN], x, y): z <- x . y over all of x's K,
 * zero initial accumulator — cutile-examples/examples/persistent_gemm.rs:35-59 */
cutile_status_t cutile_launch_gemm_persistent(cutile_stream_t stream, const cutile_mapped_partition_arg_t* z,
                                              const cutile_tensor_arg_t* x, const cutile_tensor_arg_t* y,
                                              const cutile_launch_opts_t* opts);
/* write_flat_index_rank{1,2,3}<.., MAP_SHAPE>(z: MappedPartitionMut<i32>): every tile a tile block visits is filled
 * with its row-major index in the logical grid — cutile/tests/gpu/mapped_partition_schedule_matrix.rs:30-76 */
cutile_status_t cutile_launch_mapped_tile_index(cutile_stream_t stream, const cutile_mapped_partition_arg_t* z,
                                                const cutile_launch_opts_t* opts);
/* SpecializationBits — cutile-compiler/src/specialization.rs:21-174 */
typedef struct {
  int32_t shape_div[CUTILE_MAX_RANK];   /* largest power of two <= 16 dividing shape[i] */
  int32_t stride_div[CUTILE_MAX_RANK];  /* same for strides (elements) */
  int32_t stride_one[CUTILE_MAX_RANK];  /* stride[i] == 1 */
  int32_t base_ptr_div;                 /* same for the base pointer (bytes) */
  int32_t elements_disjoint;
} cutile_spec_bits_t;
cutile_status_t cutile_compute_spec(const cutile_tensor_arg_t* t, cutile_spec_bits_t* spec);

/* saxpy<S, T>(y: &mut Tensor<T,S>, a: T, x: &Tensor<T,[-1,-1]>): y <- a*x + y with
 * one fused multiply-add per element.  Rank 1 or 2.  `a` is passed as f64 and
 * narrowed to T.  cutile-examples/examples/saxpy.rs:12-17, async_saxpy.rs:21-30. */
cutile_status_t cutile_launch_saxpy(cutile_stream_t stream, const cutile_partition_arg_t* y,
                                    double a, const cutile_tensor_arg_t* x,
                                    const cutile_launch_opts_t* opts);
/* axpy<B, T>(z: &mut Tensor<T,[B]>, a: T, x, y): z <- a*x + y, rank 1 (the
 * three-operand form of the same arithmetic; sibling of `add`, README.md:29-38). */
cutile_status_t cutile_launch_axpy(cutile_stream_t stream, const cutile_partition_arg_t* z, double a,
                                   const cutile_tensor_arg_t* x, const cutile_tensor_arg_t* y,
                                   const cutile_launch_opts_t* opts);
/* add<B>(z, x, y): z <- x + y.  README.md:29-38, cutile/tests/gpu/add_basic.rs:16-25. */
cutile_status_t cutile_launch_add(cutile_stream_t stream, const cutile_partition_arg_t* z,
                                  const cutile_tensor_arg_t* x, const cutile_tensor_arg_t* y,
                                  const cutile_launch_opts_t* opts);
/* creation::full / arange / linspace — cutile/src/kernels/_creation.rs:44-47,79-87,94-108 */
cutile_status_t cutile_launch_full(cutile_stream_t stream, double value, int64_t int_value,
                                   const cutile_partition_arg_t* t, const cutile_launch_opts_t* opts);
cutile_status_t cutile_launch_arange(cutile_stream_t stream, const cutile_partition_arg_t* t,
                                     const cutile_launch_opts_t* opts);
cutile_status_t cutile_launch_linspace(cutile_stream_t stream, const cutile_partition_arg_t* t,
                                       float start, float step, const cutile_launch_opts_t* opts);
/* creation::eye<BR, BC>(tensor: [BR, BC] tiles, f32, rank 2): 1 where row == column, 0 elsewhere —
 * cutile/src/kernels/_creation.rs:110-138 (behind api::eye / eye_rect, cutile/src/api.rs:613-639). */
cutile_status_t cutile_launch_eye(cutile_stream_t stream, const cutile_partition_arg_t* t,
                                  const cutile_launch_opts_t* opts);
/* The small kernels of the reference's example programs (all f32).
 *   relu<D>(input_output: [D] tiles, updated in place): max(0, x)           cutile-examples/examples/async_mlp.rs:56-61
 *   dropout<S>(p, _x, x_keep, out: [S] tiles): select(x_keep > p, x_keep, 0) / (1 - p), x_keep read as 0 beyond its
 *     extent; _x is an argument the tile program never reads                 cutile-examples/examples/dropout.rs:17-32
 *   scale_ptr(out_ptr, in_ptr, scale, len): out[i] = in[i] * scale, i < len, raw device pointers.  Like every launcher
 *     without a partition argument it needs opts->grid ("Launch grid required."); the tile program strides its blocks
 *     over whatever grid it gets, so the result does not depend on it        cutile-examples/examples/scale_ptr.rs:26-80
 *   matvec<BM, BK, K>(z: [BM] tiles, x: [M, K], y: [K]): z[r] <- z[r] + sum_k x[r, k] * y[k] over k / BK whole K tiles,
 *     rows and K positions that x or y lack reading 0                        cutile-examples/examples/async_mlp.rs:38-54 */
cutile_status_t cutile_launch_relu(cutile_stream_t stream, const cutile_partition_arg_t* input_output,
                                   const cutile_launch_opts_t* opts);
cutile_status_t cutile_launch_dropout(cutile_stream_t stream, float p, const cutile_tensor_arg_t* x,
                                      const cutile_tensor_arg_t* x_keep, const cutile_partition_arg_t* out,
                                      const cutile_launch_opts_t* opts);
cutile_status_t cutile_launch_scale_ptr(cutile_stream_t stream, void* out_ptr, const void* in_ptr, float scale, int32_t len,
                                        const cutile_launch_opts_t* opts);
cutile_status_t cutile_launch_matvec(cutile_stream_t stream, const cutile_partition_arg_t* z, const cutile_tensor_arg_t* x,
                                     const cutile_tensor_arg_t* y, int32_t k, const cutile_launch_opts_t* opts);
/* conversion::convert — cutile/src/kernels/_conversion.rs:78-85 */
cutile_status_t cutile_launch_convert(cutile_stream_t stream, const cutile_tensor_arg_t* src,
                                      const cutile_partition_arg_t* dst, const cutile_launch_opts_t* opts);
/* rms_norm_f16<N, BLOCK_SIZE>(x, w, out: [1,N] tiles, eps) — cutile-kernels/src/norms.rs:16-60 */
cutile_status_t cutile_launch_rms_norm_f16(cutile_stream_t stream, const cutile_tensor_arg_t* x,
                                           const cutile_tensor_arg_t* w,
                                           const cutile_partition_arg_t* out, float eps,
                                           const cutile_launch_opts_t* opts);
/* rms_norm<N, BLOCK_SIZE>(x: [-1, N] f32, w: [N] f32, out: [1, N] tiles f32, eps) — the f32 example form,
 * cutile-examples/examples/rms_norm.rs:17-61: out = x * sqrt_rd(1 / (mean(x^2) + eps)) * w with the square root
 * rounded toward minus infinity (:44-46). */
cutile_status_t cutile_launch_rms_norm_f32(cutile_stream_t stream, const cutile_tensor_arg_t* x,
                                           const cutile_tensor_arg_t* w, const cutile_partition_arg_t* out, float eps,
                                           const cutile_launch_opts_t* opts);
/* softmax<BM, BN>(x, y: [BM,BN] tiles), f16 or f32 — cutile-benchmarks/benches/softmax.rs:19-35,
 * cutile-examples/examples/softmax.rs:11-24 */
cutile_status_t cutile_launch_softmax(cutile_stream_t stream, const cutile_tensor_arg_t* x,
                                      const cutile_partition_arg_t* y, const cutile_launch_opts_t* opts);
/* The two benchmark programs with their own arithmetic: every product, sum, quotient and the square root an f16
 * operation (one rounding each, no fused multiply-add), where the entries above keep the statistics in f32.
 *   rms_norm<N, BLOCK_SIZE>(x, w, out: [1,N] tiles, eps: f16) — cutile-benchmarks/benches/rmsnorm.rs:20-66:
 *     a BLOCK_SIZE-lane f16 accumulator of x^2 over the N / BLOCK_SIZE tiles, reduce_sum, 1 / (sum / N + eps),
 *     square root rounded toward minus infinity, out = x * rms * w.  opts->generics = [N, BLOCK_SIZE] is required.
 *   softmax<BM, BN>(x, y: [BM,BN] tiles) — cutile-benchmarks/benches/softmax.rs:19-35: exp(x - max) / sum, the
 *     exponential evaluated in f32 and rounded once.
 * The tile programs leave the order of reduce_sum over a tile's lanes to their compiler; here it is the
 * stride-halving tree (a[l] += a[l + step], step = L/2 .. 1).  BLOCK_SIZE and BN must be powers of two
 * (at most 1024 and 16384), rows contiguous. */
cutile_status_t cutile_launch_rms_norm_all_f16(cutile_stream_t stream, const cutile_tensor_arg_t* x,
                                               const cutile_tensor_arg_t* w, const cutile_partition_arg_t* out, float eps,
                                               const cutile_launch_opts_t* opts);
cutile_status_t cutile_launch_softmax_all_f16(cutile_stream_t stream, const cutile_tensor_arg_t* x,
                                              const cutile_partition_arg_t* y, const cutile_launch_opts_t* opts);
/* ---- transformer-block kernels of cutile-kernels (f16 IO, f32 math) ------ */
/* add_rms_norm_f16<N, BLOCK_SIZE>(residual, x, w, out: [1,N] tiles, residual_out: [1,N] tiles, eps):
 * combined = residual + x; out = RMSNorm(combined) * w; residual_out = combined —
 * cutile-kernels/src/norms.rs:68-136 */
cutile_status_t cutile_launch_add_rms_norm_f16(cutile_stream_t stream, const cutile_tensor_arg_t* residual,
                                               const cutile_tensor_arg_t* x, const cutile_tensor_arg_t* w,
                                               const cutile_partition_arg_t* out,
                                               const cutile_partition_arg_t* residual_out, float eps,
                                               const cutile_launch_opts_t* opts);
/* qk_norm_f16<N, BLOCK_SIZE>(q, k, q_weight, k_weight, out: [1,N] tiles, eps, num_q_rows): rows
 * < num_q_rows of out are RMSNorm(q rows) * q_weight, the rest RMSNorm(k rows) * k_weight —
 * cutile-kernels/src/norms.rs:143-216 */
cutile_status_t cutile_launch_qk_norm_f16(cutile_stream_t stream, const cutile_tensor_arg_t* q,
                                          const cutile_tensor_arg_t* k, const cutile_tensor_arg_t* q_weight,
                                          const cutile_tensor_arg_t* k_weight, const cutile_partition_arg_t* out,
                                          float eps, int32_t num_q_rows, const cutile_launch_opts_t* opts);
/* add_2d_f16<BLOCK_SIZE>(out: [1,BLOCK] tiles, lhs, rhs) and silu_mul_2d_f16<BLOCK_SIZE>(out, gate, up):
 * out = sigmoid(gate) * gate * up — cutile-kernels/src/pointwise.rs:15-40, 46-78 */
cutile_status_t cutile_launch_add_2d_f16(cutile_stream_t stream, const cutile_partition_arg_t* out,
                                         const cutile_tensor_arg_t* lhs, const cutile_tensor_arg_t* rhs,
                                         const cutile_launch_opts_t* opts);
cutile_status_t cutile_launch_silu_mul_2d_f16(cutile_stream_t stream, const cutile_partition_arg_t* out,
                                              const cutile_tensor_arg_t* gate, const cutile_tensor_arg_t* up,
                                              const cutile_launch_opts_t* opts);
/* Rotary position embedding on [seq, heads, D] with out partitioned [1, 1, D/2] (grid.z = 2).
 * One entry point for the three reference launchers (cutile-kernels/src/positional.rs):
 *   rope_seq_f16(x, inv_freq, out, position_start)                 :13-64   k = NULL, position_start_dev = NULL
 *   rope_seq_dynpos_f16(x, inv_freq, position_start: [1] u32, out)  :70-130  k = NULL
 *   qk_rope_dynpos_f16(q, k, inv_freq, position_start, out, num_q_heads) :136-230  heads >= num_q_heads of out come from k */
cutile_status_t cutile_launch_rope_f16(cutile_stream_t stream, const cutile_tensor_arg_t* q,
                                       const cutile_tensor_arg_t* k, const cutile_tensor_arg_t* inv_freq,
                                       const cutile_tensor_arg_t* position_start_dev, int32_t position_start,
                                       const cutile_partition_arg_t* out, int32_t num_q_heads,
                                       const cutile_launch_opts_t* opts);
/* KV cache update: cache[h, position_start + s, :] = new[s, h, :] for s < seq_len, K and V together; caches
 * partitioned [1, rows, BLOCK_SIZE].  One entry point for kv_cache_update_seq_f16 (position_start_dev NULL; the
 * by-value position must be 0 as the reference's call sites assert) and kv_cache_update_seq_dynpos_f16
 * (position_start_dev: one u32) — cutile-kernels/src/kv_cache.rs:15-49, 58-97 */
cutile_status_t cutile_launch_kv_cache_update_f16(cutile_stream_t stream, const cutile_tensor_arg_t* new_k,
                                                  const cutile_tensor_arg_t* new_v, const cutile_partition_arg_t* k_cache,
                                                  const cutile_partition_arg_t* v_cache,
                                                  const cutile_tensor_arg_t* position_start_dev, int32_t position_start,
                                                  int32_t seq_len, const cutile_launch_opts_t* opts);
/* fmha_decode_gqa_split<GROUP, BN, D, NUM_KV_SPLITS>(q [kv_heads,GROUP,D], k, v [kv_heads,max_seq,D],
 * att_out: [1,GROUP,D] tiles of [kv_heads, NUM_KV_SPLITS*GROUP, D], lse_out: [1,GROUP] tiles, qk_scale,
 * position_start: [1] u32): keys 0..position_start, split over grid.y — cutile-kernels/src/attention.rs:737-902 */
cutile_status_t cutile_launch_fmha_decode_gqa_split(cutile_stream_t stream, const cutile_tensor_arg_t* q,
                                                    const cutile_tensor_arg_t* k, const cutile_tensor_arg_t* v,
                                                    const cutile_partition_arg_t* att_out,
                                                    const cutile_partition_arg_t* lse_out, float qk_scale,
                                                    const cutile_tensor_arg_t* position_start,
                                                    const cutile_launch_opts_t* opts);
/* attention_decode_kernel_grouped<E, HEAD_DIM, TILE_N, KV_LEN_PER_SPLIT, NUM_Q_HEAD_PER_KV, QUERY_GROUP_TILE_SIZE,
 * NUM_KV_SPLITS>(q_ptr, q_s0..3, q_str0..2, k_ptr, .., v_ptr, .., att_ptr, att_s0..4, att_str0..3, lse_ptr, lse_s0..3,
 * lse_str0..2, softmax_scale, s_kv_ptr) — cutile-kernels/src/experimental/attention.rs:385-846: the split-KV decode
 * partial on raw pointers, f16.  Each (pointer, shape scalars, stride scalars) group of the reference arrives as a
 * pointer and two arrays; strides are in elements and the innermost one (always 1) is not passed.
 *   q [B, H_kv, G, D]   k, v [B, H_kv, S, D]   att [B, H_kv, G, NUM_KV_SPLITS, D]   lse [B, H_kv, G, NUM_KV_SPLITS] f32
 * Split t covers keys [t * KV_LEN_PER_SPLIT, min((t + 1) * KV_LEN_PER_SPLIT, *s_kv)); *s_kv is one i32 in device memory
 * (keys in the cache, at most S).  A split without keys writes zeros and lse = -inf.  lse is in the log2 domain:
 * max + log2(sum) of softmax_scale * log2(e) * scores.  Launch grid (B, H_kv, NUM_KV_SPLITS) as in the reference.
 * KV_LEN_PER_SPLIT must be a multiple of TILE_N (otherwise the reference's splits overlap: no variant is built for
 * that).  Generics, when given, are checked in the order HEAD_DIM, TILE_N, KV_LEN_PER_SPLIT, NUM_Q_HEAD_PER_KV,
 * QUERY_GROUP_TILE_SIZE, NUM_KV_SPLITS. */
cutile_status_t cutile_launch_attention_decode_kernel_grouped_f16(
    cutile_stream_t stream, const void* q, const int32_t* q_shape /*4*/, const int32_t* q_strides /*3*/, const void* k,
    const int32_t* k_shape /*4*/, const int32_t* k_strides /*3*/, const void* v, const int32_t* v_shape /*4*/,
    const int32_t* v_strides /*3*/, void* att, const int32_t* att_shape /*5*/, const int32_t* att_strides /*4*/, void* lse,
    const int32_t* lse_shape /*4*/, const int32_t* lse_strides /*3*/, float softmax_scale, const void* s_kv, int32_t tile_n,
    int32_t kv_len_per_split, int32_t query_group_tile_size, const cutile_launch_opts_t* opts);
/* splitk_reduce_merge<GROUP, D, CHUNK_D, NUM_KV_SPLITS>(att_partial, lse_partial, out: [1,GROUP,CHUNK_D] tiles):
 * softmax-weighted sum of the splits — cutile-kernels/src/attention.rs:917-1013 */
cutile_status_t cutile_launch_splitk_reduce_merge(cutile_stream_t stream, const cutile_tensor_arg_t* att_partial,
                                                  const cutile_tensor_arg_t* lse_partial, const cutile_partition_arg_t* out,
                                                  const cutile_launch_opts_t* opts);
/* One decode-attention step that allocates nothing.  It has no counterpart in the reference: it is for callers
 * that cannot allocate device memory (code under graph capture, tight serving loops, harnesses that forbid it).
 * Computes what cutile_launch_fmha_decode_gqa_split followed by cutile_launch_splitk_reduce_merge compute — q
 * [kv_heads, GROUP, D], k, v [kv_heads, max_seq, D], keys 0..*position_start dealt to `num_kv_splits` splits in tiles
 * of `bn` keys, out [kv_heads, GROUP, D] partitioned [1, GROUP, CHUNK_D] — with the partial results
 * (kv_heads * num_kv_splits * GROUP rows of D f16 values, rounded up to 256 bytes, plus 4 bytes of log-sum-exp per row)
 * in a device-resident array of cutile_scratch_capacity() bytes (8 MiB) that each GPU holds from its first call until
 * the process ends.  A call that needs more fails with CUTILE_ERR_KERNEL_LAUNCH before any GPU work.  No device memory
 * is allocated or freed, here or in the kernels.  Every call on one GPU uses that GPU's one array: calls that overlap
 * on one GPU (two streams, two threads) race; calls on one stream are ordered.  Nothing in the array has to start
 * at zero — the split kernel writes every row a merge reads — so nothing is cleared between calls. */
cutile_status_t cutile_launch_fmha_decode_gqa_noalloc(cutile_stream_t stream, const cutile_tensor_arg_t* q,
                                                      const cutile_tensor_arg_t* k, const cutile_tensor_arg_t* v,
                                                      const cutile_partition_arg_t* out, float qk_scale,
                                                      const cutile_tensor_arg_t* position_start, int32_t num_kv_splits,
                                                      int32_t bn);
/* Warm-up for the entry point above; like it, without a counterpart in the reference.  The first call of the entry
 * point on a device opens the side library that holds the array, looks the array's address up (the runtime places the
 * 8 MiB then) and loads two code objects: work that is neither allocation-free nor legal while a stream is being
 * captured.  This call does all of it and enqueues nothing (the entry point in compile-only mode: the arguments are
 * checked exactly as a launch checks them, no pointer is dereferenced).  Call it once per device and shape outside any
 * capture; after it, cutile_launch_fmha_decode_gqa_noalloc with the same shapes only enqueues two kernels. */
cutile_status_t cutile_fmha_decode_gqa_noalloc_prepare(const cutile_tensor_arg_t* q, const cutile_tensor_arg_t* k,
                                                       const cutile_tensor_arg_t* v, const cutile_partition_arg_t* out,
                                                       const cutile_tensor_arg_t* position_start, int32_t num_kv_splits,
                                                       int32_t bn);
/* bytes of the device-resident scratch array behind cutile_launch_fmha_decode_gqa_noalloc (needs no GPU) */
cutile_status_t cutile_scratch_capacity(size_t* bytes);
/* gemm<T, BM, BN, BK>(z: [BM,BN] tiles, x, y, k): z <- z + x·y with f32
 * accumulation (z is read as the initial accumulator, like the reference bench;
 * `accumulate` = 0 starts from zero like the example) —
 * cutile-benchmarks/benches/gemm.rs:20-41, cutile-examples/examples/gemm.rs:20-36 */
cutile_status_t cutile_launch_gemm(cutile_stream_t stream, const cutile_partition_arg_t* z,
                                   const cutile_tensor_arg_t* x, const cutile_tensor_arg_t* y,
                                   int32_t k, int32_t accumulate, const cutile_launch_opts_t* opts);
/* batch_matmul<E, BM, BN, BK, K>(c: [1, BM, BN] tiles of [batches, M, N], a: [batches, M, K], b: [batches, K, N]):
 * c[p] = a[p] · b[p] from zero accumulators over k / BK whole K tiles, all batches in one launch, tile grid
 * (batches, M tiles, N tiles) — cutile-examples/examples/batch_matmul.rs:16-44.  E = f32 (the example), f16 or bf16
 * (f32 accumulation, one rounding at the store). */
cutile_status_t cutile_launch_batch_matmul(cutile_stream_t stream, const cutile_partition_arg_t* c,
                                           const cutile_tensor_arg_t* a, const cutile_tensor_arg_t* b, int32_t k,
                                           const cutile_launch_opts_t* opts);
/* copy_stacked_to_contiguous_f16 / copy_contiguous_to_stacked_f16(num_blocks, stacked_tensors, contiguous_tensors, nh, nl,
 * no, nt, hd) — cutile-kernels/src/experimental/kvbm.rs:112-187, 283-352.  KV cache blocks of nh heads x nl layers x
 * no offsets x nt tokens x hd values move between the stacked form (one f16 tensor per (block, layer, offset), table
 * entry (block * nl + layer) * no + offset, laid out [nt, nh, hd] or [nh, nt, hd]) and the contiguous form (one tensor
 * per block).  The reference passes the layouts as index maps in its generics (StackedLayout / ContiguousLayout,
 * kvbm.rs:358-400); here they are the two enumerators, with the same four supported pairs. */
enum { CUTILE_KVBM_STACKED_NHD = 0, CUTILE_KVBM_STACKED_HND = 1 };
enum { CUTILE_KVBM_OPERATIONAL_NHD = 0, CUTILE_KVBM_OPERATIONAL_HND = 1, CUTILE_KVBM_UNIVERSAL = 2 };
cutile_status_t cutile_launch_copy_stacked_to_contiguous_f16(cutile_stream_t stream, int32_t stacked_layout, int32_t contiguous_layout,
                                                             int32_t num_blocks, const cutile_tensor_arg_t* stacked_tensors,
                                                             const cutile_tensor_arg_t* contiguous_tensors, int32_t nh, int32_t nl,
                                                             int32_t no, int32_t nt, int32_t hd, const cutile_launch_opts_t* opts);
cutile_status_t cutile_launch_copy_contiguous_to_stacked_f16(cutile_stream_t stream, int32_t stacked_layout, int32_t contiguous_layout,
                                                             int32_t num_blocks, const cutile_tensor_arg_t* stacked_tensors,
                                                             const cutile_tensor_arg_t* contiguous_tensors, int32_t nh, int32_t nl,
                                                             int32_t no, int32_t nt, int32_t hd, const cutile_launch_opts_t* opts);
/* add_rms_norm_decode_raw_f16<N, BLOCK_SIZE>(residual_ptr, x_ptr, w_ptr, out_ptr, residual_out_ptr, eps) —
 * cutile-kernels/src/experimental/norms.rs:22-153: add_rms_norm_f16 on one row of N halves, raw device pointers. */
cutile_status_t cutile_launch_add_rms_norm_decode_raw_f16(cutile_stream_t stream, const void* residual, const void* x,
                                                          const void* w, void* out, void* residual_out, float eps,
                                                          int32_t n, const cutile_launch_opts_t* opts);
/* qk_norm_rope_kv_prefill_raw_f16<D, HALF_D, MAX_SEQ>(q_ptr, k_ptr, v_ptr, q_weight_ptr, k_weight_ptr, inv_freq_ptr,
 * q_out_ptr, k_cache_ptr, v_cache_ptr, eps, position_start, seq_len, num_q_heads, num_kv_heads) —
 * cutile-kernels/src/experimental/fused_transformer.rs:22-345.  Raw device pointers as in the reference: q, q_out
 * [seq_len, num_q_heads, D], k, v [seq_len, num_kv_heads, D], weights [D] (all f16, contiguous, 16-byte aligned),
 * inv_freq [D/2] f32, caches [num_kv_heads, MAX_SEQ, D].  One launch does Q/K RMS norm, rotary embedding at positions
 * position_start + s and the cache update.  D and MAX_SEQ are arguments here (generics 0 and 2 are checked). */
cutile_status_t cutile_launch_qk_norm_rope_kv_prefill_raw_f16(cutile_stream_t stream, const void* q, const void* k,
                                                              const void* v, const void* q_weight, const void* k_weight,
                                                              const void* inv_freq, void* q_out, void* k_cache,
                                                              void* v_cache, float eps, int32_t position_start,
                                                              int32_t seq_len, int32_t num_q_heads, int32_t num_kv_heads,
                                                              int32_t d, int32_t max_seq, const cutile_launch_opts_t* opts);
/* qk_norm_rope_kv_decode_raw_f16<D, HALF_D, MAX_SEQ>(qkv_ptr, q_weight_ptr, k_weight_ptr, inv_freq_ptr, q_out_ptr,
 * k_cache_ptr, v_cache_ptr, position_start: [1] u32, eps, num_q_heads, num_kv_heads) — fused_transformer.rs:356-625:
 * the same for one token whose q, k and v heads sit back to back in qkv [(num_q_heads + 2 num_kv_heads) * D] and whose
 * position is read from device memory. */
cutile_status_t cutile_launch_qk_norm_rope_kv_decode_raw_f16(cutile_stream_t stream, const void* qkv, const void* q_weight,
                                                             const void* k_weight, const void* inv_freq, void* q_out,
                                                             void* k_cache, void* v_cache,
                                                             const cutile_tensor_arg_t* position_start, float eps,
                                                             int32_t num_q_heads, int32_t num_kv_heads, int32_t d,
                                                             int32_t max_seq, const cutile_launch_opts_t* opts);
/* group_gemm_f16_nt_desc<BM, BN, BK, NUM_SM>(a_ptrs, b_ptrs, c_ptrs: [groups] i64 device addresses; a_metas, b_metas,
 * c_metas: [groups, 8] i32 rows = (rows, cols, row stride in elements, ...); num_groups) —
 * cutile-kernels/src/experimental/moe.rs:67-128: C_g [m, n] = A_g [m, k] . B_g [k, n] per group, f16 with f32
 * accumulation, NUM_SM persistent tile blocks over the tiles of all groups.  The descriptors live in device memory and
 * are trusted as in the reference (16-byte aligned pointers, rows / cols multiples of 16, row strides multiples of 8).
 * There is no partition to infer from: the grid comes from opts->grid or generic 3 (NUM_SM), the tile from generics
 * 0 and 1 (BM, BN; default 128 x 128). */
cutile_status_t cutile_launch_group_gemm_f16_nt_desc(cutile_stream_t stream, const cutile_tensor_arg_t* a_ptrs,
                                                     const cutile_tensor_arg_t* b_ptrs, const cutile_tensor_arg_t* c_ptrs,
                                                     const cutile_tensor_arg_t* a_metas, const cutile_tensor_arg_t* b_metas,
                                                     const cutile_tensor_arg_t* c_metas, int32_t num_groups,
                                                     const cutile_launch_opts_t* opts);
/* argmax_blocks_f16<BLOCK_SIZE>(logits: [n] f16, block_max: [blocks] f32 tiles [1], block_idx: [blocks] u32 tiles [1],
 * len) — cutile-kernels/src/argmax.rs:21-71.  Block b holds the largest of logits[b*BLOCK_SIZE ..] (positions >= len
 * count as -1e30) and the smallest index that attains it.  BLOCK_SIZE is generic 0 (default 1024). */
cutile_status_t cutile_launch_argmax_blocks_f16(cutile_stream_t stream, const cutile_tensor_arg_t* logits,
                                                const cutile_partition_arg_t* block_max,
                                                const cutile_partition_arg_t* block_idx, int32_t len,
                                                const cutile_launch_opts_t* opts);
/* lm_head_argmax_blocks_f16<K>(weights: [vocab, K] f16, hidden: [1, K] f16, block_max, block_idx, vocab_size) —
 * argmax.rs:88-158: logits = weights . hidden in f32, never stored; one block per 64 rows of weights. */
cutile_status_t cutile_launch_lm_head_argmax_blocks_f16(cutile_stream_t stream, const cutile_tensor_arg_t* weights,
                                                        const cutile_tensor_arg_t* hidden,
                                                        const cutile_partition_arg_t* block_max,
                                                        const cutile_partition_arg_t* block_idx, int32_t vocab_size,
                                                        const cutile_launch_opts_t* opts);
/* argmax_reduce_blocks_to_u32<BLOCK_SIZE>(block_max: [n] f32, block_idx: [n] u32, out: [1] u32 tile [1], num_blocks) —
 * argmax.rs:173-213: the index of the largest of the first num_blocks block maxima (ties: smallest index).
 * One tile of BLOCK_SIZE entries is read, as in the reference (generic 0, default: num_blocks rounded up to 256). */
cutile_status_t cutile_launch_argmax_reduce_blocks_to_u32(cutile_stream_t stream, const cutile_tensor_arg_t* block_max,
                                                          const cutile_tensor_arg_t* block_idx,
                                                          const cutile_partition_arg_t* out, int32_t num_blocks,
                                                          const cutile_launch_opts_t* opts);
/* embedding_batch_f16<D, BLOCK_SIZE>(token_ids: [n] u32, table: [vocab, D] f16, out: [n, D] tiles [1, BLOCK_SIZE]) —
 * cutile-kernels/src/embeddings.rs:21-41: out[r, :] = table[token_ids[r], :]. */
cutile_status_t cutile_launch_embedding_batch_f16(cutile_stream_t stream, const cutile_tensor_arg_t* token_ids,
                                                  const cutile_tensor_arg_t* table, const cutile_partition_arg_t* out,
                                                  const cutile_launch_opts_t* opts);
/* gather_row_f16<BLOCK_SIZE>(src: [rows, width] f16, out: [width] tiles [BLOCK_SIZE], row_idx) —
 * cutile-kernels/src/pointwise.rs:86-99: out = src[row_idx, :]. */
cutile_status_t cutile_launch_gather_row_f16(cutile_stream_t stream, const cutile_tensor_arg_t* src,
                                             const cutile_partition_arg_t* out, int32_t row_idx,
                                             const cutile_launch_opts_t* opts);
/* The sequence-layout attention kernels of cutile-kernels, one entry point for the five of them:
 *   flash_attn_causal_seq_f16<BM,BN,D>(q, k, v, out, qk_scale, query_group_size, kv_len, query_start)
 *       cutile-kernels/src/attention.rs:21-116   -> position_start = NULL, causal = 1
 *   flash_attn_causal_seq_dynpos_f16<BM,BN,D>(.., query_group_size, position_start)
 *       attention.rs:128-231  -> position_start given, kv_len_from_position = 1, causal = 1
 *   fmha_prefill_causal<BM,BN,D,CAUSAL,EVEN_K,LATENCY>(.., kv_len, query_start)
 *       attention.rs:242-391  -> position_start = NULL
 *   fmha_prefill_gqa<BM,BN,D,GROUP,M_EFF,CAUSAL,EVEN_K,LATENCY>(..)   (out tiles [BM, GROUP, D])
 *       attention.rs:408-587  -> position_start = NULL
 *   fmha_causal<BM,BN,D,CAUSAL,EVEN_K>(.., qk_scale: f16, query_group_size, position_start)
 *       attention.rs:598-726  -> position_start given, kv_len_from_position = 0, kv_len = dim(k, 1)
 * q and out are [q_len, q_heads, D], k and v [kv_heads, max_seq, D], all f16; out is partitioned
 * [BM, G, D] with G = 1 or the packing factor of the gqa form.  Query i of the launch stands at position
 * query_start + i (by value, or *position_start: one u32 in device memory); it attends to keys j < kv_len
 * and, when causal, j <= its position.  Rows without any key are written as zeros (l_safe = max(l, 1e-8)).
 * Generics, when given, are checked at index 0 (BM) and 2 (D). */
cutile_status_t cutile_launch_fmha_seq_f16(cutile_stream_t stream, const cutile_tensor_arg_t* q,
                                           const cutile_tensor_arg_t* k, const cutile_tensor_arg_t* v,
                                           const cutile_partition_arg_t* out, float qk_scale,
                                           int32_t query_group_size, int32_t kv_len, int32_t query_start,
                                           const cutile_tensor_arg_t* position_start, int32_t kv_len_from_position,
                                           int32_t causal, const cutile_launch_opts_t* opts);
/* fmha_prefill_gqa_lpt<BM, BN, D, GROUP, M_EFF, CAUSAL, EVEN_K, LATENCY, SCHED, MASK_SPLIT>(q_ptr, k_ptr, v_ptr, out_ptr,
 * qk_scale, query_group_size, q_len, kv_len, query_start, num_q_blocks, num_head_groups, swizzle, ...) —
 * cutile-kernels/src/experimental/attention.rs:22-377: fmha_prefill_gqa on raw pointers (q, out [q_len, heads, D];
 * k, v [kv_heads, kv_len, D], contiguous).  The reference's scheduling arguments (block order, swizzle) do not change
 * the result and have no counterpart: the kernels order their tiles themselves.  GROUP, D and CAUSAL are arguments
 * here; generics 0 (BM), 2 (D) and 3 (GROUP) are checked when given. */
cutile_status_t cutile_launch_fmha_prefill_gqa_lpt_raw_f16(cutile_stream_t stream, const void* q, const void* k, const void* v,
                                                           void* out, float qk_scale, int32_t query_group_size, int32_t q_len,
                                                           int32_t kv_len, int32_t query_start, int32_t num_head_groups,
                                                           int32_t group, int32_t d, int32_t causal,
                                                           const cutile_launch_opts_t* opts);
/* fmha<BM, BN, D, H, CAUSAL, EVEN_K>(out: [1,BM,D] tiles, q, k, v, qk_scale,
 * input_pos, query_group_size) — cutile-examples/examples/flash_attention_causal.rs:19-134,
 * cutile-benchmarks/benches/fmha.rs:20-145 (non-causal: causal = 0, input_pos = 0) */
cutile_status_t cutile_launch_fmha(cutile_stream_t stream, const cutile_partition_arg_t* out,
                                   const cutile_tensor_arg_t* q, const cutile_tensor_arg_t* k,
                                   const cutile_tensor_arg_t* v, float qk_scale, int32_t input_pos,
                                   int32_t query_group_size, int32_t causal,
                                   const cutile_launch_opts_t* opts);
/* linear_tile<BM, BN, BK, BK/32>(z: [BM,BN] tiles, x[M,K], y[N,K], x_scales[M,K/32],
 * y_scales[N,K/32], alpha): z <- alpha * (x·sx) @ (y·sy)^T, e4m3 data, e8m0
 * scales, f32 accumulation; z is f32 or bf16 — cutile-examples/examples/mxfp8.rs:34-64 */
cutile_status_t cutile_launch_linear_tile_mxfp8(cutile_stream_t stream, const cutile_partition_arg_t* z,
                                                const cutile_tensor_arg_t* x, const cutile_tensor_arg_t* y,
                                                const cutile_tensor_arg_t* x_scales,
                                                const cutile_tensor_arg_t* y_scales, float alpha,
                                                const cutile_launch_opts_t* opts);
/* NVFP4 linear_tile<BM, BN, BK, BK_PACKED, BK_SCALES>(z: [BM,BN] tiles, x, y, x_scales, y_scales, alpha):
 * z = alpha * (x . sx) @ (y . sy)^T with x [M, K/2], y [N, K/2] packed e2m1 pairs, scales [M, K/16], [N, K/16]
 * e4m3fn, one per 16 K values; z f32 (as the reference) or bf16 — cutile-examples/examples/nvfp4.rs:24-78 */
cutile_status_t cutile_launch_linear_tile_nvfp4(cutile_stream_t stream, const cutile_partition_arg_t* z,
                                                const cutile_tensor_arg_t* x, const cutile_tensor_arg_t* y,
                                                const cutile_tensor_arg_t* x_scales, const cutile_tensor_arg_t* y_scales,
                                                float alpha, const cutile_launch_opts_t* opts);

/* ======================================================================== */
/* Part E — asynchronous runtime                                             */
/* ======================================================================== */
/* Thread-local execution lock: on a thread only one DeviceOp executes at a time
 * (cuda-async/src/device_operation.rs:27-55).  Acquiring it twice on one thread
 * fails with CUTILE_ERR_STATE and the reference's "non-reentrant" message. */
cutile_status_t cutile_execution_lock_acquire(void);
void cutile_execution_lock_release(void);
int32_t cutile_execution_lock_held(void);

/* Thread-local device contexts (cuda-async/src/device_context.rs:139-450).  Each
 * thread has a default device and, per device, a scheduling policy, a dedicated
 * deallocator stream and an optional memory pool; tests isolate state by running
 * on fresh threads, as the reference's do. */
typedef enum { CUTILE_POLICY_ROUND_ROBIN = 0, CUTILE_POLICY_SINGLE_STREAM = 1 } cutile_policy_kind_t;
int32_t cutile_get_default_device(void);                      /* device_context.rs:164 */
void cutile_set_default_device(int32_t ordinal);              /* device_context.rs:363-367 */
/* init_device_contexts: a second call on a thread fails "Context already
 * initialized." (device_context.rs:178-195) */
cutile_status_t cutile_init_device_contexts(int32_t default_device, int32_t num_devices);
/* init_device with an explicit policy; a second call for the same device fails
 * "Device is already initialized." (device_context.rs:235-260).  num_streams <= 0
 * selects the default pool of 4 (device_context.rs:39). */
cutile_status_t cutile_init_device(int32_t ordinal, cutile_policy_kind_t kind, int32_t num_streams);
/* with_device_policy(|p| p.next_stream()): ordinal < 0 = the thread's default
 * device; contexts are created lazily with the round-robin policy
 * (device_context.rs:315-328,444-450; scheduling_policies.rs:35-87). */
cutile_status_t cutile_policy_next_stream(int32_t ordinal, cutile_stream_t* stream);
/* with_deallocator_stream (device_context.rs:330-338): the stream frees are queued on */
cutile_status_t cutile_deallocator_stream(int32_t ordinal, cutile_stream_t* stream);
/* set_device_pool / get_device_pool (device_context.rs:396-432); NULL clears */
cutile_status_t cutile_set_device_pool(int32_t ordinal, cutile_mempool_t pool);
cutile_status_t cutile_get_device_pool(int32_t ordinal, cutile_mempool_t* pool);

/* Completion notification for work already submitted on `stream`.  `waker(user)`
 * is called exactly once, from another thread, after that work has completed.
 * cutile_reactor_register is the flag-write path (cuda-async/src/reactor.rs:154-179):
 * take one of 1024 slots, enqueue a 32-bit stream write of that use's stamp into
 * pinned mapped memory, hand the waker to the sweeper thread; CUTILE_ERR_OUT_OF_SLOTS
 * when all slots are in flight.  cutile_completion_register is the chain
 * DeviceFuture uses (cuda-async/src/device_future.rs:103-154): reactor first,
 * hipLaunchHostFunc as fallback (or always, with CUTILE_ASYNC_HOST_SYNC=callback). */
typedef void (*cutile_waker_fn_t)(void* user);
cutile_status_t cutile_reactor_register(cutile_stream_t stream, cutile_waker_fn_t waker, void* user);
cutile_status_t cutile_completion_register(cutile_stream_t stream, cutile_waker_fn_t waker, void* user);
uint64_t cutile_reactor_registrations(void);
uint64_t cutile_reactor_wakes(void);
int32_t cutile_reactor_armed(void);

#ifdef __cplusplus
}
#endif
#endif /* CUTILE_HIP_H */
