"""ctypes binding of ``libcutile_hip.so`` for tests, the smoke check and ``bench.py``.

The product is the C-ABI library (``include/cutile_hip.h``) and the C++ host surface
above it; this module only marshals ``torch`` tensors (device memory and streams) into
the ABI's plain records.  The directory name is not a Python identifier, so the package
is imported through ``__graft_entry__.load_package()`` under the name ``cutile_rs_amd``.

Launcher functions keep the reference's argument order (the ``#[cutile::entry]``
signatures): outputs are passed as :class:`Partition` objects created with
:func:`partition`, exactly where the reference takes ``tensor.partition([...])``.
Nothing here computes on the CPU: if the library is missing, importing fails; if no
GPU is present, every launch raises :class:`CutileError`.
"""
from __future__ import annotations

import ctypes as C
import os
from dataclasses import dataclass
from typing import Optional, Sequence

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libcutile_hip.so")
# the same library plus the recording stand-in for the HIP runtime (include/cutile_hip_testing.h): what the CPU tests load
TESTING_LIB_PATH = os.path.join(_HERE, "lib", "libcutile_hip_testing.so")
MAX_RANK = 4

# cutile_dtype_t
(F32, F64, F16, BF16, I8, I16, I32, I64, U8, U16, U32, U64, BOOL, F8E4M3FN, F8E5M2, F8E8M0FNU, F4E2M1FNX2,
 DTYPE_COUNT) = range(18)


class CutileError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"[{status}] {message}")
        self.status = status
        self.message = message


class TensorArg(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("dtype", C.c_int), ("rank", C.c_int32),
                ("shape", C.c_int32 * MAX_RANK), ("strides", C.c_int32 * MAX_RANK)]


class PartitionArg(C.Structure):
    _fields_ = [("tensor", TensorArg), ("partition_shape", C.c_int32 * MAX_RANK),
                ("partition_strides", C.c_int32 * MAX_RANK), ("prefix_coverage", C.c_int32)]


class MappedPartitionArg(C.Structure):
    _fields_ = [("partition", PartitionArg), ("map_rank", C.c_int32), ("map_shape", C.c_int32 * 3),
                ("num_tile_blocks", C.c_uint32)]


class LaunchOpts(C.Structure):
    _fields_ = [("grid", C.c_uint32 * 3), ("generics", C.POINTER(C.c_char_p)), ("n_generics", C.c_int32),
                ("variant", C.c_char_p)]


class KernelInfo(C.Structure):
    _fields_ = [("function", C.c_void_p), ("symbol", C.c_char_p), ("variant", C.c_char_p),
                ("block", C.c_uint32 * 3), ("lds_bytes", C.c_uint32), ("tile", C.c_int32 * 4)]


class SpecBits(C.Structure):
    _fields_ = [("shape_div", C.c_int32 * MAX_RANK), ("stride_div", C.c_int32 * MAX_RANK),
                ("stride_one", C.c_int32 * MAX_RANK), ("base_ptr_div", C.c_int32), ("elements_disjoint", C.c_int32)]


class DeviceProps(C.Structure):
    _fields_ = [("compute_units", C.c_int32), ("clock_khz", C.c_int32), ("memory_clock_khz", C.c_int32),
                ("memory_bus_bits", C.c_int32), ("l2_bytes", C.c_int32), ("lds_bytes_per_block", C.c_int32),
                ("wavefront_size", C.c_int32), ("reserved", C.c_int32), ("total_memory_bytes", C.c_uint64)]


class LaunchRecord(C.Structure):
    _fields_ = [("symbol", C.c_char_p), ("grid", C.c_uint32 * 3), ("block", C.c_uint32 * 3),
                ("shared_mem_bytes", C.c_uint32), ("stream", C.c_void_p), ("args", C.POINTER(C.c_ubyte)),
                ("args_size", C.c_size_t), ("in_capture", C.c_int32), ("from_graph_replay", C.c_int32)]


_lib: Optional[C.CDLL] = None


def lib() -> C.CDLL:
    """The loaded C-ABI library.  Fails loudly when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is missing: run `python cutile-rs_amd/build.py` "
                              "(or __graft_entry__.build()) first; there is no fallback path")
        L = C.CDLL(LIB_PATH)
        L.cutile_last_error_message.restype = C.c_char_p
        L.cutile_status_name.restype = C.c_char_p
        L.cutile_status_name.argtypes = [C.c_int32]
        L.cutile_version.restype = C.c_char_p
        L.cutile_dtype_name.restype = C.c_char_p
        L.cutile_dtype_name.argtypes = [C.c_int]
        L.cutile_dtype_size.restype = C.c_size_t
        L.cutile_dtype_size.argtypes = [C.c_int]
        L.cutile_dtype_from_name.restype = C.c_int
        L.cutile_dtype_from_name.argtypes = [C.c_char_p]
        L.cutile_module_load_count.restype = C.c_uint64
        if hasattr(L, "cutile_testing_use_fake_hip"):      # only the testing library carries the recording runtime
            L.cutile_testing_streams_created.restype = C.c_uint64
            L.cutile_testing_bytes_allocated.restype = C.c_uint64
        vp, f32, f64, i32, i64 = C.c_void_p, C.c_float, C.c_double, C.c_int32, C.c_int64
        P = C.POINTER
        sig = {
            "cutile_launch_saxpy": [vp, P(PartitionArg), f64, P(TensorArg), P(LaunchOpts)],
            "cutile_launch_axpy": [vp, P(PartitionArg), f64, P(TensorArg), P(TensorArg), P(LaunchOpts)],
            "cutile_launch_add": [vp, P(PartitionArg), P(TensorArg), P(TensorArg), P(LaunchOpts)],
            "cutile_launch_full": [vp, f64, i64, P(PartitionArg), P(LaunchOpts)],
            "cutile_launch_arange": [vp, P(PartitionArg), P(LaunchOpts)],
            "cutile_launch_eye": [vp, P(PartitionArg), P(LaunchOpts)],
            "cutile_launch_relu": [vp, P(PartitionArg), P(LaunchOpts)],
            "cutile_launch_dropout": [vp, f32, P(TensorArg), P(TensorArg), P(PartitionArg), P(LaunchOpts)],
            "cutile_launch_scale_ptr": [vp, vp, vp, f32, i32, P(LaunchOpts)],
            "cutile_launch_matvec": [vp, P(PartitionArg), P(TensorArg), P(TensorArg), i32, P(LaunchOpts)],
            "cutile_launch_batch_matmul": [vp, P(PartitionArg), P(TensorArg), P(TensorArg), i32, P(LaunchOpts)],
            "cutile_launch_linspace": [vp, P(PartitionArg), f32, f32, P(LaunchOpts)],
            "cutile_launch_convert": [vp, P(TensorArg), P(PartitionArg), P(LaunchOpts)],
            "cutile_launch_rms_norm_f16": [vp, P(TensorArg), P(TensorArg), P(PartitionArg), f32, P(LaunchOpts)],
            "cutile_launch_rms_norm_f32": [vp, P(TensorArg), P(TensorArg), P(PartitionArg), f32, P(LaunchOpts)],
            "cutile_launch_softmax": [vp, P(TensorArg), P(PartitionArg), P(LaunchOpts)],
            "cutile_launch_rms_norm_all_f16": [vp, P(TensorArg), P(TensorArg), P(PartitionArg), f32, P(LaunchOpts)],
            "cutile_launch_softmax_all_f16": [vp, P(TensorArg), P(PartitionArg), P(LaunchOpts)],
            "cutile_launch_add_rms_norm_f16": [vp, P(TensorArg), P(TensorArg), P(TensorArg), P(PartitionArg),
                                               P(PartitionArg), f32, P(LaunchOpts)],
            "cutile_launch_qk_norm_f16": [vp, P(TensorArg), P(TensorArg), P(TensorArg), P(TensorArg), P(PartitionArg),
                                          f32, i32, P(LaunchOpts)],
            "cutile_launch_add_2d_f16": [vp, P(PartitionArg), P(TensorArg), P(TensorArg), P(LaunchOpts)],
            "cutile_launch_silu_mul_2d_f16": [vp, P(PartitionArg), P(TensorArg), P(TensorArg), P(LaunchOpts)],
            "cutile_launch_kv_cache_update_f16": [vp, P(TensorArg), P(TensorArg), P(PartitionArg), P(PartitionArg),
                                                  P(TensorArg), i32, i32, P(LaunchOpts)],
            "cutile_launch_fmha_decode_gqa_split": [vp, P(TensorArg), P(TensorArg), P(TensorArg), P(PartitionArg),
                                                    P(PartitionArg), f32, P(TensorArg), P(LaunchOpts)],
            "cutile_launch_splitk_reduce_merge": [vp, P(TensorArg), P(TensorArg), P(PartitionArg), P(LaunchOpts)],
            "cutile_launch_fmha_decode_gqa_noalloc": [vp, P(TensorArg), P(TensorArg), P(TensorArg), P(PartitionArg), f32,
                                                      P(TensorArg), i32, i32],
            "cutile_fmha_decode_gqa_noalloc_prepare": [P(TensorArg), P(TensorArg), P(TensorArg), P(PartitionArg), P(TensorArg), i32, i32],
            "cutile_scratch_capacity": [P(C.c_size_t)],
            "cutile_launch_rope_f16": [vp, P(TensorArg), P(TensorArg), P(TensorArg), P(TensorArg), i32, P(PartitionArg),
                                       i32, P(LaunchOpts)],
            "cutile_launch_gemm": [vp, P(PartitionArg), P(TensorArg), P(TensorArg), i32, i32, P(LaunchOpts)],
            "cutile_launch_fmha": [vp, P(PartitionArg), P(TensorArg), P(TensorArg), P(TensorArg), f32, i32, i32, i32,
                                   P(LaunchOpts)],
            "cutile_launch_copy_stacked_to_contiguous_f16": [vp, i32, i32, i32, P(TensorArg), P(TensorArg), i32, i32, i32, i32, i32, P(LaunchOpts)],
            "cutile_launch_copy_contiguous_to_stacked_f16": [vp, i32, i32, i32, P(TensorArg), P(TensorArg), i32, i32, i32, i32, i32, P(LaunchOpts)],
            "cutile_launch_add_rms_norm_decode_raw_f16": [vp, vp, vp, vp, vp, vp, f32, i32, P(LaunchOpts)],
            "cutile_launch_qk_norm_rope_kv_prefill_raw_f16": [vp] + [vp] * 9 + [f32, i32, i32, i32, i32, i32, i32, P(LaunchOpts)],
            "cutile_launch_qk_norm_rope_kv_decode_raw_f16": [vp] + [vp] * 7 + [P(TensorArg), f32, i32, i32, i32, i32, P(LaunchOpts)],
            "cutile_launch_group_gemm_f16_nt_desc": [vp, P(TensorArg), P(TensorArg), P(TensorArg), P(TensorArg), P(TensorArg),
                                                     P(TensorArg), i32, P(LaunchOpts)],
            "cutile_launch_argmax_blocks_f16": [vp, P(TensorArg), P(PartitionArg), P(PartitionArg), i32, P(LaunchOpts)],
            "cutile_launch_lm_head_argmax_blocks_f16": [vp, P(TensorArg), P(TensorArg), P(PartitionArg), P(PartitionArg), i32,
                                                        P(LaunchOpts)],
            "cutile_launch_argmax_reduce_blocks_to_u32": [vp, P(TensorArg), P(TensorArg), P(PartitionArg), i32, P(LaunchOpts)],
            "cutile_launch_embedding_batch_f16": [vp, P(TensorArg), P(TensorArg), P(PartitionArg), P(LaunchOpts)],
            "cutile_launch_gather_row_f16": [vp, P(TensorArg), P(PartitionArg), i32, P(LaunchOpts)],
            "cutile_launch_fmha_prefill_gqa_lpt_raw_f16": [vp, vp, vp, vp, vp, f32, i32, i32, i32, i32, i32, i32, i32, i32, P(LaunchOpts)],
            "cutile_launch_fmha_seq_f16": [vp, P(TensorArg), P(TensorArg), P(TensorArg), P(PartitionArg), f32, i32, i32, i32,
                                           P(TensorArg), i32, i32, P(LaunchOpts)],
            "cutile_launch_linear_tile_mxfp8": [vp, P(PartitionArg), P(TensorArg), P(TensorArg), P(TensorArg),
                                                P(TensorArg), f32, P(LaunchOpts)],
            "cutile_launch_linear_tile_nvfp4": [vp, P(PartitionArg), P(TensorArg), P(TensorArg), P(TensorArg),
                                                P(TensorArg), f32, P(LaunchOpts)],
            "cutile_partition_grid": [P(PartitionArg), P(C.c_uint32 * 3)],
            "cutile_mapped_partition_grid": [P(MappedPartitionArg), P(C.c_uint32 * 3)],
            "cutile_mapped_partition_index": [P(MappedPartitionArg), C.c_uint32, P(C.c_uint32 * 3), P(C.c_uint32)],
            "cutile_launch_gemm_persistent": [vp, P(MappedPartitionArg), P(TensorArg), P(TensorArg), P(LaunchOpts)],
            "cutile_launch_mapped_tile_index": [vp, P(MappedPartitionArg), P(LaunchOpts)],
            "cutile_mapped_partition_index_within": [P(MappedPartitionArg), P(C.c_int32), C.c_uint32, P(C.c_uint32 * 3),
                                                     P(C.c_uint32)],
            "cutile_launch_mapped_tile_index_within": [vp, P(MappedPartitionArg), P(C.c_int32), P(LaunchOpts)],
            "cutile_mapped_partitions_shared": [P(MappedPartitionArg), P(MappedPartitionArg)],
            "cutile_launch_mapped_shared_cache_update_f32": [vp, P(MappedPartitionArg), P(MappedPartitionArg), P(TensorArg), i32,
                                                             P(TensorArg), i32, i32, P(LaunchOpts)],
            "cutile_infer_launch_grid": [P(C.c_uint32 * 3), P(P(PartitionArg)), i32, P(C.c_uint32 * 3)],
            "cutile_compute_spec": [P(TensorArg), P(SpecBits)],
            "cutile_kernel_lookup": [vp, C.c_char_p, P(C.c_char_p), i32, C.c_char_p, P(KernelInfo)],
            "cutile_kernel_set_preferred_variant": [C.c_char_p, C.c_char_p],
            "cutile_kernel_list": [P(C.c_char_p), i32],
            "cutile_device_get": [i32, P(vp)],
            "cutile_device_count": [P(i32)],
            "cutile_device_name": [vp, C.c_char_p, C.c_size_t],
            "cutile_device_arch": [vp, C.c_char_p, C.c_size_t],
            "cutile_device_props": [vp, P(DeviceProps)],
            "cutile_device_bind_to_thread": [vp],
            "cutile_device_synchronize": [vp],
            "cutile_stream_create": [vp, P(vp)],
            "cutile_stream_release": [vp, vp],
            "cutile_stream_synchronize": [vp],
            "cutile_stream_query": [vp, P(i32)],
            "cutile_stream_begin_capture": [vp],
            "cutile_stream_end_capture": [vp, P(vp)],
            "cutile_graph_instantiate": [vp, P(vp)],
            "cutile_graph_upload": [vp, vp],
            "cutile_graph_launch": [vp, vp],
            "cutile_graph_exec_destroy": [vp],
            "cutile_graph_destroy": [vp],
            "cutile_event_create": [P(vp)],
            "cutile_event_record": [vp, vp],
            "cutile_event_synchronize": [vp],
            "cutile_event_elapsed_ms": [vp, vp, P(f32)],
            "cutile_event_destroy": [vp],
            "cutile_malloc_async": [C.c_size_t, vp, P(vp)],
            "cutile_free_async": [vp, vp],
            "cutile_memset_d8_async": [vp, C.c_uint8, C.c_size_t, vp],
            "cutile_memcpy_htod_async": [vp, vp, C.c_size_t, vp],
            "cutile_memcpy_dtoh_async": [vp, vp, C.c_size_t, vp],
            "cutile_memcpy_dtod_async": [vp, vp, C.c_size_t, vp],
            "cutile_testing_use_fake_hip": [i32],
            "cutile_testing_get_launch": [i32, P(LaunchRecord)],
            "cutile_testing_inject_failure": [C.c_char_p, i32, i32],
        }
        for name, argtypes in sig.items():
            if name.startswith("cutile_testing_") and not hasattr(L, name):
                continue
            fn = getattr(L, name)
            fn.argtypes = argtypes
            fn.restype = C.c_int32
        _lib = L
    return _lib


def check(status: int) -> None:
    if status != 0:
        raise CutileError(status, (lib().cutile_last_error_message() or b"").decode())


# ---- torch plumbing -------------------------------------------------------------------------
def _torch_dtype_code(t) -> int:
    import torch

    table = {torch.float32: F32, torch.float64: F64, torch.float16: F16, torch.bfloat16: BF16,
             torch.int8: I8, torch.int16: I16, torch.int32: I32, torch.int64: I64, torch.uint8: U8,
             torch.bool: BOOL}
    for name, code in (("float8_e4m3fn", F8E4M3FN), ("float8_e5m2", F8E5M2), ("float8_e8m0fnu", F8E8M0FNU),
                       ("uint16", U16), ("uint32", U32), ("uint64", U64)):
        if hasattr(torch, name):
            table[getattr(torch, name)] = code
    return table[t.dtype]


def tensor_arg(t, dtype: Optional[int] = None) -> TensorArg:
    """A torch tensor as the ABI's tensor record.  ``dtype`` overrides the element type
    (e.g. a uint8 tensor holding f8e4m3fn bytes)."""
    a = TensorArg()
    a.ptr = t.data_ptr()
    a.dtype = _torch_dtype_code(t) if dtype is None else dtype
    a.rank = t.dim()
    for i in range(t.dim()):
        a.shape[i] = t.shape[i]
        a.strides[i] = t.stride(i)
    return a


@dataclass
class Partition:
    """``tensor.partition(shape)`` of the reference (cutile/src/tensor.rs:1417-1429): a
    mutable tensor divided into disjoint tiles; its grid defines the launch grid."""
    tensor: object
    shape: Sequence[int]
    prefix: bool = False          # partition_prefix(): the grid is an upper bound only
    dtype: Optional[int] = None

    def arg(self) -> PartitionArg:
        p = PartitionArg()
        p.tensor = tensor_arg(self.tensor, self.dtype)
        rank = self.tensor.dim()
        if len(self.shape) != rank:
            raise CutileError(-5, f"partition rank {len(self.shape)} does not match tensor rank {rank}")
        for i in range(rank):
            p.partition_shape[i] = self.shape[i]
            # partition strides = tensor strides (cutile/src/tensor.rs:1423-1427)
            p.partition_strides[i] = self.tensor.stride(i)
        p.prefix_coverage = int(self.prefix)
        return p

    def grid(self):
        g = (C.c_uint32 * 3)()
        check(lib().cutile_partition_grid(C.byref(self.arg()), C.byref(g)))
        return tuple(g)


def partition(tensor, shape: Sequence[int], prefix: bool = False, dtype: Optional[int] = None) -> Partition:
    return Partition(tensor, list(shape), prefix, dtype)


OWNED = 0     # map-shape sentinel of an owned (not streamed) axis, cutile/src/tensor.rs:331-337


@dataclass
class MappedPartition:
    """``partition.map(map_shape, num_tile_blocks)`` of the reference (cutile/src/tensor.rs:314-350): the
    logical tile grid is walked by ``num_tile_blocks`` tile blocks in the order the map shape fixes."""
    partition: Partition
    map_shape: Sequence[int]
    num_tile_blocks: int

    def arg(self) -> MappedPartitionArg:
        m = MappedPartitionArg()
        m.partition = self.partition.arg()
        m.map_rank = len(self.map_shape)
        for i, d in enumerate(self.map_shape[:3]):
            m.map_shape[i] = d
        m.num_tile_blocks = self.num_tile_blocks
        return m

    def grid(self):
        """MappedLaunchPartition::validate (cutile/src/tensor.rs:352-400)"""
        g = (C.c_uint32 * 3)()
        check(lib().cutile_mapped_partition_grid(C.byref(self.arg()), C.byref(g)))
        return tuple(g)

    def num_items(self) -> int:
        idx, n = (C.c_uint32 * 3)(), C.c_uint32()
        check(lib().cutile_mapped_partition_index(C.byref(self.arg()), 0, C.byref(idx), C.byref(n)))
        return n.value

    def index(self, item: int):
        """block id per partition axis (owned axes 0) of stream item ``item``"""
        idx, n = (C.c_uint32 * 3)(), C.c_uint32()
        check(lib().cutile_mapped_partition_index(C.byref(self.arg()), int(item), C.byref(idx), C.byref(n)))
        return tuple(idx)[:self.partition.tensor.dim()]


def mapped(part: Partition, map_shape: Sequence[int], num_tile_blocks: int) -> MappedPartition:
    return MappedPartition(part, list(map_shape), int(num_tile_blocks))


def _opts(grid=None, generics=None, variant=None):
    o = LaunchOpts()
    keep = []
    if grid is not None:
        for i in range(3):
            o.grid[i] = grid[i]
    if generics is not None:
        arr = (C.c_char_p * len(generics))(*[str(g).encode() for g in generics])
        keep.append(arr)
        o.generics = C.cast(arr, C.POINTER(C.c_char_p))
        o.n_generics = len(generics)
    if variant is not None:
        o.variant = variant.encode()
    return o, keep


def _stream(stream) -> int:
    if stream is not None:
        return int(stream)
    import torch

    return torch.cuda.current_stream().cuda_stream if torch.cuda.is_available() else 0


# ---- entry launchers (reference argument order) ---------------------------------------------
def saxpy(y: Partition, a: float, x, *, stream=None, grid=None, generics=None, variant=None) -> None:
    """y <- a*x + y.  cutile-examples/examples/saxpy.rs:12-17."""
    o, _k = _opts(grid, generics, variant)
    xa = tensor_arg(x)
    check(lib().cutile_launch_saxpy(_stream(stream), C.byref(y.arg()), float(a), C.byref(xa), C.byref(o)))


def axpy(z: Partition, a: float, x, y, *, stream=None, grid=None, generics=None, variant=None) -> None:
    """z <- a*x + y (rank 1)."""
    o, _k = _opts(grid, generics, variant)
    xa, ya = tensor_arg(x), tensor_arg(y)
    check(lib().cutile_launch_axpy(_stream(stream), C.byref(z.arg()), float(a), C.byref(xa), C.byref(ya), C.byref(o)))


def add(z: Partition, x, y, *, stream=None, grid=None, generics=None, variant=None) -> None:
    """z <- x + y.  README.md:29-38 of the reference."""
    o, _k = _opts(grid, generics, variant)
    xa, ya = tensor_arg(x), tensor_arg(y)
    check(lib().cutile_launch_add(_stream(stream), C.byref(z.arg()), C.byref(xa), C.byref(ya), C.byref(o)))


def full(value, t: Partition, *, stream=None, grid=None, variant=None) -> None:
    o, _k = _opts(grid, None, variant)
    check(lib().cutile_launch_full(_stream(stream), float(value), int(value), C.byref(t.arg()), C.byref(o)))


def arange(t: Partition, *, stream=None, grid=None, variant=None) -> None:
    o, _k = _opts(grid, None, variant)
    check(lib().cutile_launch_arange(_stream(stream), C.byref(t.arg()), C.byref(o)))


def eye(t: Partition, *, stream=None, grid=None, generics=None) -> None:
    """creation::eye over [BR, BC] tiles of an f32 matrix (cutile/src/kernels/_creation.rs:110-138)"""
    o, _k = _opts(grid, generics, None)
    check(lib().cutile_launch_eye(_stream(stream), C.byref(t.arg()), C.byref(o)))


def relu(input_output: Partition, *, stream=None, grid=None, generics=None) -> None:
    """cutile-examples/examples/async_mlp.rs:56-61: max(0, x) in place over [D] tiles of an f32 vector"""
    o, _k = _opts(grid, generics, None)
    check(lib().cutile_launch_relu(_stream(stream), C.byref(input_output.arg()), C.byref(o)))


def dropout(p: float, x, x_keep, out: Partition, *, stream=None, grid=None, generics=None) -> None:
    """cutile-examples/examples/dropout.rs:17-32: out = select(x_keep > p, x_keep, 0) / (1 - p); x is never read"""
    o, _k = _opts(grid, generics, None)
    xa, ka = tensor_arg(x), tensor_arg(x_keep)
    check(lib().cutile_launch_dropout(_stream(stream), float(p), C.byref(xa), C.byref(ka), C.byref(out.arg()), C.byref(o)))


def scale_ptr(out_ptr: int, in_ptr: int, scale: float, length: int, *, stream=None, grid=None) -> None:
    """cutile-examples/examples/scale_ptr.rs:26-80: out[i] = in[i] * scale for i < length on raw device pointers (f32);
    the launch grid is required, as for every launcher without a partition argument"""
    o, _k = _opts(grid, None, None)
    check(lib().cutile_launch_scale_ptr(_stream(stream), C.c_void_p(out_ptr), C.c_void_p(in_ptr), float(scale), int(length),
                                        C.byref(o)))


def matvec(z: Partition, x, y, k: int, *, stream=None, grid=None, generics=None) -> None:
    """cutile-examples/examples/async_mlp.rs:38-54: z[r] += sum_k x[r, k] * y[k] over [BM] tiles of z (f32)"""
    o, _k = _opts(grid, generics, None)
    xa, ya = tensor_arg(x), tensor_arg(y)
    check(lib().cutile_launch_matvec(_stream(stream), C.byref(z.arg()), C.byref(xa), C.byref(ya), int(k), C.byref(o)))


def batch_matmul(c: Partition, a, b, k: int, *, stream=None, grid=None, generics=None, variant=None) -> None:
    """cutile-examples/examples/batch_matmul.rs:16-44: c[p] = a[p] . b[p] over [1, BM, BN] tiles of c"""
    o, _k = _opts(grid, generics, variant)
    aa, ba = tensor_arg(a), tensor_arg(b)
    check(lib().cutile_launch_batch_matmul(_stream(stream), C.byref(c.arg()), C.byref(aa), C.byref(ba), int(k), C.byref(o)))


def linspace(t: Partition, start: float, step: float, *, stream=None, grid=None) -> None:
    o, _k = _opts(grid, None, None)
    check(lib().cutile_launch_linspace(_stream(stream), C.byref(t.arg()), float(start), float(step), C.byref(o)))


def convert(src, dst: Partition, *, stream=None, grid=None) -> None:
    o, _k = _opts(grid, None, None)
    sa = tensor_arg(src)
    check(lib().cutile_launch_convert(_stream(stream), C.byref(sa), C.byref(dst.arg()), C.byref(o)))


def rms_norm_f16(x, w, out: Partition, eps: float, *, stream=None, grid=None, generics=None, variant=None) -> None:
    """cutile-kernels/src/norms.rs:16-60."""
    o, _k = _opts(grid, generics, variant)
    xa, wa = tensor_arg(x), tensor_arg(w)
    check(lib().cutile_launch_rms_norm_f16(_stream(stream), C.byref(xa), C.byref(wa), C.byref(out.arg()), float(eps),
                                           C.byref(o)))


def rms_norm_f32(x, w, out: Partition, eps: float, *, stream=None, grid=None, generics=None, variant=None) -> None:
    """the f32 example form, cutile-examples/examples/rms_norm.rs:17-61 (square root rounded toward minus infinity)"""
    o, _k = _opts(grid, generics, variant)
    xa, wa = tensor_arg(x), tensor_arg(w)
    check(lib().cutile_launch_rms_norm_f32(_stream(stream), C.byref(xa), C.byref(wa), C.byref(out.arg()), float(eps),
                                           C.byref(o)))


def rms_norm_all_f16(x, w, out: Partition, eps: float, *, generics, stream=None, grid=None) -> None:
    """cutile-benchmarks/benches/rmsnorm.rs:20-66: every operation in f16; generics = [N, BLOCK_SIZE]."""
    o, _k = _opts(grid, generics, None)
    xa, wa = tensor_arg(x), tensor_arg(w)
    check(lib().cutile_launch_rms_norm_all_f16(_stream(stream), C.byref(xa), C.byref(wa), C.byref(out.arg()), float(eps),
                                               C.byref(o)))


def softmax_all_f16(x, y: Partition, *, stream=None, grid=None, generics=None) -> None:
    """cutile-benchmarks/benches/softmax.rs:19-35 with its own arithmetic: every operation in f16."""
    o, _k = _opts(grid, generics, None)
    xa = tensor_arg(x)
    check(lib().cutile_launch_softmax_all_f16(_stream(stream), C.byref(xa), C.byref(y.arg()), C.byref(o)))


def softmax(x, y: Partition, *, stream=None, grid=None, generics=None, variant=None) -> None:
    """cutile-benchmarks/benches/softmax.rs:19-35."""
    o, _k = _opts(grid, generics, variant)
    xa = tensor_arg(x)
    check(lib().cutile_launch_softmax(_stream(stream), C.byref(xa), C.byref(y.arg()), C.byref(o)))


def add_rms_norm_f16(residual, x, w, out: Partition, residual_out: Partition, eps: float, *, stream=None, grid=None,
                     generics=None, variant=None) -> None:
    """combined = residual + x; out = RMSNorm(combined) * w; residual_out = combined (cutile-kernels norms.rs:68-136)"""
    ra, xa, wa = tensor_arg(residual), tensor_arg(x), tensor_arg(w)
    o, keep = _opts(grid, generics, variant)
    check(lib().cutile_launch_add_rms_norm_f16(_stream(stream), C.byref(ra), C.byref(xa), C.byref(wa), C.byref(out.arg()),
                                               C.byref(residual_out.arg()), C.c_float(eps), C.byref(o)))


def qk_norm_f16(q, k, q_weight, k_weight, out: Partition, eps: float, num_q_rows: int, *, stream=None, grid=None,
                generics=None, variant=None) -> None:
    """rows < num_q_rows of out: RMSNorm(q) * q_weight; the rest: RMSNorm(k) * k_weight (norms.rs:143-216)"""
    qa, ka, qw, kw = tensor_arg(q), tensor_arg(k), tensor_arg(q_weight), tensor_arg(k_weight)
    o, keep = _opts(grid, generics, variant)
    check(lib().cutile_launch_qk_norm_f16(_stream(stream), C.byref(qa), C.byref(ka), C.byref(qw), C.byref(kw),
                                          C.byref(out.arg()), C.c_float(eps), int(num_q_rows), C.byref(o)))


def add_2d_f16(out: Partition, lhs, rhs, *, stream=None, grid=None, generics=None, variant=None) -> None:
    la, ra = tensor_arg(lhs), tensor_arg(rhs)
    o, keep = _opts(grid, generics, variant)
    check(lib().cutile_launch_add_2d_f16(_stream(stream), C.byref(out.arg()), C.byref(la), C.byref(ra), C.byref(o)))


def silu_mul_2d_f16(out: Partition, gate, up, *, stream=None, grid=None, generics=None, variant=None) -> None:
    """out = sigmoid(gate) * gate * up (pointwise.rs:46-78)"""
    ga, ua = tensor_arg(gate), tensor_arg(up)
    o, keep = _opts(grid, generics, variant)
    check(lib().cutile_launch_silu_mul_2d_f16(_stream(stream), C.byref(out.arg()), C.byref(ga), C.byref(ua), C.byref(o)))


def rope_f16(out: Partition, x, inv_freq, position_start=0, *, k=None, num_q_heads: int = 0, stream=None, grid=None,
             generics=None) -> None:
    """Rotary embedding (positional.rs).  `position_start` is an int (rope_seq_f16) or a one-element
    uint32/int32 device tensor (the dynpos forms); with `k`, heads >= num_q_heads of out come from k."""
    xa, fa = tensor_arg(x), tensor_arg(inv_freq)
    ka = tensor_arg(k) if k is not None else None
    pos_dev = None
    pos = 0
    if isinstance(position_start, int):
        pos = position_start
    else:
        pos_dev = tensor_arg(position_start, dtype=U32)
    o, keep = _opts(grid, generics, None)
    check(lib().cutile_launch_rope_f16(_stream(stream), C.byref(xa), C.byref(ka) if ka is not None else None, C.byref(fa),
                                       C.byref(pos_dev) if pos_dev is not None else None, int(pos), C.byref(out.arg()),
                                       int(num_q_heads), C.byref(o)))


def kv_cache_update_f16(new_k, new_v, k_cache: Partition, v_cache: Partition, position_start, seq_len: int, *, stream=None,
                        grid=None, generics=None) -> None:
    """cache[h, position_start + s] = new[s, h] (kv_cache.rs); position_start: int or one-element device tensor"""
    ka, va = tensor_arg(new_k), tensor_arg(new_v)
    pos_dev, pos = (None, int(position_start)) if isinstance(position_start, int) else (tensor_arg(position_start, dtype=U32), 0)
    o, keep = _opts(grid, generics, None)
    check(lib().cutile_launch_kv_cache_update_f16(_stream(stream), C.byref(ka), C.byref(va), C.byref(k_cache.arg()),
                                                  C.byref(v_cache.arg()), C.byref(pos_dev) if pos_dev is not None else None,
                                                  pos, int(seq_len), C.byref(o)))


def fmha_decode_gqa_split(q, k, v, att_out: Partition, lse_out: Partition, qk_scale: float, position_start, *, stream=None,
                          grid=None, generics=None, variant=None) -> None:
    """split-KV decode attention (attention.rs:737-902); position_start: one-element device tensor"""
    qa, ka, va, pa = tensor_arg(q), tensor_arg(k), tensor_arg(v), tensor_arg(position_start, dtype=U32)
    o, keep = _opts(grid, generics, variant)
    check(lib().cutile_launch_fmha_decode_gqa_split(_stream(stream), C.byref(qa), C.byref(ka), C.byref(va),
                                                    C.byref(att_out.arg()), C.byref(lse_out.arg()), C.c_float(qk_scale),
                                                    C.byref(pa), C.byref(o)))


def attention_decode_kernel_grouped_f16(q, k, v, att, lse, softmax_scale: float, s_kv, *, tile_n: int = 64,
                                        kv_len_per_split: int, query_group_tile_size=None, stream=None, grid=None,
                                        generics=None) -> None:
    """experimental/attention.rs:385-846 on device tensors: q [B, H_kv, G, D], k and v [B, H_kv, S, D],
    att [B, H_kv, G, splits, D], lse [B, H_kv, G, splits] (f32), s_kv one int32 in device memory."""
    def group(t, rank):
        if t.dim() != rank or t.stride(-1) != 1:
            raise ValueError(f"attention_decode_kernel_grouped: expected rank {rank} with unit innermost stride")
        return (C.c_void_p(t.data_ptr()), (C.c_int32 * rank)(*t.shape), (C.c_int32 * (rank - 1))(*t.stride()[:-1]))
    o, keep = _opts(grid, generics, None)
    qgts = int(query_group_tile_size) if query_group_tile_size is not None else max(int(q.shape[2]), 1)
    check(lib().cutile_launch_attention_decode_kernel_grouped_f16(
        _stream(stream), *group(q, 4), *group(k, 4), *group(v, 4), *group(att, 5), *group(lse, 4), C.c_float(softmax_scale),
        C.c_void_p(s_kv.data_ptr()), int(tile_n), int(kv_len_per_split), qgts, C.byref(o)))


def splitk_reduce_merge(att_partial, lse_partial, out: Partition, *, stream=None, grid=None, generics=None) -> None:
    aa, la = tensor_arg(att_partial), tensor_arg(lse_partial)
    o, keep = _opts(grid, generics, None)
    check(lib().cutile_launch_splitk_reduce_merge(_stream(stream), C.byref(aa), C.byref(la), C.byref(out.arg()), C.byref(o)))


def fmha_decode_gqa_noalloc(q, k, v, out: Partition, qk_scale: float, position_start, num_kv_splits: int, bn: int = 64, *,
                            stream=None) -> None:
    """split-KV decode attention and merge in one call that allocates nothing: the partial results live in the
    library's device-resident scratch array (8 MiB per GPU); position_start: one-element device tensor"""
    qa, ka, va, pa = tensor_arg(q), tensor_arg(k), tensor_arg(v), tensor_arg(position_start, dtype=U32)
    check(lib().cutile_launch_fmha_decode_gqa_noalloc(_stream(stream), C.byref(qa), C.byref(ka), C.byref(va),
                                                      C.byref(out.arg()), C.c_float(qk_scale), C.byref(pa),
                                                      int(num_kv_splits), int(bn)))


def fmha_decode_gqa_noalloc_prepare(q, k, v, out: Partition, position_start, num_kv_splits: int, bn: int = 64) -> None:
    """the once-per-device-and-shape work of fmha_decode_gqa_noalloc (side library, scratch address, code objects) done
    ahead of time, outside any stream capture; nothing is enqueued"""
    qa, ka, va, pa = tensor_arg(q), tensor_arg(k), tensor_arg(v), tensor_arg(position_start, dtype=U32)
    check(lib().cutile_fmha_decode_gqa_noalloc_prepare(C.byref(qa), C.byref(ka), C.byref(va), C.byref(out.arg()), C.byref(pa),
                                                       int(num_kv_splits), int(bn)))


def scratch_capacity() -> int:
    n = C.c_size_t(0)
    check(lib().cutile_scratch_capacity(C.byref(n)))
    return int(n.value)


def gemm(z: Partition, x, y, k: int, *, accumulate: bool = True, stream=None, grid=None, generics=None,
         variant=None) -> None:
    """cutile-benchmarks/benches/gemm.rs:20-41 (z is read as the initial accumulator)."""
    o, _k = _opts(grid, generics, variant)
    xa, ya = tensor_arg(x), tensor_arg(y)
    check(lib().cutile_launch_gemm(_stream(stream), C.byref(z.arg()), C.byref(xa), C.byref(ya), int(k),
                                   int(accumulate), C.byref(o)))


def gemm_persistent(z: MappedPartition, x, y, *, stream=None, grid=None, generics=None, variant=None) -> None:
    """cutile-examples/examples/persistent_gemm.rs:35-59: z <- x . y, tiles walked by z.num_tile_blocks tile blocks."""
    o, _k = _opts(grid, generics, variant)
    xa, ya = tensor_arg(x), tensor_arg(y)
    check(lib().cutile_launch_gemm_persistent(_stream(stream), C.byref(z.arg()), C.byref(xa), C.byref(ya), C.byref(o)))


def _ranges(z: MappedPartition, ranges):
    flat = [int(v) for pair in ranges for v in pair]
    if len(flat) != 2 * len(z.map_shape):
        raise ValueError(f"sub-range iteration expects {len(z.map_shape)} (start_tile, num_tiles) pairs, got {len(ranges)}")
    return (C.c_int32 * len(flat))(*flat)


def mapped_indices_within(z: MappedPartition, ranges):
    """the block ids of ``for index in z.iter_indices_within(ranges)`` in stream order (cutile/src/_core.rs:912-930)"""
    r, n, idx = _ranges(z, ranges), C.c_uint32(0), (C.c_uint32 * 3)()
    check(lib().cutile_mapped_partition_index_within(C.byref(z.arg()), r, 0, None, C.byref(n)))
    out = []
    for t in range(n.value):
        check(lib().cutile_mapped_partition_index_within(C.byref(z.arg()), r, t, idx, None))
        out.append(tuple(idx)[:len(z.map_shape)])
    return out


def mapped_tile_index_within(z: MappedPartition, ranges, *, stream=None, grid=None) -> None:
    """only the tiles inside ``ranges`` receive their row-major index in the whole logical grid
    (cutile/tests/gpu/mapped_partition_schedule_matrix.rs:75-106)"""
    o, _k = _opts(grid, None, None)
    check(lib().cutile_launch_mapped_tile_index_within(_stream(stream), C.byref(z.arg()), _ranges(z, ranges), C.byref(o)))


def mapped_partitions_shared(a: MappedPartition, b: MappedPartition) -> None:
    """the checks of ``a.iter_indices_with(&b)`` (cutile/src/_core.rs:904-911); raises CutileError when they fail"""
    check(lib().cutile_mapped_partitions_shared(C.byref(a.arg()), C.byref(b.arg())))


def mapped_shared_cache_update_f32(k_cache: MappedPartition, v_cache: MappedPartition, new_k, n_tiles: int, *, start_tile: int = 0,
                                   position=None, source_seq_major: bool = False, stream=None, grid=None) -> None:
    """dynpos_shared_rank3 / prefill_shared_rank3 of cutile/tests/gpu/mapped_partition_schedule_matrix.rs:107-153"""
    o, _k = _opts(grid, None, None)
    na = tensor_arg(new_k)
    pa = tensor_arg(position) if position is not None else None
    check(lib().cutile_launch_mapped_shared_cache_update_f32(
        _stream(stream), C.byref(k_cache.arg()), C.byref(v_cache.arg()), C.byref(na), int(source_seq_major),
        C.byref(pa) if pa is not None else None, int(start_tile), int(n_tiles), C.byref(o)))


def mapped_tile_index(z: MappedPartition, *, stream=None, grid=None) -> None:
    """every tile of the i32 tensor receives its row-major index in the logical grid
    (cutile/tests/gpu/mapped_partition_schedule_matrix.rs:30-76)"""
    o, _k = _opts(grid, None, None)
    check(lib().cutile_launch_mapped_tile_index(_stream(stream), C.byref(z.arg()), C.byref(o)))


def fmha(out: Partition, q, k, v, qk_scale: float, input_pos: int = 0, query_group_size: int = 1, *,
         causal: bool = False, stream=None, grid=None, generics=None, variant=None) -> None:
    """cutile-examples/examples/flash_attention_causal.rs:19-134."""
    o, _k = _opts(grid, generics, variant)
    qa, ka, va = tensor_arg(q), tensor_arg(k), tensor_arg(v)
    check(lib().cutile_launch_fmha(_stream(stream), C.byref(out.arg()), C.byref(qa), C.byref(ka), C.byref(va),
                                   float(qk_scale), int(input_pos), int(query_group_size), int(causal), C.byref(o)))


KVBM_STACKED_NHD, KVBM_STACKED_HND = 0, 1
KVBM_OPERATIONAL_NHD, KVBM_OPERATIONAL_HND, KVBM_UNIVERSAL = 0, 1, 2


def kvbm_copy_f16(to_stacked: bool, stacked_layout: int, contiguous_layout: int, num_blocks: int, stacked_tensors, contiguous_tensors,
                  nh: int, nl: int, no: int, nt: int, hd: int, *, stream=None) -> None:
    """copy_stacked_to_contiguous_f16 / copy_contiguous_to_stacked_f16 (cutile-kernels/src/experimental/kvbm.rs:112-352);
    the tables are int64 device tensors of tensor addresses"""
    sa, ca = tensor_arg(stacked_tensors), tensor_arg(contiguous_tensors)
    o, _k = _opts(None, None, None)
    fn = lib().cutile_launch_copy_contiguous_to_stacked_f16 if to_stacked else lib().cutile_launch_copy_stacked_to_contiguous_f16
    check(fn(_stream(stream), int(stacked_layout), int(contiguous_layout), int(num_blocks), C.byref(sa), C.byref(ca), int(nh), int(nl),
             int(no), int(nt), int(hd), C.byref(o)))


def add_rms_norm_decode_raw_f16(residual, x, w, out, residual_out, eps: float, *, stream=None, generics=None) -> None:
    """cutile-kernels/src/experimental/norms.rs:22-153: one row of N halves, the tensors' addresses passed as raw pointers"""
    o, _k = _opts(None, generics, None)
    check(lib().cutile_launch_add_rms_norm_decode_raw_f16(_stream(stream), *[C.c_void_p(t.data_ptr()) for t in (residual, x, w, out, residual_out)],
                                                          C.c_float(eps), int(w.numel()), C.byref(o)))


def qk_norm_rope_kv_prefill_raw_f16(q, k, v, q_weight, k_weight, inv_freq, q_out, k_cache, v_cache, eps: float, position_start: int,
                                    seq_len: int, *, stream=None, generics=None) -> None:
    """cutile-kernels/src/experimental/fused_transformer.rs:22-345; the reference takes raw pointers, this wrapper takes the
    contiguous tensors q [seq, q_heads, D], k / v [seq, kv_heads, D], caches [kv_heads, MAX_SEQ, D] and passes their addresses"""
    o, _k = _opts(None, generics, None)
    for t in (q, k, v, q_weight, k_weight, inv_freq, q_out, k_cache, v_cache):
        if not t.is_contiguous():
            raise CutileError(-5, "qk_norm_rope_kv_prefill_raw_f16: raw-pointer kernel, every tensor must be contiguous")
    check(lib().cutile_launch_qk_norm_rope_kv_prefill_raw_f16(
        _stream(stream), *[C.c_void_p(t.data_ptr()) for t in (q, k, v, q_weight, k_weight, inv_freq, q_out, k_cache, v_cache)],
        C.c_float(eps), int(position_start), int(seq_len), int(q.shape[1]), int(k.shape[1]), int(q.shape[2]), int(k_cache.shape[1]),
        C.byref(o)))


def qk_norm_rope_kv_decode_raw_f16(qkv, q_weight, k_weight, inv_freq, q_out, k_cache, v_cache, position_start, eps: float,
                                   num_q_heads: int, num_kv_heads: int, *, stream=None, generics=None) -> None:
    """cutile-kernels/src/experimental/fused_transformer.rs:356-625; qkv: one token's q, k and v heads back to back"""
    o, _k = _opts(None, generics, None)
    pa = tensor_arg(position_start, dtype=U32)
    d = int(k_cache.shape[2])
    check(lib().cutile_launch_qk_norm_rope_kv_decode_raw_f16(
        _stream(stream), *[C.c_void_p(t.data_ptr()) for t in (qkv, q_weight, k_weight, inv_freq, q_out, k_cache, v_cache)],
        C.byref(pa), C.c_float(eps), int(num_q_heads), int(num_kv_heads), d, int(k_cache.shape[1]), C.byref(o)))


def group_gemm_f16_nt_desc(a_ptrs, b_ptrs, c_ptrs, a_metas, b_metas, c_metas, num_groups: int, *, stream=None, grid=None,
                           generics=None, variant=None) -> None:
    """cutile-kernels/src/experimental/moe.rs:67-128: pointer tables (int64) and descriptor tables (int32 [groups, 8]:
    rows, cols, row stride) in device memory; generics [BM, BN, BK, NUM_SM]"""
    o, _k = _opts(grid, generics, variant)
    t = [tensor_arg(x) for x in (a_ptrs, b_ptrs, c_ptrs, a_metas, b_metas, c_metas)]
    check(lib().cutile_launch_group_gemm_f16_nt_desc(_stream(stream), *[C.byref(x) for x in t], int(num_groups), C.byref(o)))


def _u32_partition(p: Partition) -> PartitionArg:
    """the argument record of a partition of u32 values held in an int32 / uint32 tensor"""
    return (p if p.dtype is not None else Partition(p.tensor, p.shape, p.prefix, U32)).arg()


def argmax_blocks_f16(logits, block_max: Partition, block_idx: Partition, length: int, *, stream=None, grid=None, generics=None) -> None:
    """cutile-kernels/src/argmax.rs:21-71; block_idx: an int32 / uint32 tensor of u32 indices"""
    o, _k = _opts(grid, generics, None)
    la = tensor_arg(logits)
    check(lib().cutile_launch_argmax_blocks_f16(_stream(stream), C.byref(la), C.byref(block_max.arg()), C.byref(_u32_partition(block_idx)),
                                                int(length), C.byref(o)))


def lm_head_argmax_blocks_f16(weights, hidden, block_max: Partition, block_idx: Partition, vocab_size: int, *, stream=None,
                              grid=None, generics=None) -> None:
    """cutile-kernels/src/argmax.rs:88-158"""
    o, _k = _opts(grid, generics, None)
    wa, ha = tensor_arg(weights), tensor_arg(hidden)
    check(lib().cutile_launch_lm_head_argmax_blocks_f16(_stream(stream), C.byref(wa), C.byref(ha), C.byref(block_max.arg()),
                                                        C.byref(_u32_partition(block_idx)), int(vocab_size), C.byref(o)))


def argmax_reduce_blocks_to_u32(block_max, block_idx, out: Partition, num_blocks: int, *, stream=None, grid=None, generics=None) -> None:
    """cutile-kernels/src/argmax.rs:173-213"""
    o, _k = _opts(grid, generics, None)
    ma, ia = tensor_arg(block_max), tensor_arg(block_idx, dtype=U32)
    check(lib().cutile_launch_argmax_reduce_blocks_to_u32(_stream(stream), C.byref(ma), C.byref(ia), C.byref(_u32_partition(out)),
                                                          int(num_blocks), C.byref(o)))


def embedding_batch_f16(token_ids, table, out: Partition, *, stream=None, grid=None, generics=None) -> None:
    """cutile-kernels/src/embeddings.rs:21-41; token_ids: an int32 / uint32 tensor of u32 ids"""
    o, _k = _opts(grid, generics, None)
    ia, ta = tensor_arg(token_ids, dtype=U32), tensor_arg(table)
    check(lib().cutile_launch_embedding_batch_f16(_stream(stream), C.byref(ia), C.byref(ta), C.byref(out.arg()), C.byref(o)))


def gather_row_f16(src, out: Partition, row_idx: int, *, stream=None, grid=None, generics=None) -> None:
    """cutile-kernels/src/pointwise.rs:86-99"""
    o, _k = _opts(grid, generics, None)
    sa = tensor_arg(src)
    check(lib().cutile_launch_gather_row_f16(_stream(stream), C.byref(sa), C.byref(out.arg()), int(row_idx), C.byref(o)))


def fmha_seq_f16(q, k, v, out: Partition, qk_scale: float, query_group_size: int, *, kv_len: int = 0, query_start: int = 0,
                 position_start=None, kv_len_from_position: bool = False, causal: bool = True, stream=None, grid=None,
                 generics=None, variant=None) -> None:
    """The sequence-layout attention kernels of cutile-kernels/src/attention.rs (q, out [q_len, q_heads, D]; k, v
    [kv_heads, max_seq, D]; out tiles [BM, G, D]):
      flash_attn_causal_seq_f16 (:21-116)         kv_len, query_start by value, causal
      flash_attn_causal_seq_dynpos_f16 (:128-231) position_start (one u32 on the device), kv_len_from_position
      fmha_prefill_causal (:242-391), fmha_prefill_gqa (:408-587)   kv_len, query_start by value, causal or not
      fmha_causal (:598-726)                      position_start, every key of k"""
    o, _k = _opts(grid, generics, variant)
    qa, ka, va = tensor_arg(q), tensor_arg(k), tensor_arg(v)
    pa = tensor_arg(position_start, dtype=U32) if position_start is not None else None
    check(lib().cutile_launch_fmha_seq_f16(_stream(stream), C.byref(qa), C.byref(ka), C.byref(va), C.byref(out.arg()),
                                           C.c_float(qk_scale), int(query_group_size), int(kv_len), int(query_start),
                                           C.byref(pa) if pa is not None else None, int(kv_len_from_position), int(causal),
                                           C.byref(o)))


def fmha_prefill_gqa_lpt_raw_f16(q, k, v, out, qk_scale: float, query_group_size: int, kv_len: int, query_start: int, group: int, *,
                                 causal: bool = True, stream=None, generics=None) -> None:
    """cutile-kernels/src/experimental/attention.rs:22-377; contiguous q / out [q_len, q_heads, D] and k / v [kv_heads, kv_len, D]
    passed as raw addresses"""
    o, _k = _opts(None, generics, None)
    check(lib().cutile_launch_fmha_prefill_gqa_lpt_raw_f16(
        _stream(stream), *[C.c_void_p(t.data_ptr()) for t in (q, k, v, out)], C.c_float(qk_scale), int(query_group_size), int(q.shape[0]),
        int(kv_len), int(query_start), int(q.shape[1]) // int(group), int(group), int(q.shape[2]), int(causal), C.byref(o)))


def linear_tile_mxfp8(z: Partition, x, y, x_scales, y_scales, alpha: float = 1.0, *, stream=None, grid=None,
                      generics=None, variant=None) -> None:
    """cutile-examples/examples/mxfp8.rs:34-64.  x, y: uint8 (or float8_e4m3fn) tensors of
    e4m3fn bytes; scales: uint8 (or float8_e8m0fnu) tensors of e8m0 bytes."""
    o, _k = _opts(grid, generics, variant)
    xa, ya = tensor_arg(x, F8E4M3FN), tensor_arg(y, F8E4M3FN)
    xsa, ysa = tensor_arg(x_scales, F8E8M0FNU), tensor_arg(y_scales, F8E8M0FNU)
    check(lib().cutile_launch_linear_tile_mxfp8(_stream(stream), C.byref(z.arg()), C.byref(xa), C.byref(ya),
                                                C.byref(xsa), C.byref(ysa), float(alpha), C.byref(o)))


def linear_tile_nvfp4(z: Partition, x, y, x_scales, y_scales, alpha: float = 1.0, *, stream=None, grid=None,
                      generics=None, variant=None) -> None:
    """cutile-examples/examples/nvfp4.rs:24-78.  x [M, K/2], y [N, K/2]: uint8 tensors of packed e2m1 pairs (low
    nibble first); scales [M, K/16], [N, K/16]: uint8 (or float8_e4m3fn) tensors of e4m3fn bytes; z f32 or bf16."""
    o, _k = _opts(grid, generics, variant)
    xa, ya = tensor_arg(x, F4E2M1FNX2), tensor_arg(y, F4E2M1FNX2)
    xsa, ysa = tensor_arg(x_scales, F8E4M3FN), tensor_arg(y_scales, F8E4M3FN)
    check(lib().cutile_launch_linear_tile_nvfp4(_stream(stream), C.byref(z.arg()), C.byref(xa), C.byref(ya),
                                                C.byref(xsa), C.byref(ysa), float(alpha), C.byref(o)))


# ---- table / device helpers -------------------------------------------------------------------
def kernel_list() -> list[str]:
    n = lib().cutile_kernel_list(None, 0)
    arr = (C.c_char_p * n)()
    lib().cutile_kernel_list(arr, n)
    return [a.decode() for a in arr]


def set_preferred_variant(function: str, variant: Optional[str]) -> None:
    check(lib().cutile_kernel_set_preferred_variant(function.encode(), variant.encode() if variant else None))


def set_preferred_variant_for(function: str, bucket: str, variant: Optional[str]) -> None:
    check(lib().cutile_kernel_set_preferred_variant_for(function.encode(), bucket.encode(), variant.encode() if variant else None))


def tuning_reload(directory: Optional[str] = None) -> str:
    """drop the applied tuning records and load `directory` (None = the directory beside the library); returns the report"""
    check(lib().cutile_tuning_reload(directory.encode() if directory is not None else None))
    return tuning_report()


def tuning_report() -> str:
    L = lib()
    L.cutile_tuning_report.restype = C.c_char_p
    return L.cutile_tuning_report().decode()


def last_resolved() -> dict:
    """what the calling thread's last launcher call resolved: kernel, variant, where the choice came from, its shape class"""
    L = lib()
    L.cutile_last_resolved_source.restype = C.c_char_p
    L.cutile_last_resolved_bucket.restype = C.c_char_p
    fn = C.c_char_p()
    info = KernelInfo()
    check(L.cutile_last_resolved_kernel(C.byref(fn), C.byref(info)))
    return {"function": fn.value.decode(), "variant": info.variant.decode(), "symbol": info.symbol.decode(),
            "source": L.cutile_last_resolved_source().decode(), "bucket": L.cutile_last_resolved_bucket().decode()}


def kernel_fingerprint(function: str, variant: Optional[str] = None) -> str:
    buf = C.create_string_buffer(17)
    check(lib().cutile_kernel_fingerprint(function.encode(), variant.encode() if variant else None, buf))
    return buf.value.decode()


def device(ordinal: int = 0) -> int:
    d = C.c_void_p()
    check(lib().cutile_device_get(ordinal, C.byref(d)))
    return d.value


def device_props(ordinal: int = 0) -> DeviceProps:
    p = DeviceProps()
    check(lib().cutile_device_props(device(ordinal), C.byref(p)))
    return p


def device_arch(ordinal: int = 0) -> str:
    buf = C.create_string_buffer(256)
    check(lib().cutile_device_arch(device(ordinal), buf, 256))
    return buf.value.decode()


def kernel_lookup(function: str, generics: Sequence[str] = (), variant: Optional[str] = None,
                  ordinal: int = 0) -> KernelInfo:
    info = KernelInfo()
    arr = (C.c_char_p * max(1, len(generics)))(*[str(g).encode() for g in generics])
    check(lib().cutile_kernel_lookup(device(ordinal), function.encode(), arr, len(generics),
                                     variant.encode() if variant else None, C.byref(info)))
    return info


class Rng:
    """Device random fills through the C ABI (cuda-core/src/api.rs:214-293): Philox4x32-10; `seed=None` keeps seed 0."""

    def __init__(self, seed: Optional[int] = None):
        self.handle = C.c_void_p()
        L = lib()
        vp, sz, u64 = C.c_void_p, C.c_size_t, C.c_uint64
        L.cutile_rng_create.argtypes = [C.POINTER(vp)]
        L.cutile_rng_set_seed.argtypes = [vp, u64]
        L.cutile_rng_set_offset.argtypes = [vp, u64]
        L.cutile_rng_get_offset.argtypes = [vp, C.POINTER(u64)]
        L.cutile_rng_normal_f32.argtypes = [vp, vp, sz, C.c_float, C.c_float, vp]
        L.cutile_rng_normal_f64.argtypes = [vp, vp, sz, C.c_double, C.c_double, vp]
        L.cutile_rng_uniform_f32.argtypes = [vp, vp, sz, vp]
        L.cutile_rng_uniform_f64.argtypes = [vp, vp, sz, vp]
        L.cutile_rng_destroy.argtypes = [vp]
        check(L.cutile_rng_create(C.byref(self.handle)))
        if seed is not None:
            check(L.cutile_rng_set_seed(self.handle, seed))

    def set_seed(self, seed: int) -> None:
        check(lib().cutile_rng_set_seed(self.handle, seed))

    @property
    def offset(self) -> int:
        v = C.c_uint64()
        check(lib().cutile_rng_get_offset(self.handle, C.byref(v)))
        return int(v.value)

    @offset.setter
    def offset(self, value: int) -> None:
        check(lib().cutile_rng_set_offset(self.handle, value))

    def _fill(self, t, kind, mean, std, stream):
        import torch

        if not t.is_contiguous() or t.dtype not in (torch.float32, torch.float64):
            raise ValueError("Rng fills take contiguous f32 or f64 tensors")
        L, f32 = lib(), t.dtype == torch.float32
        ptr, n, st = C.c_void_p(t.data_ptr()), t.numel(), _stream(stream)
        if kind == "normal":
            check((L.cutile_rng_normal_f32 if f32 else L.cutile_rng_normal_f64)(self.handle, ptr, n, mean, std, st))
        else:
            check((L.cutile_rng_uniform_f32 if f32 else L.cutile_rng_uniform_f64)(self.handle, ptr, n, st))

    def normal_(self, t, mean: float = 0.0, std: float = 1.0, *, stream=None) -> None:
        self._fill(t, "normal", mean, std, stream)

    def uniform_(self, t, *, stream=None) -> None:
        self._fill(t, "uniform", 0.0, 1.0, stream)

    def close(self) -> None:
        if self.handle:
            lib().cutile_rng_destroy(self.handle)
            self.handle = C.c_void_p()


class Module:
    """A code object loaded through the driver layer of the C ABI (cuda-core/src/runtime.rs:309-328, 828-835) and
    launched with a parameter array (cuda-core/src/api.rs:48-70)."""

    def __init__(self, image: bytes, ordinal: int = 0):
        self.handle = C.c_void_p()
        self._image = image
        L = lib()
        L.cutile_module_load_data.argtypes = [C.c_void_p, C.c_char_p, C.c_size_t, C.POINTER(C.c_void_p)]
        L.cutile_module_get_function.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_void_p)]
        L.cutile_launch_kernel.argtypes = [C.c_void_p, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.c_uint32, C.c_void_p,
                                           C.POINTER(C.c_void_p)]
        L.cutile_module_unload.argtypes = [C.c_void_p]
        check(L.cutile_module_load_data(device(ordinal), image, len(image), C.byref(self.handle)))

    def function(self, name: str) -> int:
        f = C.c_void_p()
        check(lib().cutile_module_get_function(self.handle, name.encode(), C.byref(f)))
        return f.value

    @staticmethod
    def launch(function: int, grid, block, params, *, shared_mem_bytes: int = 0, stream=None) -> None:
        """params: ctypes values in the kernel's signature order"""
        ptrs = (C.c_void_p * max(1, len(params)))(*[C.cast(C.pointer(p), C.c_void_p) for p in params])
        check(lib().cutile_launch_kernel(function, (C.c_uint32 * 3)(*grid), (C.c_uint32 * 3)(*block), shared_mem_bytes,
                                         _stream(stream), ptrs))

    def close(self) -> None:
        if self.handle:
            lib().cutile_module_unload(self.handle)
            self.handle = C.c_void_p()


class CapturedGraph:
    """Stream capture and replay through the C ABI (cuda-async/src/cuda_graph.rs:61-244): the launches `record` issues on
    this object's stream are captured once and replayed with one call per step.

        g = CapturedGraph().capture(lambda stream: (ct.saxpy(..., stream=stream), ct.add(..., stream=stream)))
        g.launch(); g.synchronize()
    """

    def __init__(self, device: int = 0):
        self.device, self.stream, self.graph, self.exec_ = C.c_void_p(), C.c_void_p(), C.c_void_p(), C.c_void_p()
        check(lib().cutile_device_get(int(device), C.byref(self.device)))
        check(lib().cutile_stream_create(self.device, C.byref(self.stream)))

    def capture(self, record) -> "CapturedGraph":
        check(lib().cutile_stream_begin_capture(self.stream))
        try:
            record(self.stream.value)
        finally:
            status = lib().cutile_stream_end_capture(self.stream, C.byref(self.graph))
        check(status)
        check(lib().cutile_graph_instantiate(self.graph, C.byref(self.exec_)))
        check(lib().cutile_graph_upload(self.exec_, self.stream))
        return self

    def launch(self) -> None:
        check(lib().cutile_graph_launch(self.exec_, self.stream))

    def synchronize(self) -> None:
        check(lib().cutile_stream_synchronize(self.stream))

    def close(self) -> None:
        if self.exec_:
            lib().cutile_graph_exec_destroy(self.exec_)
            self.exec_ = C.c_void_p()
        if self.graph:
            lib().cutile_graph_destroy(self.graph)
            self.graph = C.c_void_p()
        if self.stream:
            lib().cutile_stream_release(self.device, self.stream)
            self.stream = C.c_void_p()


class EventTimer:
    """HIP-event timing on a given stream through the C ABI (cutile/src/bench.rs:162-211)."""

    def __init__(self, stream=None):
        self.stream = _stream(stream)
        self.start_ev, self.stop_ev = C.c_void_p(), C.c_void_p()
        check(lib().cutile_event_create(C.byref(self.start_ev)))
        check(lib().cutile_event_create(C.byref(self.stop_ev)))

    def start(self):
        check(lib().cutile_event_record(self.start_ev, self.stream))

    def stop(self) -> float:
        check(lib().cutile_event_record(self.stop_ev, self.stream))
        check(lib().cutile_event_synchronize(self.stop_ev))
        ms = C.c_float()
        check(lib().cutile_event_elapsed_ms(self.start_ev, self.stop_ev, C.byref(ms)))
        return ms.value

    def close(self):
        lib().cutile_event_destroy(self.start_ev)
        lib().cutile_event_destroy(self.stop_ev)


class EventSeries:
    """n + 1 HIP events on one stream, recorded between n back-to-back launches: the duration of every launch of a
    sustained run without a host synchronisation in between (the events are read after the last one completes)."""

    def __init__(self, n: int, stream=None):
        self.stream = _stream(stream)
        self.events = []
        for _ in range(n + 1):
            ev = C.c_void_p()
            check(lib().cutile_event_create(C.byref(ev)))
            self.events.append(ev)
        self.k = 0

    def mark(self):
        check(lib().cutile_event_record(self.events[self.k], self.stream))
        self.k += 1

    def gaps_ms(self) -> list:
        check(lib().cutile_event_synchronize(self.events[self.k - 1]))
        out = []
        for a, b in zip(self.events[: self.k - 1], self.events[1: self.k]):
            ms = C.c_float()
            check(lib().cutile_event_elapsed_ms(a, b, C.byref(ms)))
            out.append(ms.value)
        return out

    def close(self):
        for ev in self.events:
            lib().cutile_event_destroy(ev)
        self.events = []
