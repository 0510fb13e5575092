"""CPU tests of the C-ABI library's host side: exported symbols, grid / specialization
logic against the reference's own unit-test vectors, and the launchers' validation,
variant selection, grid translation and argument marshalling observed through the
recording stand-in for the HIP runtime (no kernel runs, nothing is computed)."""
import ctypes as C
import os
import re
import struct

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b(cutile_[a-z0-9_]+)\s*\(", text))


def test_library_exports_every_declared_symbol(ct):
    import __graft_entry__ as entry

    L = ct.lib()
    declared = _declared("cutile_hip.h")
    assert len(declared) > 100
    missing = [s for s in sorted(declared) if not hasattr(L, s)]
    assert not missing, missing
    # the test hooks live in the testing library only: the product library carries none of them
    hooks = _declared("cutile_hip_testing.h")
    assert len(hooks) >= 8 and not [s for s in hooks if hasattr(L, s)]
    T = entry.load_package(testing=True).lib()
    assert not [s for s in sorted(declared | hooks) if not hasattr(T, s)]


def test_status_names_and_dtypes(ct):
    L = ct.lib()
    assert L.cutile_status_name(0) == b"CUTILE_SUCCESS" and L.cutile_status_name(-4) == b"CUTILE_ERR_KERNEL_LAUNCH"
    assert L.cutile_status_name(700) == b"DriverError"
    # names are the strings passed in .generics (cuda-core/src/dtype.rs:189-229)
    for name, size in [("f32", 4), ("f64", 8), ("f16", 2), ("bf16", 2), ("i32", 4), ("u8", 1), ("f8e4m3fn", 1),
                       ("f8e8m0fnu", 1), ("bool", 1), ("i64", 8)]:
        code = L.cutile_dtype_from_name(name.encode())
        assert code < ct.DTYPE_COUNT and L.cutile_dtype_name(code) == name.encode() and L.cutile_dtype_size(code) == size
    assert L.cutile_dtype_from_name(b"f128") == ct.DTYPE_COUNT


def test_without_a_gpu_compute_entry_points_fail_loudly(ct):
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    y = torch.zeros(8)
    with pytest.raises(ct.CutileError) as e:
        ct.saxpy(ct.partition(y, [4]), 2.0, torch.ones(8))
    assert e.value.status != 0 and "DriverError" in e.value.message or "shared object" in e.value.message
    assert torch.equal(y, torch.zeros(8))          # nothing was computed on the host


# ---- Partition::grid / infer_launch_grid (cutile/src/tensor.rs:447-468, tile_kernel.rs:782-808,934-967) ----
def test_partition_grid(ct):
    assert ct.partition(torch.zeros(128, 256), [32, 64]).grid() == (4, 4, 1)       # doc example tensor.rs:440-442
    assert ct.partition(torch.zeros(1000), [128]).grid() == (8, 1, 1)               # div_ceil
    assert ct.partition(torch.zeros(4, 5, 6), [1, 2, 4]).grid() == (4, 3, 2)
    with pytest.raises(ct.CutileError, match="at most rank 3"):
        ct.partition(torch.zeros(2, 2, 2, 2), [1, 1, 1, 1]).grid()


def _infer(ct, explicit, bounds):
    """bounds: list of (grid tuple, exact?) realised as rank-3 partitions with unit tiles."""
    parts = []
    for g, exact in bounds:
        p = ct.partition(torch.zeros(*g), [1, 1, 1], prefix=not exact).arg()
        parts.append(p)
    arr = (C.POINTER(ct.PartitionArg) * max(1, len(parts)))(*[C.pointer(p) for p in parts])
    eg = (C.c_uint32 * 3)(*explicit)
    out = (C.c_uint32 * 3)()
    ct.check(ct.lib().cutile_infer_launch_grid(C.byref(eg), arr, len(parts), C.byref(out)))
    return tuple(out)


def test_infer_launch_grid_truth_table(ct):
    EX, AM = True, False
    # tile_kernel.rs:1567-1594
    with pytest.raises(ct.CutileError, match="partial-coverage"):
        _infer(ct, (0, 0, 0), [((3, 1, 1), AM)])
    assert _infer(ct, (0, 0, 0), [((3, 1, 1), EX), ((4, 1, 1), AM)]) == (3, 1, 1)
    with pytest.raises(ct.CutileError):
        _infer(ct, (0, 0, 0), [((3, 1, 1), EX), ((2, 1, 1), AM)])
    assert _infer(ct, (2, 1, 1), [((3, 1, 1), AM)]) == (2, 1, 1)
    with pytest.raises(ct.CutileError, match="exceeds the partial-coverage"):
        _infer(ct, (4, 1, 1), [((3, 1, 1), AM)])
    with pytest.raises(ct.CutileError, match="Launch grid required."):
        _infer(ct, (0, 0, 0), [])
    # tile_kernel.rs:1548-1565: per-axis prefix, never total count; exact keeps strict equality
    for g, ok in [((3, 2, 1), True), ((2, 2, 1), True), ((2, 1, 1), True), ((4, 1, 1), False), ((1, 3, 1), False),
                  ((6, 1, 1), False)]:
        if ok:
            assert _infer(ct, g, [((3, 2, 1), AM)]) == g
        else:
            with pytest.raises(ct.CutileError):
                _infer(ct, g, [((3, 2, 1), AM)])
    with pytest.raises(ct.CutileError, match="does not match the inferred partition grid"):
        _infer(ct, (2, 1, 1), [((3, 1, 1), EX), ((3, 1, 1), AM)])
    assert _infer(ct, (3, 1, 1), [((3, 1, 1), EX), ((4, 1, 1), AM)]) == (3, 1, 1)
    # tile_kernel.rs:1509-1517: matching / mismatching exact grids
    assert _infer(ct, (4, 1, 1), [((4, 1, 1), EX)]) == (4, 1, 1)
    with pytest.raises(ct.CutileError):
        _infer(ct, (4, 1, 1), [((2, 1, 1), EX)])


def _spec(ct, ptr, shape, strides):
    t = ct.TensorArg()
    t.ptr, t.rank = ptr, len(shape)
    for i, (s, st) in enumerate(zip(shape, strides)):
        t.shape[i], t.strides[i] = s, st
    sb = ct.SpecBits()
    ct.check(ct.lib().cutile_compute_spec(C.byref(t), C.byref(sb)))
    r = len(shape)
    return list(sb.shape_div)[:r], list(sb.stride_div)[:r], [bool(v) for v in sb.stride_one][:r], sb.base_ptr_div, bool(sb.elements_disjoint)


def test_compute_spec_vectors(ct):
    # cutile-compiler/src/specialization_tests.rs:68-205
    assert _spec(ct, 0x1000, [1024], [1]) == ([16], [1], [True], 16, True)
    assert _spec(ct, 0x1000, [128, 256], [256, 1]) == ([16, 16], [16, 1], [False, True], 16, True)
    assert _spec(ct, 0x1000, [1023], [1])[:3] == ([1], [1], [True])
    assert _spec(ct, 0x1004, [128], [1])[3] == 4
    assert _spec(ct, 0x1000, [4, 8], [8, 1])[4] is True
    assert _spec(ct, 0x1000, [4, 8], [4, 1])[4] is False           # overlapping rows
    for v, d in [(1, 1), (2, 2), (8, 8), (16, 16), (32, 16), (3, 1), (6, 2), (12, 4), (24, 8), (48, 16), (1023, 1), (0, 16)]:
        assert _spec(ct, 0x1000, [max(v, 1)], [v])[1] == [d]        # max_pow2_divisor, clamped to 16, 0 -> 16


# ---- launchers through the recording runtime ------------------------------------------------
def _last(fake_hip):
    n = fake_hip.lib().cutile_testing_launch_count()
    rec = fake_hip.LaunchRecord()
    fake_hip.check(fake_hip.lib().cutile_testing_get_launch(n - 1, C.byref(rec)))
    return rec, bytes(rec.args[:rec.args_size])


def test_saxpy_argument_marshalling_and_variant_choice(fake_hip):
    ct = fake_hip
    y, x = torch.zeros(4, 8), torch.ones(4, 8)
    ct.saxpy(ct.partition(y, [2, 2]), 2.0, x)
    rec, args = _last(ct)
    assert rec.symbol == b"saxpy_entry__f32_r2_flat" and tuple(rec.block) == (256, 1, 1) and tuple(rec.grid) == (1, 1, 1)
    # (ptr, shape[2], strides[2], partition_shape[2], partition_strides[2]) a (ptr, shape[2], strides[2]) tile grid
    # — the push order of cutile/src/tensor.rs:1723-1739, 2005-2016
    yp, s0, s1, st0, st1, p0, p1, ps0, ps1, a, _pad, xp, xs0, xs1, xst0, xst1, gx, gy, gz, _ = struct.unpack("<Q8ifiQ4i4I", args)
    assert (yp, xp) == (y.data_ptr(), x.data_ptr()) and (s0, s1, st0, st1) == (4, 8, 8, 1)
    assert (p0, p1, ps0, ps1) == (2, 2, 8, 1) and a == 2.0 and (xs0, xs1, xst0, xst1) == (4, 8, 8, 1) and (gx, gy, gz) == (2, 4, 1)
    # a strided view cannot take the flat path; one workgroup per tile
    big = torch.zeros(4, 16)
    ct.saxpy(ct.partition(big[:, :8], [2, 2]), 2.0, x)
    rec, _ = _last(ct)
    assert rec.symbol == b"saxpy_entry__f32_r2_tiled" and tuple(rec.grid) == (2, 4, 1)
    # asking for a variant that does not fit the arguments is an error, not a silent switch
    with pytest.raises(ct.CutileError, match="does not fit"):
        ct.saxpy(ct.partition(big[:, :8], [2, 2]), 2.0, x, variant="f32_r2_flat")


def test_validation_happens_before_any_gpu_work(fake_hip):
    ct = fake_hip
    L = ct.lib()
    L.cutile_testing_clear_log()
    z = torch.zeros(512, 512, dtype=torch.bfloat16)
    a, b = torch.zeros(512, 256, dtype=torch.bfloat16), torch.zeros(256, 512, dtype=torch.bfloat16)
    cases = [
        (lambda: ct.gemm(ct.partition(z, [256, 256]), a, b, 256, grid=(1, 1, 1)), "does not match the inferred partition grid"),
        (lambda: ct.gemm(ct.partition(z, [256, 256], prefix=True), a, b, 256), "partial-coverage"),
        (lambda: ct.gemm(ct.partition(z, [100, 100]), a, b, 256, variant="bf16_256x256x64_d4x2"), "does not fit these arguments"),
        (lambda: ct.gemm(ct.partition(z, [256, 256]), a, b, 256, generics=["bf16", 128, 256, 64]), "generic BM"),
        (lambda: ct.gemm(ct.partition(z, [256, 256]), a.float(), b, 256), "x and y must both be"),
        (lambda: ct.gemm(ct.partition(z, [256, 256]), a.float(), b.float(), 256), "no kernel for f32 operands with bf16 z"),
        (lambda: ct.rms_norm_f16(torch.zeros(4, 64, dtype=torch.half), torch.zeros(32, dtype=torch.half),
                                 ct.partition(torch.zeros(4, 64, dtype=torch.half), [1, 64]), 1e-6), "expected N = 64"),
        (lambda: ct.rms_norm_f16(torch.zeros(4, 64, dtype=torch.half), torch.zeros(64, dtype=torch.half),
                                 ct.partition(torch.zeros(4, 64, dtype=torch.half), [2, 64]), 1e-6), r"partitioned \[1, 64\]"),
        (lambda: ct.softmax(torch.zeros(4, 64), ct.partition(torch.zeros(4, 64, dtype=torch.half), [1, 64])), "both be f16 or both f32"),
        (lambda: ct.fmha(ct.partition(torch.zeros(4, 64, 32, dtype=torch.bfloat16), [1, 32, 32]),
                         *(torch.zeros(1, 4, 64, 32, dtype=torch.bfloat16) for _ in range(3)), 0.1, 0, 3), "do not agree"),
        (lambda: ct.saxpy(ct.partition(torch.zeros(8), [4]), 1.0, torch.zeros(8, dtype=torch.float64)), "element type f32"),
    ]
    for fn, msg in cases:
        with pytest.raises(ct.CutileError, match=msg):
            fn()
    assert L.cutile_testing_launch_count() == 0


def test_grid_translation_per_kernel_family(fake_hip):
    ct = fake_hip
    h = torch.half
    # row-wise: four single-wave rows per workgroup for N <= 8192 in registers
    x, w, o = torch.zeros(100, 1024, dtype=h), torch.zeros(1024, dtype=h), torch.zeros(100, 1024, dtype=h)
    ct.rms_norm_f16(x, w, ct.partition(o, [1, 1024]), 1e-6, generics=[1024, 512])
    rec, _ = _last(ct)
    assert rec.symbol == b"rms_norm_f16_entry__w1v2" and tuple(rec.grid) == (25, 1, 1)
    ct.rms_norm_f16(x, w, ct.partition(o, [1, 1024]), 1e-6, variant="w4v4")
    assert tuple(_last(ct)[0].grid) == (100, 1, 1)
    # N = 1001 is not a whole number of 16-byte vectors: the any-shape kernel takes it
    x1, w1, o1 = torch.zeros(8, 1001, dtype=h), torch.zeros(1001, dtype=h), torch.zeros(8, 1001, dtype=h)
    ct.rms_norm_f16(x1, w1, ct.partition(o1, [1, 1001]), 1e-6)
    assert _last(ct)[0].symbol == b"rms_norm_f16_entry__generic"
    # chunk softmax: 16 rows x 4 column tiles = 64 segments of 2048
    xs, ys = torch.zeros(16, 8192, dtype=h), torch.zeros(16, 8192, dtype=h)
    ct.softmax(xs, ct.partition(ys, [1, 2048]))
    rec, _ = _last(ct)
    assert rec.symbol == b"softmax_entry__f16_w1v4" and tuple(rec.grid) == (16, 1, 1)
    # GEMM: one workgroup per output tile on a 1-D grid (the kernel remaps ids per XCD)
    z = torch.zeros(1000, 520, dtype=torch.bfloat16)
    a, b = torch.zeros(1000, 256, dtype=torch.bfloat16), torch.zeros(256, 520, dtype=torch.bfloat16)
    ct.gemm(ct.partition(z, [128, 128]), a, b, 256)
    rec, args = _last(ct)
    assert rec.symbol == b"gemm_entry__bf16_128x128x64_d2x2" and tuple(rec.grid) == (8 * 5, 1, 1) and tuple(rec.block) == (256, 1, 1)
    k_total, gx, gy, gz, _, acc = struct.unpack_from("<i4Ii", args, 88)
    assert (k_total, gx, gy, gz, acc) == (256, 8, 5, 1, 1)
    # FMHA: (batch*heads, query tiles)
    q = torch.zeros(2, 4, 512, 128, dtype=torch.bfloat16)
    out = torch.zeros(8, 512, 128, dtype=torch.bfloat16)
    ct.fmha(ct.partition(out, [1, 128, 128]), q, q, q, 0.088, 0, 1, causal=True, generics=[128, 64, 128, 4, 1, 1])
    rec, _ = _last(ct)
    assert rec.symbol == b"fmha_entry__bf16_128x64x128" and tuple(rec.grid) == (8, 4, 1) and tuple(rec.block) == (256, 1, 1)
    # MXFP8: the reference example's 16x16 tiles are covered by one 32x32 kernel tile
    u8 = torch.uint8
    ct.linear_tile_mxfp8(ct.partition(torch.zeros(16, 16), [16, 16]), torch.zeros(16, 128, dtype=u8), torch.zeros(16, 128, dtype=u8),
                         torch.zeros(16, 4, dtype=u8), torch.zeros(16, 4, dtype=u8), 1.0, generics=[16, 16, 64, 2])
    rec, _ = _last(ct)
    assert rec.symbol == b"linear_tile_entry__mxfp8_f32_32x32x128_w1x1" and tuple(rec.grid) == (1, 1, 1)


def test_eye_launcher_on_the_recording_runtime(fake_hip):
    ct = fake_hip
    t = torch.zeros(40, 72)
    ct.eye(ct.partition(t, [16, 16]), generics=[16, 16])
    rec, args = _last(ct)
    assert rec.symbol == b"eye_entry__f32" and tuple(rec.block) == (256, 1, 1) and tuple(rec.grid) == (3, 1, 1)   # ceil(40*72 / 1024)
    ptr, s0, s1, st0, st1, p0, p1, _ps0, _ps1, gx, gy, gz, _ = struct.unpack("<Q8i4I", args)
    assert ptr == t.data_ptr() and (s0, s1, st0, st1, p0, p1) == (40, 72, 72, 1, 16, 16) and (gx, gy, gz) == (3, 5, 1)
    n = ct.lib().cutile_testing_launch_count()
    with pytest.raises(ct.CutileError, match="must be f32"):
        ct.eye(ct.partition(torch.zeros(16, 16, dtype=torch.half), [16, 16]))
    with pytest.raises(ct.CutileError, match="generic BC"):
        ct.eye(ct.partition(t, [16, 16]), generics=[16, 8])
    with pytest.raises(ct.CutileError):
        ct.eye(ct.partition(torch.zeros(64), [16]))                 # rank 1
    assert ct.lib().cutile_testing_launch_count() == n


def test_example_program_launchers_on_the_recording_runtime(fake_hip):
    ct = fake_hip
    # relu: (partition, tile grid); flat over the covered elements, 4096 per workgroup
    t = torch.zeros(10000)
    ct.relu(ct.partition(t, [100]), generics=[100])
    rec, args = _last(ct)
    assert rec.symbol == b"relu_entry__f32" and tuple(rec.grid) == (3, 1, 1) and tuple(rec.block) == (256, 1, 1)
    ptr, n, st, p, _ps, gx, gy, gz, _ = struct.unpack("<Q4i4I", args)
    assert ptr == t.data_ptr() and (n, st, p) == (10000, 1, 100) and (gx, gy, gz) == (100, 1, 1)
    # dropout: p first, then the two tensors, the partition, the tile grid (signature order)
    x, keep, out = torch.zeros(16), torch.zeros(16), torch.zeros(16)
    ct.dropout(0.4, x, keep, ct.partition(out, [4]), generics=[4])
    rec, args = _last(ct)
    assert rec.symbol == b"dropout_entry__f32" and tuple(rec.grid) == (1, 1, 1)
    pv, xp, xn, xs, kp, kn, ks, op = struct.unpack_from("<f4xQ2iQ2iQ", args, 0)
    assert abs(pv - 0.4) < 1e-7 and (xp, xn, xs) == (x.data_ptr(), 16, 1) and (kp, kn, ks) == (keep.data_ptr(), 16, 1) and op == out.data_ptr()
    # scale_ptr: raw pointers, scale, len; the caller's grid is required but does not shape the dispatch
    ct.scale_ptr(out.data_ptr(), x.data_ptr(), 3.0, 16, grid=(4, 1, 1))
    rec, args = _last(ct)
    assert rec.symbol == b"scale_ptr_entry__f32" and tuple(rec.grid) == (1, 1, 1)
    assert struct.unpack("<QQfi", args) == (out.data_ptr(), x.data_ptr(), 3.0, 16)
    # matvec: one wavefront per row, four rows per workgroup; k is cut to whole K tiles
    z, xm, y = torch.zeros(1000), torch.zeros(1000, 70), torch.zeros(70)
    ct.matvec(ct.partition(z, [8]), xm, y, 70, generics=[8, 16, 70])
    rec, args = _last(ct)
    assert rec.symbol == b"matvec_entry__f32" and tuple(rec.grid) == (250, 1, 1)
    assert struct.unpack_from("<i4I", args, 24 + 24 + 16) == (64, 125, 1, 1, 0)
    # batch_matmul: tile grid (batches, M tiles, N tiles); pipelined variant on (M tiles * N tiles, batches), any-layout on 64 x 64 blocks
    a, b, c = torch.zeros(3, 256, 64, dtype=torch.bfloat16), torch.zeros(3, 64, 384, dtype=torch.bfloat16), torch.zeros(3, 256, 384, dtype=torch.bfloat16)
    ct.batch_matmul(ct.partition(c, [1, 128, 128]), a, b, 64, generics=["bf16", 128, 128, 64, 64])
    rec, args = _last(ct)
    assert rec.symbol == b"batch_matmul_entry__bf16_128x128x64_d2x2" and tuple(rec.grid) == (6, 3, 1) and tuple(rec.block) == (256, 1, 1)
    assert struct.unpack_from("<i4I", args, 56 + 32 + 32) == (64, 3, 2, 3, 0)
    ct.batch_matmul(ct.partition(torch.zeros(4, 128, 256), [1, 64, 64]), torch.zeros(4, 128, 64), torch.zeros(4, 64, 256), 64, generics=["f32", 64, 64, 32, 64])
    rec, _ = _last(ct)
    assert rec.symbol == b"batch_matmul_entry__f32_generic" and tuple(rec.grid) == (2, 4, 4)
    n = ct.lib().cutile_testing_launch_count()
    with pytest.raises(ct.CutileError, match="Launch grid required."):
        ct.scale_ptr(out.data_ptr(), x.data_ptr(), 3.0, 16)
    with pytest.raises(ct.CutileError, match="generic D"):
        ct.relu(ct.partition(t, [100]), generics=[64])
    with pytest.raises(ct.CutileError, match="must be f32"):
        ct.matvec(ct.partition(z.half(), [8]), xm, y, 70)
    with pytest.raises(ct.CutileError, match=r"partitioned \[1, BM, BN\]"):
        ct.batch_matmul(ct.partition(c, [3, 128, 128]), a, b, 64)
    many = 65536                                    # one more batch than the grid axis that carries the batch can hold
    with pytest.raises(ct.CutileError, match="65535 workgroups of the grid axis"):
        ct.batch_matmul(ct.partition(torch.zeros(many, 8, 8), [1, 8, 8]), torch.zeros(many, 8, 8), torch.zeros(many, 8, 8), 8)
    assert ct.lib().cutile_testing_launch_count() == n


def test_kernel_table_lookup_and_single_flight_module_load(fake_hip):
    ct = fake_hip
    L = ct.lib()
    before = L.cutile_module_load_count()
    info = ct.kernel_lookup("gemm", ["bf16", "256", "256", "64"])
    assert info.symbol.startswith(b"gemm_entry__bf16_256x256x64") and tuple(info.tile)[:3] == (256, 256, 64)
    info2 = ct.kernel_lookup("gemm", ["bf16", "128", "128", "64"])
    assert info2.symbol == b"gemm_entry__bf16_128x128x64_d2x2" and tuple(info2.block) == (256, 1, 1)
    assert L.cutile_module_load_count() == before + 1          # one code object per kernel family per device
    assert ct.kernel_lookup("gemm", ["bf16", "48", "48", "16"]).symbol == b"gemm_entry__bf16_generic"   # any tile shape
    with pytest.raises(ct.CutileError, match="available: "):
        ct.kernel_lookup("gemm", ["f64", "48", "48", "16"])
    with pytest.raises(ct.CutileError):
        ct.kernel_lookup("no_such_kernel")
    names = ct.kernel_list()
    assert "saxpy:f32_r1_flat" in names and "fmha:bf16_256x64x128" in names and len(set(names)) == len(names)
    # pinned preference (autotuner output) is honoured and validated
    ct.set_preferred_variant("gemm", "bf16_256x256x64_w2x2")
    z = torch.zeros(256, 256, dtype=torch.bfloat16)
    ct.gemm(ct.partition(z, [256, 256]), z, z, 256)
    assert _last(ct)[0].symbol == b"gemm_entry__bf16_256x256x64_w2x2"
    ct.set_preferred_variant("gemm", None)
    with pytest.raises(ct.CutileError):
        ct.set_preferred_variant("gemm", "nope")


def test_driver_layer_on_the_recording_runtime(fake_hip):
    ct = fake_hip
    L = ct.lib()
    n = C.c_int32()
    ct.check(L.cutile_device_count(C.byref(n)))
    assert n.value == 1
    dev = ct.device(0)
    assert ct.device(0) == dev                                  # one handle per ordinal
    with pytest.raises(ct.CutileError, match="DriverError"):
        ct.device(3)                                            # cuda-async/tests/error_handling.rs:174-190
    assert "gfx950" in ct.device_arch(0) and ct.device_props(0).wavefront_size == 64
    # streams are pooled: a released stream is handed out again, never destroyed
    s1, s2 = C.c_void_p(), C.c_void_p()
    created = L.cutile_testing_streams_created()
    ct.check(L.cutile_stream_create(dev, C.byref(s1)))
    ct.check(L.cutile_stream_release(dev, s1))
    ct.check(L.cutile_stream_create(dev, C.byref(s2)))
    assert s1.value == s2.value and L.cutile_testing_streams_created() == created + 1
    # async alloc / copies / memset round trip
    p = C.c_void_p()
    ct.check(L.cutile_malloc_async(64, s2, C.byref(p)))
    src = (C.c_ubyte * 64)(*range(64))
    dst = (C.c_ubyte * 64)()
    ct.check(L.cutile_memcpy_htod_async(p, src, 64, s2))
    ct.check(L.cutile_memcpy_dtoh_async(dst, p, 64, s2))
    ct.check(L.cutile_stream_synchronize(s2))
    assert bytes(dst) == bytes(range(64))
    ct.check(L.cutile_memset_d8_async(p, 7, 64, s2))
    ct.check(L.cutile_memcpy_dtoh_async(dst, p, 64, s2))
    assert bytes(dst) == bytes([7] * 64)
    ct.check(L.cutile_free_async(p, s2))
    # a module image that is not ELF is rejected before the driver sees it (runtime.rs:309-328)
    mod = C.c_void_p()
    L.cutile_module_load_data.argtypes = [C.c_void_p, C.c_char_p, C.c_size_t, C.POINTER(C.c_void_p)]
    assert L.cutile_module_load_data(dev, b"not an elf image", 16, C.byref(mod)) == -2
    # driver failures surface as DriverError(code) with the runtime's text
    ct.check(L.cutile_testing_inject_failure(b"hipMallocAsync", 2, 1))
    st = L.cutile_malloc_async(64, s2, C.byref(p))
    assert st == 2 and b"DriverError(2)" in L.cutile_last_error_message()


def test_decode_mapped_and_fp4_launchers_on_the_recording_runtime(fake_hip):
    """grid translation, argument records and validation of the launchers added for the decode path,
    mapped partitions and NVFP4 — no GPU involved"""
    ct = fake_hip
    L = ct.lib()
    h = torch.half
    # decode split: one workgroup per (KV head, split); the variant follows (GROUP, D)
    q, kv = torch.zeros(8, 4, 128, dtype=h), torch.zeros(8, 1024, 128, dtype=h)
    att, lse = torch.zeros(8, 16 * 4, 128, dtype=h), torch.zeros(8, 16 * 4)
    pos = torch.zeros(1, dtype=torch.int32)
    ct.fmha_decode_gqa_split(q, kv, kv, ct.partition(att, [1, 4, 128]), ct.partition(lse, [1, 4]), 0.088, pos, generics=[4, 64, 128, 16])
    rec, args = _last(ct)
    assert rec.symbol == b"fmha_decode_gqa_split_entry__f16_g4_d128_mfma" and tuple(rec.grid) == (8, 16, 1) and tuple(rec.block) == (256, 1, 1)
    # q (32) + k (32) + v (32) + att partition (56) + lse partition (40) = 192, then scale, pad, position pointer, bn, tile grid
    scale, = struct.unpack_from("<f", args, 192)
    ptr, bn = struct.unpack_from("<Qi", args, 200)
    assert abs(scale - 0.088) < 1e-7 and ptr == pos.data_ptr() and bn == 64
    assert struct.unpack_from("<4I", args, 212)[:3] == (8, 16, 1)
    out = torch.zeros(8, 4, 128, dtype=h)
    ct.splitk_reduce_merge(att, lse, ct.partition(out, [1, 4, 64]))
    rec, _ = _last(ct)
    assert rec.symbol == b"splitk_reduce_merge_entry__f16" and tuple(rec.grid) == (8 * 4, 1, 1)
    # kv cache update: a grid-stride copy sized by the rows written
    nk = torch.zeros(33, 8, 128, dtype=h)
    kc = torch.zeros(8, 96, 128, dtype=h)
    ct.kv_cache_update_f16(nk, nk, ct.partition(kc, [1, 16, 64]), ct.partition(kc.clone(), [1, 16, 64]), 0, 33)
    rec, _ = _last(ct)
    assert rec.symbol == b"kv_cache_update_entry__f16" and tuple(rec.grid) == (-(-33 * 8 * 16 // 256), 1, 1)
    # persistent GEMM: (num_tile_blocks, 1, 1) workgroups and the mapped record after the three tensors
    z = torch.zeros(1024, 768, dtype=torch.bfloat16)
    a, b = torch.zeros(1024, 256, dtype=torch.bfloat16), torch.zeros(256, 768, dtype=torch.bfloat16)
    ct.gemm_persistent(ct.mapped(ct.partition(z, [256, 256]), [2, 1], 5), a, b)
    rec, args = _last(ct)
    assert rec.symbol == b"gemm_persistent_entry__bf16_256x256x64_q2x4" and tuple(rec.grid) == (5, 1, 1) and tuple(rec.block) == (512, 1, 1)
    assert struct.unpack_from("<4i4I", args, 88) == (2, 1, 1, 2, 4, 3, 1, 12)      # map, rank, logical grid, stream items
    # NVFP4: the reference example's 16x16 tiles run on the 32x32 kernel when the launch covers the tensor
    x4, s4 = torch.zeros(16, 64, dtype=torch.uint8), torch.zeros(16, 8, dtype=torch.uint8)
    z4 = torch.zeros(16, 16)
    ct.linear_tile_nvfp4(ct.partition(z4, [16, 16]), x4, x4, s4, s4, 1.0, generics=[16, 16, 64, 32, 4])
    rec, _ = _last(ct)
    assert rec.symbol == b"linear_tile_nvfp4_entry__f32_32x32x64_w1x1" and tuple(rec.grid) == (1, 1, 1) and tuple(rec.block) == (64, 1, 1)
    zb = torch.zeros(512, 512)
    xb, sb = torch.zeros(512, 128, dtype=torch.uint8), torch.zeros(512, 16, dtype=torch.uint8)
    ct.linear_tile_nvfp4(ct.partition(zb, [256, 256]), xb, xb, sb, sb, 1.0)
    assert _last(ct)[0].symbol == b"linear_tile_nvfp4_entry__f32_256x256x64_q2x4" and tuple(_last(ct)[0].grid) == (4, 1, 1)

    n0 = L.cutile_testing_launch_count()
    q3 = torch.zeros(8, 3, 128, dtype=h)
    att3, lse3 = torch.zeros(8, 6, 128, dtype=h), torch.zeros(8, 6)
    cases = [
        (lambda: ct.fmha_decode_gqa_split(q3, kv, kv, ct.partition(att3, [1, 3, 128]), ct.partition(lse3, [1, 3]), 0.1, pos), "no precompiled variant"),
        (lambda: ct.fmha_decode_gqa_split(q, kv, kv, ct.partition(att, [1, 4, 128]), ct.partition(lse, [1, 4]), 0.1, pos, generics=[4, 64, 128, 8]), "NUM_KV_SPLITS"),
        (lambda: ct.fmha_decode_gqa_split(q, kv, kv, ct.partition(att, [1, 4, 128]), ct.partition(lse[:, :32], [1, 4]), 0.1, pos), "do not agree"),
        (lambda: ct.splitk_reduce_merge(att, lse, ct.partition(out, [1, 4, 48])), "CHUNK_D dividing D"),
        (lambda: ct.kv_cache_update_f16(nk, nk, ct.partition(kc, [1, 16, 64]), ct.partition(kc.clone(), [1, 16, 64]), 4, 33), "position_start must be 0"),
        (lambda: ct.kv_cache_update_f16(nk, nk, ct.partition(kc, [1, 16, 64]), ct.partition(kc.clone(), [1, 16, 64]), 0, 34), "seq_len = 34"),
        (lambda: ct.gemm_persistent(ct.mapped(ct.partition(z, [256, 256]), [2, 1], 13), a, b), "cannot exceed the streamed logical tile count"),
        (lambda: ct.gemm_persistent(ct.mapped(ct.partition(z, [256, 256]), [2, 0], 2), a, b), "both axes streamed"),
        (lambda: ct.gemm_persistent(ct.mapped(ct.partition(z, [256, 256]), [2, 1], 5), a, b, grid=(4, 1, 1)), "does not match the inferred partition grid"),
        (lambda: ct.linear_tile_nvfp4(ct.partition(z4, [16, 16]), x4, x4, s4[:, :4], s4, 1.0), "scales must be"),
        (lambda: ct.linear_tile_nvfp4(ct.partition(z4, [16, 16]), x4, x4, s4, s4, 1.0, generics=[16, 16, 64, 32, 2]), "BK_SCALES"),
        (lambda: ct.linear_tile_nvfp4(ct.partition(torch.zeros(16, 16, dtype=h), [16, 16]), x4, x4, s4, s4, 1.0), "z must be f32 or bf16"),
    ]
    for fn, msg in cases:
        with pytest.raises(ct.CutileError, match=msg):
            fn()
    assert L.cutile_testing_launch_count() == n0


def test_operands_of_2_gib_and_more_leave_the_32_bit_offset_kernels(fake_hip):
    """The pipelined matrix kernels address an operand through one descriptor with 32-bit byte offsets (0x80000000 means
    'outside'), so an operand that spans 2 GiB or more must not reach them: GEMM falls to the any-layout kernel
    (64-bit addresses), the block-scaled GEMMs and attention refuse.  Untouched host memory stands in for the operands."""
    ct = fake_hip
    bf = torch.bfloat16
    z = torch.empty(256, 256, dtype=bf)
    small_a, small_b = torch.empty(256, 512, dtype=bf), torch.empty(512, 256, dtype=bf)
    ct.gemm(ct.partition(z, [256, 256]), small_a, small_b, 512)
    assert _last(ct)[0].symbol.startswith(b"gemm_entry__bf16_256x256x64_d")
    # x spans (255 * (2^22 + 2^15) + 512) * 2 bytes = 2^31 + 8.2 MB through its row stride
    wide = torch.empty(256 * ((1 << 22) + (1 << 15)), dtype=bf).as_strided((256, 512), ((1 << 22) + (1 << 15), 1))
    ct.gemm(ct.partition(z, [256, 256]), wide, small_b, 512)
    assert _last(ct)[0].symbol == b"gemm_entry__bf16_generic"
    just_below = torch.empty(256 * (1 << 22), dtype=bf).as_strided((256, 512), (1 << 22, 1))          # 2^31 - 8.4 MB
    ct.gemm(ct.partition(z, [256, 256]), just_below, small_b, 512)
    assert _last(ct)[0].symbol.startswith(b"gemm_entry__bf16_256x256x64_d")
    with pytest.raises(ct.CutileError, match="does not fit these arguments"):
        ct.gemm(ct.partition(z, [256, 256]), wide, small_b, 512, variant="bf16_256x256x64_d4x2")
    zm = ct.mapped(ct.partition(z, [256, 256]), [1, 1], 1)
    ct.gemm_persistent(zm, wide, small_b)
    assert _last(ct)[0].symbol == b"gemm_persistent_entry__bf16_generic"
    # block-scaled GEMM: no any-layout kernel exists, so the launch is refused before any GPU work
    n_before = ct.lib().cutile_testing_launch_count()
    u8 = torch.uint8
    xq = torch.empty(256 * ((1 << 23) + (1 << 16)), dtype=u8).as_strided((256, 256), ((1 << 23) + (1 << 16), 1))
    yq, sc = torch.empty(256, 256, dtype=u8), torch.empty(256, 8, dtype=u8)
    zf = torch.empty(256, 256)
    with pytest.raises(ct.CutileError, match="below 2 GiB"):
        ct.linear_tile_mxfp8(ct.partition(zf, [256, 256]), xq, yq, sc, sc, 1.0)
    # attention: one (batch, head) of k spanning 2 GiB
    q = torch.empty(1, 1, 256, 128, dtype=bf)
    k = torch.empty(256 * ((1 << 22) + (1 << 15)), dtype=bf).as_strided((1, 1, 256, 128), (0, 0, (1 << 22) + (1 << 15), 1))
    out = torch.empty(1, 256, 128, dtype=bf)
    with pytest.raises(ct.CutileError, match="below 2 GiB"):
        ct.fmha(ct.partition(out, [1, 256, 128]), q, k, k, 0.1, 0, 1)
    assert ct.lib().cutile_testing_launch_count() == n_before


def test_rng_fills_on_the_recording_runtime(fake_hip):
    """cutile_rng_*: the fill kernel, its arguments and the stream position (4 f32 or 2 f64 values per Philox block)"""
    ct = fake_hip
    rng = ct.Rng(0x1122334455667788)
    t = torch.zeros(1001)
    rng.normal_(t, 0.5, 2.0)
    rec, args = _last(ct)
    assert rec.symbol == b"rng_fill_entry__f32" and tuple(rec.block) == (256, 1, 1) and tuple(rec.grid) == (1, 1, 1)
    ptr, n, seed, offset, kind, mean, std = struct.unpack("<QQQQiff", args[:44])
    assert (ptr, n, seed, offset, kind, mean, std) == (t.data_ptr(), 1001, 0x1122334455667788, 0, 1, 0.5, 2.0)
    assert rng.offset == 251
    d = torch.zeros(7, dtype=torch.float64)
    rng.uniform_(d)
    rec, args = _last(ct)
    assert rec.symbol == b"rng_fill_entry__f64"
    ptr, n, seed, offset, kind = struct.unpack("<QQQQi", args[:36])
    assert (n, offset, kind) == (7, 251, 0) and rng.offset == 255
    rng.set_seed(3)
    assert rng.offset == 0
    # compile-only (1) and specialize-only (2) calls enqueue nothing, so the stream position must not move
    L = ct.lib()
    L.cutile_set_launch_mode.argtypes = [C.c_int32]
    before = L.cutile_testing_launch_count()
    for mode in (1, 2):
        ct.check(L.cutile_set_launch_mode(mode))
        try:
            rng.uniform_(torch.zeros(64))
        finally:
            ct.check(L.cutile_set_launch_mode(0))
        assert rng.offset == 0 and L.cutile_testing_launch_count() == before
    rng.uniform_(torch.zeros(64))
    assert rng.offset == 16
    rng.set_seed(3)
    before = ct.lib().cutile_testing_launch_count()
    rng.uniform_(torch.zeros(0))                                   # nothing to fill: no launch
    assert ct.lib().cutile_testing_launch_count() == before
    with pytest.raises(ValueError):
        rng.uniform_(torch.zeros(4, dtype=torch.float16))
    rng.close()


def test_tuning_records_choose_variants_per_shape_class_and_stale_ones_are_refused(fake_hip, tmp_path):
    """cutile/src/tune.rs:762-1016 applied at start-up: a verified record's winner is what a launch of its shape class
    uses; without the record the table's order decides; a record whose provenance is stale is refused as a whole."""
    import json, subprocess, os

    ct = fake_hip
    bf = torch.bfloat16
    z, a, b = torch.empty(512, 512, dtype=bf), torch.empty(512, 256, dtype=bf), torch.empty(256, 512, dtype=bf)
    launch = lambda: ct.gemm(ct.partition(z, [256, 256]), a, b, 256)
    try:
        assert "switched off" in ct.tuning_reload("")
        launch()
        base = ct.last_resolved()
        assert base["source"] == "table" and base["bucket"] == "bf16_256x256|tiles<=256" and base["variant"] == "bf16_256x256x64_d4x2"
        # records are written by the C++ surface (tune::Record::save); build one through it so the config ids are the library's own
        helper = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "tests", "cpp", "bin", "write_record")
        def write(name, kernel, bucket, variant, **kw):
            path = tmp_path / name
            args = [helper, str(path), kernel, bucket, variant] + [f"{k}={v}" for k, v in kw.items()]
            subprocess.check_call(args)
            return path
        write("gemm.json", "gemm", base["bucket"], "bf16_256x256x64_d2x4")
        report = ct.tuning_reload(str(tmp_path))
        assert "applied" in report and "1 bucket(s) of kernel gemm" in report
        launch()
        got = ct.last_resolved()
        assert got["variant"] == "bf16_256x256x64_d2x4" and got["source"] == "record:" + base["bucket"]
        assert _last(ct)[0].symbol == b"gemm_entry__bf16_256x256x64_d2x4"
        # another shape class is not touched by that entry
        zb = torch.empty(8192, 8192, dtype=bf)
        ct.gemm(ct.partition(zb, [256, 256]), torch.empty(8192, 64, dtype=bf), torch.empty(64, 8192, dtype=bf), 64)
        assert ct.last_resolved()["source"] == "table" and ct.last_resolved()["bucket"] == "bf16_256x256|tiles>256"
        # the caller's variant still wins over the record
        ct.gemm(ct.partition(z, [256, 256]), a, b, 256, variant="bf16_256x256x64_w2x2")
        assert ct.last_resolved()["source"] == "caller"
        # a function-wide pin set at run time wins over the record; taking it away gives the record back
        ct.set_preferred_variant("gemm", "bf16_256x256x64_w2x2")
        launch()
        assert ct.last_resolved()["source"] == "pinned" and ct.last_resolved()["variant"] == "bf16_256x256x64_w2x2"
        ct.set_preferred_variant("gemm", None)
        launch()
        assert ct.last_resolved()["source"] == "record:" + base["bucket"] and ct.last_resolved()["variant"] == "bf16_256x256x64_d2x4"
        # a record whose winner does not fit the arguments (another tile) is ignored for this launch
        ct.set_preferred_variant_for("gemm", base["bucket"], "bf16_128x128x64_d2x2")
        launch()
        assert ct.last_resolved()["source"] == "table"
        # stale provenance: each is refused and said so; the launch falls back to the table's order
        for kw, why in (({"source_hash": "0123456789abcdef"}, "source_hash mismatch"), ({"arch": "gfx942"}, "arch mismatch"),
                        ({"l2_key": "fedcba9876543210"}, "l2 key"), ({"tileiras_fingerprint": "another compiler"}, "another device toolchain"),
                        ({"schema": 7}, "schema mismatch")):
            for f in tmp_path.iterdir():
                f.unlink()
            write("gemm.json", "gemm", base["bucket"], "bf16_256x256x64_d2x4", **kw)
            report = ct.tuning_reload(str(tmp_path))
            assert "refused" in report and why in report, (kw, report)
            assert ct.lib().cutile_tuning_applied_count() == 0
            launch()
            assert ct.last_resolved()["source"] == "table" and ct.last_resolved()["variant"] == base["variant"]
        # a torn file is refused too, and does not stop the other files
        (tmp_path / "aaa.json").write_text("{ not json")
        write("rms.json", "rms_norm_f16", "n<=1024", "w1v2")
        report = ct.tuning_reload(str(tmp_path))
        assert "refused" in report and "1 bucket(s) of kernel rms_norm_f16" in report
    finally:
        ct.tuning_reload(None)
