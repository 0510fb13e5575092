"""GPU parity tests: every hot-path kernel through the C ABI against the CPU oracle on the
same seeded inputs.  Tolerances: saxpy / add / creation bit exact; RMSNorm and softmax
f16 within 1 f16 ulp of the oracle (the oracle's f32 sums are ordered differently);
bf16 GEMM rel-L2 <= 1e-2; FMHA max-abs <= 2e-2; MXFP8 GEMM rel-L2 <= 3e-2 against the
f32 dequantised reference."""
import numpy as np
import pytest
import torch

import oracle
from util import (assert_rounded_close, f16_ulp_diff, from_dev_bf16_bits, from_dev_f16_bits, normal_bf16_bits, normal_f16_bits, rel_l2,
                  to_dev_bf16, to_dev_f16)

pytestmark = pytest.mark.gpu


def sync():
    torch.cuda.synchronize()


# ---- K1: saxpy / add ------------------------------------------------------------------------
def test_device_is_gfx950(ct, dev):
    assert "gfx950" in ct.device_arch(0)
    p = ct.device_props(0)
    assert p.wavefront_size == 64 and p.compute_units > 0


def test_saxpy_reference_vectors(ct, dev):
    # cutile-examples/examples/saxpy.rs:27-53: arange(32) as [4,8], tiles [2,2], a = 2
    base = torch.arange(32, dtype=torch.float32, device=dev)
    x = base.clone().reshape(4, 8)
    y = base.clone().reshape(4, 8)
    ct.saxpy(ct.partition(y, [2, 2]), 2.0, x)
    sync()
    assert torch.equal(y.flatten(), 2.0 * base + base)


@pytest.mark.parametrize("variant", [None, "f32_r1_tiled"])
@pytest.mark.parametrize("n", [1 << 20, 1000003, 1024, 5])
def test_saxpy_1d_bit_exact(ct, dev, n, variant):
    x, y = oracle.uniform_f32(n, 11), oracle.uniform_f32(n, 12)
    yd = torch.from_numpy(y.copy()).to(dev)
    ct.saxpy(ct.partition(yd, [1024]), 2.0, torch.from_numpy(x).to(dev), variant=variant)
    sync()
    assert np.array_equal(yd.cpu().numpy(), oracle.saxpy_f32(2.0, x, y))


def test_axpy_separate_output_bit_exact(ct, dev):
    n = (1 << 20) + 3
    x, y = oracle.uniform_f32(n, 21), oracle.uniform_f32(n, 22)
    zd = torch.empty(n, dtype=torch.float32, device=dev)
    ct.axpy(ct.partition(zd, [1024]), 2.0, torch.from_numpy(x).to(dev), torch.from_numpy(y).to(dev))
    sync()
    assert np.array_equal(zd.cpu().numpy(), oracle.saxpy_f32(2.0, x, y))


def test_saxpy_2d_ragged_and_padded_input(ct, dev):
    # y [37, 53] tiled [8, 16] (ragged both ways); x is smaller: rows/cols beyond it read 0
    y = oracle.uniform_f32((37, 53), 31)
    x = oracle.uniform_f32((30, 40), 32)
    yd = torch.from_numpy(y.copy()).to(dev)
    ct.saxpy(ct.partition(yd, [8, 16]), 1.5, torch.from_numpy(x).to(dev))
    sync()
    xp = np.zeros_like(y)
    xp[:30, :40] = x
    assert np.array_equal(yd.cpu().numpy(), oracle.saxpy_f32(1.5, xp, y).reshape(37, 53))


def test_saxpy_strided_view(ct, dev):
    big = torch.from_numpy(oracle.uniform_f32((64, 96), 41)).to(dev)
    yv = big[:, 16:80]                      # row stride 96, 64 columns
    x = torch.from_numpy(oracle.uniform_f32((64, 64), 42)).to(dev)
    expect = torch.from_numpy(oracle.saxpy_f32(3.0, x.cpu().numpy(), yv.cpu().numpy().copy())).reshape(64, 64)
    untouched = big[:, :16].clone()
    ct.saxpy(ct.partition(yv, [16, 16]), 3.0, x)
    sync()
    assert torch.equal(yv.cpu(), expect) and torch.equal(big[:, :16], untouched)


def test_saxpy_prefix_grid_leaves_tail_untouched(ct, dev):
    n = 8192
    x, y = oracle.uniform_f32(n, 51), oracle.uniform_f32(n, 52)
    yd = torch.from_numpy(y.copy()).to(dev)
    ct.saxpy(ct.partition(yd, [1024], prefix=True), 2.0, torch.from_numpy(x).to(dev), grid=(3, 1, 1))
    sync()
    got = yd.cpu().numpy()
    assert np.array_equal(got[:3072], oracle.saxpy_f32(2.0, x[:3072], y[:3072])) and np.array_equal(got[3072:], y[3072:])


def test_add_ones(ct, dev):
    # cutile/tests/gpu/add_basic.rs:29-43
    x = torch.ones(4096, device=dev)
    z = torch.zeros(4096, device=dev)
    ct.add(ct.partition(z, [128]), x, x)
    sync()
    assert torch.equal(z, torch.full_like(z, 2.0))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_add_16bit(ct, dev, dtype):
    n = 1 << 18
    x = torch.from_numpy(oracle.uniform_f32(n, 61)).to(dev).to(dtype)
    y = torch.from_numpy(oracle.uniform_f32(n, 62)).to(dev).to(dtype)
    z = torch.zeros_like(x)
    ct.add(ct.partition(z, [16384]), x, y)
    sync()
    assert torch.equal(z, x + y)


# ---- K7: creation / conversion --------------------------------------------------------------
@pytest.mark.parametrize("dtype,value", [(torch.float32, 3.5), (torch.float16, -2.25), (torch.bfloat16, 1.0),
                                         (torch.int32, 7), (torch.int64, -9), (torch.uint8, 200), (torch.float64, 0.1)])
def test_full(ct, dev, dtype, value):
    t = torch.zeros(1000, dtype=dtype, device=dev)
    ct.full(value, ct.partition(t, [128]))
    sync()
    assert torch.equal(t, torch.full_like(t, value))


@pytest.mark.parametrize("dtype", [torch.float32, torch.int32, torch.int64, torch.float16])
def test_arange(ct, dev, dtype):
    t = torch.zeros(1000, dtype=dtype, device=dev)
    ct.arange(ct.partition(t, [128]))
    sync()
    assert torch.equal(t, torch.arange(1000, device=dev).to(dtype))


def test_linspace(ct, dev):
    t = torch.zeros(257, device=dev)
    ct.linspace(ct.partition(t, [128]), 1.0, 0.5)
    sync()
    assert torch.equal(t, 1.0 + torch.arange(257, device=dev).float() * 0.5)


@pytest.mark.parametrize("rows,cols,tile", [(4, 4, 16), (32, 32, 16), (16, 32, 16), (32, 16, 16),      # cutile/tests/arange.rs:106-186
                                            (100, 37, 16), (1, 1, 16), (513, 1025, 64), (48, 48, 8)])
def test_eye(ct, dev, rows, cols, tile):
    t = torch.full((rows, cols), float("nan"), device=dev)
    ct.eye(ct.partition(t, [tile, tile]))
    sync()
    assert torch.equal(t, torch.eye(rows, cols, device=dev))


def test_eye_on_a_strided_view_and_a_prefix_grid(ct, dev):
    base = torch.full((40, 96), -1.0, device=dev)
    view = base[:, 8:72:2]                                   # 40 x 32, row stride 96, column stride 2
    ct.eye(ct.partition(view, [16, 16]))
    sync()
    assert torch.equal(view, torch.eye(40, 32, device=dev))
    mask = torch.ones_like(base, dtype=torch.bool)
    mask[:, 8:72:2] = False
    assert torch.all(base[mask] == -1.0)                     # nothing beside the view was written
    # a prefix partition launched over 2 x 1 tiles touches rows 0..31, columns 0..15 only
    t = torch.full((40, 40), -1.0, device=dev)
    ct.eye(ct.partition(t, [16, 16], prefix=True), grid=(2, 1, 1))
    sync()
    want = torch.full((40, 40), -1.0, device=dev)
    want[:32, :16] = torch.eye(32, 16, device=dev)
    assert torch.equal(t, want)


@pytest.mark.parametrize("src,dst", [(torch.int32, torch.float32), (torch.float32, torch.float16),
                                     (torch.float32, torch.bfloat16), (torch.float16, torch.float32),
                                     (torch.float64, torch.int64), (torch.bfloat16, torch.float16)])
def test_convert(ct, dev, src, dst):
    s = (torch.from_numpy(oracle.uniform_f32(1024, 71, -100, 100)).to(dev)).to(src)
    d = torch.zeros(1024, dtype=dst, device=dev)
    ct.convert(s, ct.partition(d, [128]))
    sync()
    assert torch.equal(d, s.to(dst))


def test_creation_and_convert_vector_paths_tails_and_layouts(ct, dev):
    """16-byte paths with a ragged tail, a base that is not 16-byte aligned, a source shorter than the
    destination (zero padding, cutile/src/_core.rs:651-657) and a strided destination"""
    n = 100003
    t = torch.full((n + 1,), 5.0, dtype=torch.float16, device=dev)
    ct.full(-2.25, ct.partition(t[1:], [128]))                     # base 2 bytes past an aligned address
    sync()
    assert t[0] == 5.0 and torch.all(t[1:] == -2.25)
    for dtype in (torch.int64, torch.float16, torch.uint8 if hasattr(ct, "U8") else torch.int32):
        a = torch.zeros(n, dtype=dtype, device=dev)
        ct.arange(ct.partition(a, [128]))
        sync()
        assert torch.equal(a, torch.arange(n, device=dev).to(dtype))
    lin = torch.zeros(n, device=dev)
    ct.linspace(ct.partition(lin, [128]), -3.0, 0.25)
    sync()
    assert torch.equal(lin, -3.0 + torch.arange(n, device=dev).float() * 0.25)
    src = torch.from_numpy(oracle.uniform_f32(70001, 73, -100, 100)).to(dev)
    for dst_dtype in (torch.float16, torch.bfloat16, torch.float64, torch.int32):
        d = torch.full((n,), 7, dtype=dst_dtype, device=dev)
        ct.convert(src, ct.partition(d, [128]))
        sync()
        assert torch.equal(d[:70001], src.to(dst_dtype)) and torch.all(d[70001:] == 0)
    h = src.to(torch.float16)
    wide = torch.zeros(2 * 70001, dtype=torch.float32, device=dev)
    ct.convert(h, ct.partition(wide[::2], [128]))                  # strided destination: element by element
    sync()
    assert torch.equal(wide[::2], h.float()) and torch.all(wide[1::2] == 0)
    d = torch.zeros(70000, dtype=torch.float32, device=dev)
    ct.convert(h[1:], ct.partition(d, [128]))                      # source base not 16-byte aligned
    sync()
    assert torch.equal(d, h[1:].float())


# ---- K2: RMSNorm ----------------------------------------------------------------------------
@pytest.mark.parametrize("rows,n,variant", [
    (64, 512, None), (33, 1024, None), (16, 2048, None), (16, 4096, None), (32, 8192, None),
    (32, 8192, "w4v4"), (32, 8192, "w2v8"), (32, 8192, "w4v8"), (8, 16384, None), (8, 32768, None),
    (16, 8192, "generic"), (7, 1000, None), (5, 24, None), (4, 8, None),
    (777, 128, None), (1500, 64, None), (515, 256, None), (300, 128, "s32"),        # short rows, ragged last workgroup
])
def test_rms_norm_f16(ct, dev, rows, n, variant):
    xb = normal_f16_bits((rows, n), 101)
    wb = oracle.f32_to_f16_bits(oracle.uniform_f32(n, 102, 0.5, 1.5))
    out = torch.zeros(rows, n, dtype=torch.float16, device=dev)
    ct.rms_norm_f16(to_dev_f16(xb, dev), to_dev_f16(wb, dev), ct.partition(out, [1, n]), 1e-6, variant=variant)
    sync()
    ref = oracle.rms_norm_f16(xb, wb, 1e-6)
    assert f16_ulp_diff(from_dev_f16_bits(out), ref).max() <= 1


@pytest.mark.parametrize("rows,n", [(64, 512), (33, 8192), (7, 1000), (5, 13)])
def test_rms_norm_f32_example_form(ct, dev, rows, n):
    """cutile-examples/examples/rms_norm.rs:17-61; the kernel adds the squares in another order than the oracle and the
    downward rounding turns a last-bit difference into a whole ulp of the scale: 2e-6 relative on the outputs (f32 sums of
    up to 8192 squares in two different tree orders)"""
    x, w = oracle.normal_f32((rows, n), 121), oracle.uniform_f32(n, 122, 0.5, 1.5)
    out = torch.zeros(rows, n, device=dev)
    ct.rms_norm_f32(torch.from_numpy(x).to(dev), torch.from_numpy(w).to(dev), ct.partition(out, [1, n]), 1e-6, generics=[n])
    sync()
    ref = oracle.rms_norm_f32_example(x, w, 1e-6)
    np.testing.assert_allclose(out.cpu().numpy(), ref, rtol=2e-6, atol=0)
    with pytest.raises(ct.CutileError, match="must be f32"):
        ct.rms_norm_f32(torch.from_numpy(x).to(dev).half(), torch.from_numpy(w).to(dev), ct.partition(out, [1, n]), 1e-6)


def test_rms_norm_f16_strided_rows_and_prefix(ct, dev):
    rows, n = 24, 1024
    xb = normal_f16_bits((rows, 2 * n), 111)
    wb = oracle.f32_to_f16_bits(oracle.uniform_f32(n, 112, 0.5, 1.5))
    xd = to_dev_f16(xb, dev)[:, :n]          # row stride 2n
    out = torch.zeros(rows, n, dtype=torch.float16, device=dev)
    ct.rms_norm_f16(xd, to_dev_f16(wb, dev), ct.partition(out, [1, n], prefix=True), 1e-6, grid=(10, 1, 1))
    sync()
    ref = oracle.rms_norm_f16(np.ascontiguousarray(xb[:, :n]), wb, 1e-6)
    got = from_dev_f16_bits(out)
    assert f16_ulp_diff(got[:10], ref[:10]).max() <= 1 and not got[10:].any()


# ---- K3: softmax ----------------------------------------------------------------------------
@pytest.mark.parametrize("m,n,bm,bn,variant", [
    (64, 1024, 1, 1024, None), (16, 8192, 1, 8192, None), (16, 8192, 2, 8192, "f16_w4v4"),
    (16, 8192, 1, 2048, None),          # chunk softmax: four independent tiles per row
    (9, 4096, 4, 4096, None), (6, 1000, 2, 1000, None), (6, 1000, 2, 512, None),
    (8, 16384, 1, 16384, None), (16, 4096, 1, 4096, "f16_generic"),
])
def test_softmax_f16(ct, dev, m, n, bm, bn, variant):
    xb = normal_f16_bits((m, n), 201, 2.0)
    y = torch.zeros(m, n, dtype=torch.float16, device=dev)
    ct.softmax(to_dev_f16(xb, dev), ct.partition(y, [bm, bn]), variant=variant)
    sync()
    ref = oracle.softmax_f16(xb, bm, bn)
    got = from_dev_f16_bits(y)
    assert f16_ulp_diff(got, ref).max() <= 1


@pytest.mark.parametrize("m,n,bm,bn", [(4, 8, 2, 8), (32, 4096, 2, 4096), (8, 8192, 1, 8192), (5, 100, 1, 100),
                                       (8, 2048, 1, 512)])
def test_softmax_f32(ct, dev, m, n, bm, bn):
    x = oracle.normal_f32((m, n), 211, 0, 2.0) if (m, n) != (4, 8) else np.arange(32, dtype=np.float32).reshape(4, 8)
    y = torch.zeros(m, n, device=dev)
    ct.softmax(torch.from_numpy(x).to(dev), ct.partition(y, [bm, bn]))
    sync()
    got = y.cpu().numpy()
    ref = oracle.softmax_f32(x, bm, bn)
    np.testing.assert_allclose(got, ref, rtol=2e-5, atol=1e-9)
    if bn == n:  # cutile-examples/examples/softmax.rs:55-60: rows sum to 1
        np.testing.assert_allclose(got.sum(axis=1), 1.0, atol=1e-4)


# ---- K4: bf16 GEMM --------------------------------------------------------------------------
GEMM_VARIANTS = ["bf16_256x256x64_q2x4", "bf16_128x128x64_q2x2", "bf16_256x256x64_r2x4", "bf16_256x256x64_r4x2", "bf16_128x128x64_r2x2", "bf16_256x256x64_d4x2", "bf16_256x256x64_d2x4", "bf16_128x128x64_d2x2", "bf16_256x256x64_w2x2", "bf16_256x256x64_w2x4", "bf16_256x256x64_w4x2", "bf16_256x128x64_w2x2",
                 "bf16_128x256x64_w2x2", "bf16_128x128x64_w2x2", "bf16_64x128x64_w2x2"]


@pytest.mark.parametrize("variant", GEMM_VARIANTS)
def test_gemm_bf16_variants(ct, dev, variant):
    bm, bn = (int(v) for v in variant.split("_")[1].split("x")[:2])
    m, n, k = 512, 768, 320
    a, b = normal_bf16_bits((m, k), 301, k ** -0.5), normal_bf16_bits((k, n), 302, k ** -0.5)
    z = torch.zeros(m, n, dtype=torch.bfloat16, device=dev)
    ct.gemm(ct.partition(z, [bm, bn]), to_dev_bf16(a, dev), to_dev_bf16(b, dev), k, accumulate=False, variant=variant)
    sync()
    ref = oracle.gemm_bf16(a, b, f32out=True)
    got = z.float().cpu().numpy()
    assert rel_l2(got, ref) <= 1e-2
    # tighter: bf16 rounding of an f32-accumulated result is within 1 bf16 ulp-ish of the oracle
    np.testing.assert_allclose(got, ref, rtol=1.6e-2, atol=2e-3)


@pytest.mark.parametrize("variant", ["bf16_256x256x64_q2x4", "bf16_128x128x64_q2x2", "bf16_256x256x64_r2x4", "bf16_128x128x64_r2x2"])
@pytest.mark.parametrize("k_tiles", [1, 2, 3, 6, 7, 13])
def test_gemm_ring_pipeline_every_loop_shape(ct, dev, variant, k_tiles):
    # the ring pipeline repeats its stage names every 6 K tiles: cover the unrolled
    # loop, every remainder, and M, N that are not multiples of the tile
    bm, bn = (int(v) for v in variant.split("_")[1].split("x")[:2])
    m, n, k = 328, 520, 64 * k_tiles
    a, b = normal_bf16_bits((m, k), 331 + k_tiles, k ** -0.5), normal_bf16_bits((k, n), 332 + k_tiles, k ** -0.5)
    z = torch.zeros(m, n, dtype=torch.bfloat16, device=dev)
    ct.gemm(ct.partition(z, [bm, bn]), to_dev_bf16(a, dev), to_dev_bf16(b, dev), k, accumulate=False, variant=variant)
    sync()
    ref = oracle.gemm_bf16(a, b, f32out=True)
    np.testing.assert_allclose(z.float().cpu().numpy(), ref, rtol=1.6e-2, atol=2e-3)


@pytest.mark.parametrize("k", [8, 40, 64, 72, 200, 328])
def test_gemm_16x16x32_ring_masks_a_ragged_last_k_tile(ct, dev, k):
    # K is any multiple of 8: the last K tile is partly (or, for K < 64, mostly) beyond K and reads zeros; y may also
    # have fewer rows than K says
    m, n = 300, 520
    a, b = normal_bf16_bits((m, k), 341 + k, k ** -0.5), normal_bf16_bits((k, n), 342 + k, k ** -0.5)
    z = torch.full((m, n), 7.0, dtype=torch.bfloat16, device=dev)
    ct.gemm(ct.partition(z, [256, 256]), to_dev_bf16(a, dev), to_dev_bf16(b, dev), k, accumulate=False, generics=["bf16", 256, 256, 8],
            variant="bf16_256x256x64_q2x4")
    sync()
    ref = oracle.gemm_bf16(a, b, f32out=True)
    np.testing.assert_allclose(z.float().cpu().numpy(), ref, rtol=1.6e-2, atol=2e-3)


@pytest.mark.parametrize("variant,k,accumulate", [("bf16_128x128x64_q2x2", 200, False), ("bf16_128x128x64_q2x2", 448, True),
                                                  ("f16_128x128x64_q2x2", 328, True)])
def test_gemm_16x16x32_ring_at_128x128(ct, dev, variant, k, accumulate):
    # the same ring on four wavefronts (two workgroups to a compute unit): ragged K, ragged M and N, z as the initial
    # accumulator, both 16-bit operand types
    f16 = variant.startswith("f16")
    bits, to_dev, to_f32 = (normal_f16_bits, to_dev_f16, oracle.f16_bits_to_f32) if f16 else (normal_bf16_bits, to_dev_bf16, oracle.bf16_bits_to_f32)
    m, n = 300, 520
    a, b = bits((m, k), 351 + k, k ** -0.5), bits((k, n), 352 + k, k ** -0.5)
    z0 = bits((m, n), 353 + k, 0.5)
    z = to_dev(z0, dev).clone()
    ct.gemm(ct.partition(z, [128, 128]), to_dev(a, dev), to_dev(b, dev), k, accumulate=accumulate, generics=["f16" if f16 else "bf16", 128, 128, 8],
            variant=variant)
    sync()
    ref = to_f32(a).astype(np.float64) @ to_f32(b).astype(np.float64) + (to_f32(z0) if accumulate else 0.0)
    np.testing.assert_allclose(z.float().cpu().numpy(), ref, rtol=1.6e-2, atol=4e-3)


def test_gemm_ring_variant_rejects_ragged_k(ct, dev):
    m = n = 256
    k = 96
    x = torch.ones(m, k, dtype=torch.bfloat16, device=dev)
    y = torch.ones(k, n, dtype=torch.bfloat16, device=dev)
    z = torch.zeros(m, n, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ct.CutileError, match="does not fit"):
        ct.gemm(ct.partition(z, [256, 256]), x, y, k, generics=["bf16", 256, 256, 32], variant="bf16_256x256x64_r2x4")
    ct.gemm(ct.partition(z, [256, 256]), x, y, k, generics=["bf16", 256, 256, 32])  # falls back to a two-stage variant
    sync()
    assert torch.equal(z.float(), torch.full((m, n), float(k), device=dev))


def test_gemm_ones_known_answer_non_divisible(ct, dev):
    # cutile/tests/slice_non_divisible.rs:459-500: ones x ones = K, M and N not multiples of the tile
    m, n, k = 200, 264, 128
    x = torch.ones(m, k, dtype=torch.bfloat16, device=dev)
    y = torch.ones(k, n, dtype=torch.bfloat16, device=dev)
    z = torch.zeros(m, n, dtype=torch.bfloat16, device=dev)
    ct.gemm(ct.partition(z, [128, 128]), x, y, k)
    sync()
    assert torch.equal(z.float(), torch.full((m, n), float(k), device=dev))


def test_gemm_any_layout_reference_f32_case_and_odd_layouts(ct, dev):
    # cutile/tests/slice_non_divisible.rs:458-497 as the reference runs it: f32, tiles 16x16x8, M = N = 100
    m, n, k = 100, 100, 64
    z = torch.zeros(m, n, device=dev)
    ct.gemm(ct.partition(z, [16, 16]), torch.ones(m, k, device=dev), torch.ones(k, n, device=dev), k,
            generics=["f32", 16, 16, 8])
    sync()
    assert torch.all((z - float(k)).abs() < 1e-3)
    # random f32 against the oracle's cpu_gemm; y passed as a transposed view (inner stride != 1), z accumulated into
    m, n, k = 77, 53, 40
    x, y = oracle.normal_f32((m, k), 341), oracle.normal_f32((k, n), 342)
    z0 = oracle.normal_f32((m, n), 343)
    z = torch.from_numpy(z0.copy()).to(dev)
    yt = torch.from_numpy(np.ascontiguousarray(y.T)).to(dev).t()
    ct.gemm(ct.partition(z, [32, 16]), torch.from_numpy(x).to(dev), yt, k, accumulate=True, generics=["f32", 32, 16, 8])
    sync()
    np.testing.assert_allclose(z.cpu().numpy(), oracle.cpu_gemm_f32(x, y) + z0, rtol=1e-5, atol=1e-5)
    # bf16 with N not a multiple of 8 (rows not 16-byte aligned): the matrix-core variants cannot take it
    m, n, k = 130, 100, 96
    a, b = normal_bf16_bits((m, k), 344, k ** -0.5), normal_bf16_bits((k, n), 345, k ** -0.5)
    z = torch.zeros(m, n, dtype=torch.bfloat16, device=dev)
    ct.gemm(ct.partition(z, [128, 128]), to_dev_bf16(a, dev), to_dev_bf16(b, dev), k, accumulate=False,
            generics=["bf16", 128, 128, 32])
    sync()
    assert rel_l2(z.float().cpu().numpy(), oracle.gemm_bf16(a, b, f32out=True)) <= 1e-2
    # f16 in, f16 out; only the first tile row is launched (prefix coverage): the rest of z stays untouched
    m, n, k = 64, 48, 32
    xh = torch.from_numpy(oracle.f32_to_f16_bits(oracle.normal_f32((m, k), 346)).view(np.float16)).to(dev)
    yh = torch.from_numpy(oracle.f32_to_f16_bits(oracle.normal_f32((k, n), 347)).view(np.float16)).to(dev)
    z = torch.full((m, n), 7.0, dtype=torch.float16, device=dev)
    ct.gemm(ct.partition(z, [16, 16], prefix=True), xh, yh, k, accumulate=False, grid=(1, 3, 1), generics=["f16", 16, 16, 16])
    sync()
    ref = xh.float() @ yh.float()
    assert torch.allclose(z[:16].float(), ref[:16], rtol=2e-3, atol=2e-3) and torch.all(z[16:] == 7.0)


def test_gemm_accumulates_into_z_and_f32_out(ct, dev):
    m = n = k = 256
    a, b = normal_bf16_bits((m, k), 311, k ** -0.5), normal_bf16_bits((k, n), 312, k ** -0.5)
    z0 = oracle.normal_f32((m, n), 313)
    z = torch.from_numpy(z0.copy()).to(dev)
    ct.gemm(ct.partition(z, [128, 128]), to_dev_bf16(a, dev), to_dev_bf16(b, dev), k, accumulate=True)
    sync()
    ref = oracle.gemm_bf16(a, b, f32out=True) + z0
    np.testing.assert_allclose(z.cpu().numpy(), ref, rtol=1e-4, atol=1e-4)


def test_gemm_k_not_multiple_of_kernel_tile(ct, dev):
    m, n, k = 128, 128, 96                    # three BK=32 tiles of the tile program, 1.5 kernel K tiles
    a, b = normal_bf16_bits((m, k), 321, k ** -0.5), normal_bf16_bits((k, n), 322, k ** -0.5)
    z = torch.zeros(m, n, dtype=torch.float32, device=dev)
    ct.gemm(ct.partition(z, [128, 128]), to_dev_bf16(a, dev), to_dev_bf16(b, dev), k, accumulate=False,
            generics=["bf16", 128, 128, 32])
    sync()
    np.testing.assert_allclose(z.cpu().numpy(), oracle.gemm_bf16(a, b, f32out=True), rtol=1e-4, atol=1e-4)


# ---- K5: FMHA -------------------------------------------------------------------------------
def _fmha_case(ct, dev, b, h, hkv, s, d, bm, causal, input_pos, dtype=torch.bfloat16, variant=None, seed=401):
    rnd = lambda shape, sd: oracle.normal_f32(shape, sd)
    cast = (lambda x: oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(x))) if dtype == torch.bfloat16 else (
        lambda x: oracle.f16_bits_to_f32(oracle.f32_to_f16_bits(x)))
    q, k, v = cast(rnd((b, h, s, d), seed)), cast(rnd((b, hkv, s, d), seed + 1)), cast(rnd((b, hkv, s, d), seed + 2))
    out = torch.zeros(b * h, s, d, dtype=dtype, device=dev)
    td = lambda t: torch.from_numpy(t).to(dev).to(dtype)
    scale = 1.0 / np.sqrt(d)
    ct.fmha(ct.partition(out, [1, bm, d]), td(q), td(k), td(v), scale, input_pos, h // hkv, causal=causal,
            variant=variant)
    sync()
    ref = oracle.fmha_ref_cpu(q, k, v, scale, input_pos, h // hkv, causal).reshape(b * h, s, d)
    got = out.float().cpu().numpy()
    assert np.isfinite(got).all()
    return np.max(np.abs(got - ref))


@pytest.mark.parametrize("causal,input_pos", [(False, 0), (True, 5), (True, 0)])
def test_fmha_reference_example_shape(ct, dev, causal, input_pos):
    # cutile-examples/examples/flash_attention_causal.rs:216-222: (2, 8, 8, 64, 32), tiles (32, 32)
    assert _fmha_case(ct, dev, 2, 8, 8, 64, 32, 32, causal, input_pos) <= 2e-2


@pytest.mark.parametrize("variant", ["bf16_128x64x128", "bf16_128x128x128", "bf16_256x64x128", "bf16_256x64x128_pp"])
@pytest.mark.parametrize("causal", [False, True])
def test_fmha_d128(ct, dev, variant, causal):
    bm = int(variant.split("_")[1].split("x")[0])
    assert _fmha_case(ct, dev, 1, 2, 2, 512, 128, bm, causal, 0, variant=variant) <= 2e-2


@pytest.mark.parametrize("s,causal,input_pos", [(64, False, 0), (128, True, 0), (192, True, 3), (320, False, 0),
                                                 (1000, True, 0), (1000, False, 0), (1536, True, 17)])
def test_fmha_pingpong_every_loop_shape(ct, dev, s, causal, input_pos):
    # 1, 2, 3, 5 and many KV tiles (the pipeline is unrolled by two and peels its last
    # tile), ragged sequence ends, causal offsets, two kv heads shared by four query heads
    assert _fmha_case(ct, dev, 1, 4, 2, s, 128, 256, causal, input_pos, variant="bf16_256x64x128_pp", seed=431) <= 2e-2


@pytest.mark.parametrize("s,input_pos", [(256, 0), (320, 0), (448, 64), (512, 40), (704, 100), (832, 130), (576, 200)])
def test_fmha_pingpong_causal_halves_stop_at_their_own_last_tile(ct, dev, s, input_pos):
    # under a causal mask the upper 128 rows of a 256-row query tile run as the trailing half of the workgroup and
    # multiply only the KV tiles they can see (zero, one or two fewer than the lower rows, at either parity of the
    # unrolled-by-two pipeline); positions that start inside a KV tile, and key ranges that end before the queries do
    assert _fmha_case(ct, dev, 1, 2, 1, s, 128, 256, True, input_pos, variant="bf16_256x64x128_pp", seed=451 + s) <= 2e-2


def test_fmha_pingpong_f16(ct, dev):
    assert _fmha_case(ct, dev, 1, 2, 2, 640, 128, 256, True, 0, dtype=torch.float16, variant="f16_256x64x128_pp") <= 2e-2


def test_fmha_gqa_and_ragged_lengths(ct, dev):
    # 4 query heads share 2 kv heads; seq 200 is not a multiple of BM=64 or BN=64
    assert _fmha_case(ct, dev, 1, 4, 2, 200, 64, 64, True, 0) <= 2e-2
    assert _fmha_case(ct, dev, 1, 4, 2, 200, 64, 64, False, 0) <= 2e-2


@pytest.mark.parametrize("causal", [False, True])
def test_fmha_d256(ct, dev, causal):
    """head dimension 256 (128 x 32 tiles, accumulators in the second register file), grouped heads, ragged length"""
    assert _fmha_case(ct, dev, 1, 4, 2, 300, 256, 128, causal, 0, seed=441) <= 2e-2
    assert _fmha_case(ct, dev, 1, 2, 2, 256, 256, 128, causal, 7, dtype=torch.float16, seed=442) <= 2e-2


def test_fmha_f16(ct, dev):
    assert _fmha_case(ct, dev, 1, 2, 2, 256, 128, 128, True, 0, dtype=torch.float16) <= 2e-2


# ---- K6: MXFP8 GEMM -------------------------------------------------------------------------
def test_mxfp8_all_ones_known_answer(ct, dev):
    # cutile-examples/examples/mxfp8.rs:84-135: e4m3 0x38 (1.0), e8m0 0x7F (2^0) -> every output = K
    m = n = 16
    k = 128
    x = torch.full((m, k), 0x38, dtype=torch.uint8, device=dev)
    y = torch.full((n, k), 0x38, dtype=torch.uint8, device=dev)
    xs = torch.full((m, k // 32), 0x7F, dtype=torch.uint8, device=dev)
    ys = torch.full((n, k // 32), 0x7F, dtype=torch.uint8, device=dev)
    z = torch.zeros(m, n, device=dev)
    ct.linear_tile_mxfp8(ct.partition(z, [16, 16]), x, y, xs, ys, 1.0, generics=[16, 16, 64, 2])
    sync()
    assert torch.allclose(z, torch.full_like(z, float(k)), atol=1e-3)


@pytest.mark.parametrize("m,n,k,tile,out_dtype,variant", [
    (128, 128, 256, 128, torch.float32, None), (256, 256, 512, 256, torch.float32, None),
    (256, 256, 512, 256, torch.bfloat16, None), (512, 256, 384, 256, torch.bfloat16, "mxfp8_bf16_256x256x128_w2x4"),
    (96, 160, 256, 32, torch.float32, None), (64, 64, 128, 64, torch.float32, None),
    # the pipelined variants: one, two (a pair), three and seven K tiles; M, N off the tile
    (256, 256, 128, 256, torch.float32, "mxfp8_f32_256x256x128_d2x4"),
    (256, 512, 256, 256, torch.float32, "mxfp8_f32_256x256x128_d2x4"),
    (328, 520, 384, 256, torch.float32, "mxfp8_f32_256x256x128_d2x4"),
    (520, 328, 896, 256, torch.bfloat16, "mxfp8_bf16_256x256x128_d2x4"),
    (328, 520, 896, 256, torch.bfloat16, "mxfp8_bf16_256x256x128_d4x2"),
    # the 16 x 16 x 128 matrix instruction: one, two, three, five and eight K tiles (every place in a scale block,
    # the loop of four and its remainders); M, N off the tile
    (256, 256, 128, 256, torch.float32, "mxfp8_f32_256x256x128_e4x2"),
    (256, 512, 256, 256, torch.float32, "mxfp8_f32_256x256x128_e4x2"),
    (328, 520, 384, 256, torch.float32, "mxfp8_f32_256x256x128_e4x2"),
    (520, 328, 640, 256, torch.float32, "mxfp8_f32_256x256x128_e4x2"),
    (328, 520, 896, 256, torch.bfloat16, "mxfp8_bf16_256x256x128_e4x2"),
    (512, 768, 1024, 256, torch.bfloat16, "mxfp8_bf16_256x256x128_e4x2"),
    (512, 512, 1024, 256, torch.bfloat16, "mxfp8_bf16_256x256x128_w2x2"),
])
def test_mxfp8_random_blocks(ct, dev, m, n, k, tile, out_dtype, variant):
    # per-row scale spread exercises distinct e8m0 codes per 32-block
    xf = oracle.normal_f32((m, k), 501) * np.exp2(oracle.uniform_f32((m, k // 32), 503, -6, 6)).repeat(32, axis=1)
    yf = oracle.normal_f32((n, k), 502) * np.exp2(oracle.uniform_f32((n, k // 32), 504, -6, 6)).repeat(32, axis=1)
    xq, xs = oracle.mx_quantize_e4m3(xf)
    yq, ys = oracle.mx_quantize_e4m3(yf)
    assert len(np.unique(xs)) > 4
    z = torch.zeros(m, n, dtype=out_dtype, device=dev)
    td = lambda t: torch.from_numpy(t).to(dev)
    ct.linear_tile_mxfp8(ct.partition(z, [tile, tile]), td(xq), td(yq), td(xs), td(ys), 0.5, variant=variant)
    sync()
    ref = oracle.mx_gemm_f32(xq, yq, xs, ys, 0.5)
    # Sign bits cleared: each element's sum of |products|.  The scaled matrix instruction adds the 64 products of a
    # step aligned to the largest of them and keeps about 14 bits below it: measured, an element is within 4.5e-5 of
    # this sum of the exactly accumulated value, so 1e-4 of it is the absolute term (one missing product is ~1/K of it).
    mag = oracle.mx_gemm_f32(xq & 0x7F, yq & 0x7F, xs, ys, 0.5)
    got = z.float().cpu().numpy()
    tol = 3e-2
    assert rel_l2(got, ref) <= tol
    if out_dtype == torch.float32:      # exact products of fp8 values: only summation order differs
        assert rel_l2(got, ref) <= 1e-4
        assert_rounded_close(got, ref, (tile, tile), rel_ulp=1e-5, atol_frac=1e-4, what="mxfp8 f32", mag=mag)
    else:                               # bf16 output: the f32 sum rounded once
        assert_rounded_close(got, ref, (tile, tile), atol_frac=1e-4, what="mxfp8 bf16", mag=mag)
