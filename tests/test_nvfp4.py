"""NVFP4 block-scaled GEMM (cutile-examples/examples/nvfp4.rs): packed e2m1 operands, one e4m3fn scale per 16 K
values, f32 accumulation.

CPU: the oracle's codecs and GEMM pinned by the e2m1 value table, torch's float8_e4m3fn, the reference example's
all-ones known answer (z = K) and a float64 evaluation.  GPU: the HIP kernel against the oracle; the kernel expands
the operands to f16 exactly, so results differ from the oracle only by the order of f32 additions (rel-L2 <= 1e-5;
small integer-valued cases are bit-exact)."""
import numpy as np
import pytest
import torch

import oracle
from util import assert_rounded_close, rel_l2

E2M1 = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]


# ---- oracle (CPU) ---------------------------------------------------------------------------
def test_oracle_e2m1_codec_is_the_ocp_value_table():
    assert [oracle.e2m1_to_f32(c) for c in range(8)] == E2M1
    assert [oracle.e2m1_to_f32(c | 8) for c in range(1, 8)] == [-v for v in E2M1[1:]]
    assert oracle.e2m1_to_f32(0x2) == 1.0                     # cuda-core/src/dtype.rs:228: one() is nibble 0x2
    for c in range(16):                                       # every code round-trips
        assert oracle.f32_to_e2m1(oracle.e2m1_to_f32(c)) == c or c == 8   # -0.0 keeps its sign bit
    # nearest value, ties to the even mantissa, saturation at 6
    assert [oracle.f32_to_e2m1(v) for v in (0.2, 0.25, 0.3, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 5.1, 100.0, -0.6)] == \
           [0, 0, 1, 2, 2, 4, 4, 6, 6, 7, 7, 9]


def test_oracle_nvfp4_layout_scales_and_known_answer():
    # the reference example: every value 1.0 (nibble 0x2, byte 0x22), every scale 1.0 (0x38) -> z = K
    m, n, k = 16, 16, 128
    x = np.full((m, k // 2), 0x22, np.uint8)
    s = np.full((m, k // 16), 0x38, np.uint8)
    z = oracle.nvfp4_gemm_f32(x, x[:n], s, s[:n], 1.0)
    assert z.shape == (m, n) and np.all(z == float(k))
    assert np.all(oracle.nvfp4_gemm_f32(x, x[:n], s, s[:n], 0.5) == 0.5 * k)      # alpha
    # low nibble is the first value of a pair (dtype.rs:60-99); one scale per 16 values
    data = np.zeros((1, 16), np.uint8)
    data[0, 0] = 0x72            # values 0 and 1: 1.0 (0x2), 6.0 (0x7)
    data[0, 8] = 0x0B            # value 16: -1.5 (0xB); value 17: 0
    scales = np.array([[0x40, 0x30]], np.uint8)               # e4m3fn 2.0 and 0.5
    dq = oracle.nvfp4_dequantize(data, scales)
    assert dq.shape == (1, 32) and dq[0, 0] == 2.0 and dq[0, 1] == 12.0 and dq[0, 16] == -0.75 and dq[0, 17] == 0.0
    # scales decode as torch's float8_e4m3fn for every byte that is not NaN
    codes = np.arange(256, dtype=np.uint8)
    ref = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    ones = np.full((256, 8), 0x22, np.uint8)
    got = oracle.nvfp4_dequantize(ones, codes.reshape(256, 1))[:, 0]
    ok = ~np.isnan(ref)
    assert np.array_equal(got[ok], ref[ok]) and np.all(np.isnan(got[~ok]))


def test_oracle_nvfp4_gemm_is_the_dequantised_product():
    m, n, k = 24, 40, 192
    xq, xs = oracle.nvfp4_quantize(oracle.normal_f32((m, k), 901))
    yq, ys = oracle.nvfp4_quantize(oracle.normal_f32((n, k), 902))
    z = oracle.nvfp4_gemm_f32(xq, yq, xs, ys, 1.5)
    xd, yd = oracle.nvfp4_dequantize(xq, xs).astype(np.float64), oracle.nvfp4_dequantize(yq, ys).astype(np.float64)
    assert rel_l2(z, 1.5 * xd @ yd.T) < 1e-6
    rows = np.array([3, 17], np.int64)
    assert np.array_equal(oracle.nvfp4_gemm_f32(xq, yq, xs, ys, 1.5, rows=rows), z[rows])
    # the quantiser (not in the reference): the block maximum maps onto the largest code, error within half a step
    src = oracle.normal_f32((8, 64), 903)
    q, s = oracle.nvfp4_quantize(src)
    dq = oracle.nvfp4_dequantize(q, s)
    sf = torch.from_numpy(s).view(torch.float8_e4m3fn).float().numpy().repeat(16, axis=1)
    assert np.all(np.abs(dq - src) <= sf * 1.0 + 1e-6)         # largest gap between neighbouring codes is 2 scale units
    assert np.all(np.abs(dq).reshape(8, 4, 16).max(axis=2) <= 6.0 * sf[:, ::16] + 1e-6)


# ---- HIP kernel (GPU) ------------------------------------------------------------------------
def _dev(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


@pytest.mark.gpu
def test_gpu_nvfp4_reference_example(ct, dev):
    """nvfp4.rs:96-160 as written: M = N = 16, K = 128, tiles 16x16x64, all ones -> every output is K"""
    m, n, k = 16, 16, 128
    x = torch.full((m, k // 2), 0x22, dtype=torch.uint8, device=dev)
    y = torch.full((n, k // 2), 0x22, dtype=torch.uint8, device=dev)
    xs = torch.full((m, k // 16), 0x38, dtype=torch.uint8, device=dev)
    ys = torch.full((n, k // 16), 0x38, dtype=torch.uint8, device=dev)
    z = torch.zeros(m, n, dtype=torch.float32, device=dev)
    ct.linear_tile_nvfp4(ct.partition(z, [16, 16]), x, y, xs, ys, 1.0, generics=[16, 16, 64, 32, 4])
    torch.cuda.synchronize()
    assert torch.all(z == float(k))
    with pytest.raises(ct.CutileError, match="BK_PACKED"):
        ct.linear_tile_nvfp4(ct.partition(z, [16, 16]), x, y, xs, ys, 1.0, generics=[16, 16, 64, 64, 4])
    with pytest.raises(ct.CutileError, match="scales must be"):
        ct.linear_tile_nvfp4(ct.partition(z, [16, 16]), x, y, xs[:, :4], ys, 1.0)


@pytest.mark.gpu
@pytest.mark.parametrize("m,n,k,tile,variant,out", [
    (256, 256, 256, 256, None, "f32"),
    (512, 768, 1024, 256, "f32_256x256x64_w4x2", "f32"),
    (512, 768, 1024, 256, "f32_256x256x64_w2x4", "f32"),
    (512, 768, 1024, 256, "f32_256x256x64_q4x2", "f32"),      # the 16 x 16 x 32 forms
    (1000, 264, 192, 256, "f32_256x256x64_q2x4", "f32"),
    (300, 520, 64, 256, "bf16_256x256x64_q4x2", "bf16"),
    (520, 264, 320, 256, "bf16_256x256x64_q2x4", "bf16"),
    (300, 520, 64, 256, "f32_256x256x64_w4x2", "f32"),       # one K tile
    (256, 256, 128, 256, "f32_256x256x64_w2x4", "f32"),      # two
    (1000, 264, 192, 256, "f32_256x256x64_w4x2", "f32"),     # three, ragged edges
    (256, 512, 256, 256, "f32_256x256x64_w2x4", "f32"),      # four
    (520, 264, 320, 256, "bf16_256x256x64_w4x2", "bf16"),    # five
    (300, 200, 192, 128, None, "f32"),                    # ragged edges
    (96, 160, 64, 32, None, "f32"),                       # one K tile, smallest kernel tile
    (128, 128, 128, 64, None, "f32"),
    (520, 264, 320, 256, None, "bf16"),
    (256, 384, 512, 128, None, "bf16"),
])
def test_gpu_nvfp4_gemm(ct, dev, m, n, k, tile, variant, out):
    xq, xs = oracle.nvfp4_quantize(oracle.normal_f32((m, k), 911))
    yq, ys = oracle.nvfp4_quantize(oracle.normal_f32((n, k), 912))
    dt = torch.float32 if out == "f32" else torch.bfloat16
    z = torch.full((m, n), float("nan"), dtype=dt, device=dev)
    ct.linear_tile_nvfp4(ct.partition(z, [tile, tile]), _dev(xq, dev), _dev(yq, dev), _dev(xs, dev), _dev(ys, dev), 0.75, variant=variant)
    torch.cuda.synchronize()
    ref = oracle.nvfp4_gemm_f32(xq, yq, xs, ys, 0.75)
    got = z.float().cpu().numpy()
    assert np.all(np.isfinite(got))
    assert rel_l2(got, ref) <= (1e-5 if out == "f32" else 4e-3)     # f32: order of additions only; bf16: output rounding
    # and element by element, the last (partial) tile's rows and columns on their own
    mag = oracle.nvfp4_gemm_f32(xq & 0x77, yq & 0x77, xs, ys, 0.75)      # sign bits of both nibbles cleared: sums of |products|
    assert_rounded_close(got, ref, (tile, tile), rel_ulp=1e-5 if out == "f32" else 2.0 ** -7, atol_frac=1e-4, what=f"nvfp4 {out}", mag=mag)


@pytest.mark.gpu
def test_gpu_nvfp4_every_code_and_scale_is_expanded_exactly(ct, dev):
    """x = one row per (code, scale) pair times a single 1.0 in y: the product is exactly value(code) * scale"""
    codes = np.arange(16, dtype=np.uint8)
    scale_bytes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], np.uint8)       # every e4m3fn byte but NaN
    m, k = 16 * len(scale_bytes), 64
    x = np.zeros((m, k // 2), np.uint8)
    xs = np.zeros((m, k // 16), np.uint8)
    for si, sb in enumerate(scale_bytes):
        for c in codes:
            r = si * 16 + int(c)
            x[r, 9] = int(c) << 4                 # value 19 (high nibble of byte 9), block 1
            xs[r, 1] = sb
    n = 32
    y = np.zeros((n, k // 2), np.uint8)
    y[:, 9] = 0x20                            # value 19 = 1.0
    ys = np.full((n, k // 16), 0x38, np.uint8)
    z = torch.zeros(m, n, dtype=torch.float32, device=dev)
    ct.linear_tile_nvfp4(ct.partition(z, [32, 32]), _dev(x, dev), _dev(y, dev), _dev(xs, dev), _dev(ys, dev), 1.0)
    torch.cuda.synchronize()
    ref = oracle.nvfp4_gemm_f32(x, y, xs, ys, 1.0)
    assert np.array_equal(z.cpu().numpy(), ref)
    want = np.array([oracle.e2m1_to_f32(int(c)) for c in codes], np.float32)[None, :] * \
        torch.from_numpy(scale_bytes).view(torch.float8_e4m3fn).float().numpy()[:, None]
    assert np.array_equal(ref[:, 0].reshape(len(scale_bytes), 16), want)
