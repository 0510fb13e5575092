"""The headline configurations at their full sizes, through the C ABI.

The oracle cannot evaluate a whole 8192^3 product or 4 x 32 x 4096^2 attention scores in seconds, so each case
is checked two ways: against the oracle on a seeded sample of output rows (same tolerances as the small cases:
saxpy bit exact; RMSNorm / softmax within 1 f16 ulp; bf16 GEMM rel-L2 <= 1e-2; FMHA max-abs <= 2e-2; MXFP8
rel-L2 <= 3e-2) and, over the WHOLE output, through properties that do not depend on the size:
products with the identity and with all-ones operands are exact (cutile/tests/slice_non_divisible.rs:459-500,
cutile-examples/examples/mxfp8.rs:91-135, nvfp4.rs:96-160), softmax rows sum to 1
(cutile-examples/examples/softmax.rs:55-60), normalised rows have unit mean square, and attention with zero
queries returns the mean of the visible V rows."""
import numpy as np
import pytest
import torch

import oracle
from util import assert_rounded_close, f16_ulp_diff, from_dev_f16_bits, normal_f16_bits, rel_l2, to_dev_bf16, to_dev_f16

pytestmark = pytest.mark.gpu

M_ROWS, N_COLS = 16384, 8192


def _sample(total, count, seed):
    return np.sort(np.random.default_rng(seed).choice(total, size=count, replace=False)).astype(np.int64)


def test_saxpy_16m_bit_exact(ct, dev):
    n = 1 << 24
    x, y = oracle.uniform_f32(n, 1), oracle.uniform_f32(n, 2)
    yd = torch.from_numpy(y.copy()).to(dev)
    ct.saxpy(ct.partition(yd, [1024]), 2.0, torch.from_numpy(x).to(dev))
    torch.cuda.synchronize()
    assert np.array_equal(yd.cpu().numpy(), oracle.saxpy_f32(2.0, x, y))


def test_rms_norm_16384x8192(ct, dev):
    xb = normal_f16_bits((M_ROWS, N_COLS), 3)
    wb = oracle.f32_to_f16_bits(oracle.uniform_f32(N_COLS, 4, 0.5, 1.5))
    x, w = to_dev_f16(xb, dev), to_dev_f16(wb, dev)
    out = torch.zeros(M_ROWS, N_COLS, dtype=torch.float16, device=dev)
    ct.rms_norm_f16(x, w, ct.partition(out, [1, N_COLS]), 1e-6)
    torch.cuda.synchronize()
    rows = _sample(M_ROWS, 256, 5)
    ref = oracle.rms_norm_f16(np.ascontiguousarray(xb[rows]), wb, 1e-6)
    got = from_dev_f16_bits(out[torch.from_numpy(rows).to(dev)])
    assert f16_ulp_diff(got, ref).max() <= 1
    # every row: out / w has unit mean square (f16 rounding of the outputs: a few 1e-4)
    ms = ((out.float() / w.float()) ** 2).mean(dim=1)
    assert torch.all(torch.isfinite(ms)) and float((ms - 1.0).abs().max()) < 2e-3


def test_softmax_16384x8192(ct, dev):
    xb = normal_f16_bits((M_ROWS, N_COLS), 6, 2.0)
    x = to_dev_f16(xb, dev)
    y = torch.zeros(M_ROWS, N_COLS, dtype=torch.float16, device=dev)
    ct.softmax(x, ct.partition(y, [1, N_COLS]))
    torch.cuda.synchronize()
    rows = _sample(M_ROWS, 256, 7)
    ref = oracle.softmax_f16(np.ascontiguousarray(xb[rows]), 1, N_COLS)
    got = from_dev_f16_bits(y[torch.from_numpy(rows).to(dev)])
    assert f16_ulp_diff(got, ref).max() <= 1
    sums = y.float().sum(dim=1)
    assert float((sums - 1.0).abs().max()) < 2e-3                     # 8192 f16 roundings per row
    peak = x.float().amax(dim=1, keepdim=True)
    assert torch.all((y.float().amax(dim=1, keepdim=True) == y.float())[x.float() == peak])   # the maximum stays the maximum


@pytest.mark.parametrize("s", [4096, 8192])
def test_gemm_bf16_full_size(ct, dev, s):
    ab = oracle.f32_to_bf16_bits(oracle.normal_f32((s, s), 8, 0, s ** -0.5))
    bb = oracle.f32_to_bf16_bits(oracle.normal_f32((s, s), 9, 0, s ** -0.5))
    a, b = to_dev_bf16(ab, dev), to_dev_bf16(bb, dev)
    z = torch.zeros(s, s, dtype=torch.bfloat16, device=dev)
    zp = ct.partition(z, [256, 256])
    ct.gemm(zp, a, b, s, accumulate=True)                             # the benchmark's form: z is the initial accumulator
    torch.cuda.synchronize()
    rows = _sample(s, 64, 10)
    ref = oracle.gemm_bf16(ab, bb, rows=rows, f32out=True)
    idx = torch.from_numpy(rows).to(dev)
    assert rel_l2(z[idx].float().cpu().numpy(), ref) <= 1e-2
    # element by element on the sampled rows: one bf16 rounding of the f32 sum (the sample spans every column tile)
    assert_rounded_close(z[idx].float().cpu().numpy(), ref, (len(rows), 256), what=f"gemm {s}")
    ct.gemm(zp, a, b, s, accumulate=True)                             # a second pass adds the same product again
    torch.cuda.synchronize()
    assert rel_l2(z[idx].float().cpu().numpy(), 2.0 * ref) <= 1e-2
    # A . I = A, bit for bit, over the whole output; ones . ones = K everywhere
    eye = torch.eye(s, dtype=torch.bfloat16, device=dev)
    ct.gemm(zp, a, eye, s, accumulate=False)
    torch.cuda.synchronize()
    assert torch.equal(z, a)
    ones = torch.ones(s, s, dtype=torch.bfloat16, device=dev)
    ct.gemm(zp, ones, ones, s, accumulate=False)
    torch.cuda.synchronize()
    assert torch.all(z == float(s))


@pytest.mark.parametrize("causal", [False, True])
def test_fmha_4x32x4096x128(ct, dev, causal):
    b, h, s, d = 4, 32, 4096, 128
    qb, kb, vb = (oracle.f32_to_bf16_bits(oracle.normal_f32((b, h, s, d), 11 + i)) for i in range(3))
    q, k, v = (to_dev_bf16(t, dev) for t in (qb, kb, vb))
    o = torch.zeros(b * h, s, d, dtype=torch.bfloat16, device=dev)
    op = ct.partition(o, [1, 256, d])
    ct.fmha(op, q, k, v, d ** -0.5, 0, 1, causal=causal)
    torch.cuda.synchronize()
    rows = _sample(b * h * s, 4096, 14)
    ref = oracle.fmha_ref_cpu(*(oracle.bf16_bits_to_f32(t) for t in (qb, kb, vb)), d ** -0.5, 0, 1, causal, rows=rows)
    got = o.reshape(b * h * s, d)[torch.from_numpy(rows).to(dev)].float().cpu().numpy()
    assert float(np.max(np.abs(got - ref))) <= 2e-2
    # zero queries: uniform weights over the visible keys, so every output row is their mean V row
    ct.fmha(op, torch.zeros_like(q), k, v, d ** -0.5, 0, 1, causal=causal)
    torch.cuda.synchronize()
    vf = v.reshape(b * h, s, d).float()
    if causal:
        want = vf.cumsum(dim=1) / torch.arange(1, s + 1, device=dev, dtype=torch.float32)[None, :, None]
    else:
        want = vf.mean(dim=1, keepdim=True).expand(-1, s, -1)
    assert float((o.float() - want).abs().max()) <= 2e-2


def test_mxfp8_8192(ct, dev):
    s = 8192
    xq, xs = oracle.mx_quantize_e4m3(oracle.normal_f32((s, s), 15))
    yq, ys = oracle.mx_quantize_e4m3(oracle.normal_f32((s, s), 16))
    td = lambda t: torch.from_numpy(t).to(dev)
    z = torch.zeros(s, s, dtype=torch.bfloat16, device=dev)
    zp = ct.partition(z, [256, 256])
    ct.linear_tile_mxfp8(zp, td(xq), td(yq), td(xs), td(ys), 1.0)
    torch.cuda.synchronize()
    rows = _sample(s, 32, 17)
    ref = oracle.mx_gemm_f32(xq, yq, xs, ys, 1.0, rows=rows)
    assert rel_l2(z[torch.from_numpy(rows).to(dev)].float().cpu().numpy(), ref) <= 3e-2
    assert_rounded_close(z[torch.from_numpy(rows).to(dev)].float().cpu().numpy(), ref, (len(rows), 256), what="mxfp8 8192")
    # cutile-examples/examples/mxfp8.rs:91-135 at full size: e4m3 1.0 (0x38) and e8m0 2^0 (0x7F) everywhere -> K
    one = torch.full((s, s), 0x38, dtype=torch.uint8, device=dev)
    unit = torch.full((s, s // 32), 0x7F, dtype=torch.uint8, device=dev)
    ct.linear_tile_mxfp8(zp, one, one, unit, unit, 1.0)
    torch.cuda.synchronize()
    assert torch.all(z == float(s))


def test_nvfp4_8192_all_ones(ct, dev):
    # cutile-examples/examples/nvfp4.rs:96-160 at full size: nibble 0x2 = 1.0, scale 0x38 = 1.0 -> K
    s = 8192
    x = torch.full((s, s // 2), 0x22, dtype=torch.uint8, device=dev)
    sc = torch.full((s, s // 16), 0x38, dtype=torch.uint8, device=dev)
    z = torch.zeros(s, s, dtype=torch.bfloat16, device=dev)
    ct.linear_tile_nvfp4(ct.partition(z, [256, 256]), x, x, sc, sc, 1.0)
    torch.cuda.synchronize()
    assert torch.all(z == float(s))
