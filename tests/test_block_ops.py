"""Transformer-block kernels of cutile-kernels (norms.rs, pointwise.rs, positional.rs): the
oracle's restatements pinned by closed forms and library routines (CPU), then the HIP kernels
against the oracle through the C ABI (GPU).  The reference has no numeric test for any of them
(cutile-kernels/tests/smoke.rs compiles them only), so parity is pinned by the mathematics."""
import numpy as np
import pytest
import torch
from scipy.special import expit

import oracle
from util import f16_ulp_diff, normal_f16_bits

f16 = lambda a: oracle.f32_to_f16_bits(np.asarray(a, np.float32))
f32 = oracle.f16_bits_to_f32


# ---- oracle (CPU) ---------------------------------------------------------------------------
def test_oracle_add_rms_norm_reduces_to_rms_norm_and_keeps_the_sum_unrounded():
    x, w = normal_f16_bits((6, 96), 601), f16(oracle.uniform_f32((96,), 602, 0.5, 1.5))
    zero = f16(np.zeros((6, 96)))
    out, res = oracle.add_rms_norm_f16(zero, x, w, 1e-6)
    assert np.array_equal(out, oracle.rms_norm_f16(x, w, 1e-6)) and np.array_equal(res, x)
    # residual + x is normalised BEFORE rounding to f16: 1 + 2^-11 is lost by the f16 residual, not by the norm
    r = f16(np.full((1, 8), 1.0)); xx = f16(np.full((1, 8), 2.0 ** -11)); ones = f16(np.ones(8))
    out, res = oracle.add_rms_norm_f16(r, xx, ones, 0.0)
    assert np.all(f32(res) == 1.0)                       # 1 + 2^-11 rounds to 1 in f16 (tie to even)
    assert np.all(f32(out) == 1.0)                       # (1 + 2^-11) / rms(1 + 2^-11) = 1 exactly
    # float64 evaluation of the definition
    r, xx = normal_f16_bits((5, 200), 603), normal_f16_bits((5, 200), 604)
    w = f16(oracle.uniform_f32((200,), 605, 0.5, 1.5))
    out, res = oracle.add_rms_norm_f16(r, xx, w, 1e-5, block=64)
    c = f32(r).astype(np.float64) + f32(xx).astype(np.float64)
    ref = c / np.sqrt((c * c).mean(axis=1, keepdims=True) + 1e-5) * f32(w)
    assert np.max(f16_ulp_diff(out, f16(ref))) <= 1 and np.array_equal(res, f16(c))


def test_oracle_qk_norm_is_rms_norm_on_stacked_rows_with_two_weights():
    q, k = normal_f16_bits((5, 128), 611), normal_f16_bits((3, 128), 612)
    qw, kw = f16(oracle.uniform_f32((128,), 613, 0.5, 1.5)), f16(oracle.uniform_f32((128,), 614, 0.5, 1.5))
    out = oracle.qk_norm_f16(q, k, qw, kw, 1e-6)
    assert out.shape == (8, 128)
    assert np.array_equal(out[:5], oracle.rms_norm_f16(q, qw, 1e-6)) and np.array_equal(out[5:], oracle.rms_norm_f16(k, kw, 1e-6))
    assert not np.array_equal(out[5:], oracle.rms_norm_f16(k, qw, 1e-6))      # the k rows really use k_weight


def test_oracle_pointwise_vs_library():
    a, b = normal_f16_bits((7, 33), 621, 4.0), normal_f16_bits((7, 33), 622, 4.0)
    assert np.array_equal(oracle.add_f16(a, b), (a.view(np.float16) + b.view(np.float16)).view(np.uint16))
    got = oracle.silu_mul_f16(a, b)
    g, u = f32(a).astype(np.float64), f32(b).astype(np.float64)
    assert np.max(f16_ulp_diff(got, f16(expit(g) * g * u))) <= 1
    # known values: silu(0) = 0; large gate -> gate * up; large negative gate -> 0
    k = oracle.silu_mul_f16(f16([0.0, 20.0, -20.0]), f16([3.0, 0.5, 7.0]))
    assert f32(k).tolist() == [0.0, 10.0, -0.0] or np.allclose(f32(k), [0.0, 10.0, 0.0], atol=1e-6)


def test_oracle_rope_is_a_rotation_by_position_times_frequency():
    seq, heads, d = 9, 3, 16
    x = normal_f16_bits((seq, heads, d), 631)
    inv_freq = (1.0 / 10000.0 ** (np.arange(d // 2) / (d // 2))).astype(np.float32)
    y = f32(oracle.rope_seq_f16(x, inv_freq, 5)).astype(np.float64)
    xf = f32(x).astype(np.float64)
    z = (xf[..., : d // 2] + 1j * xf[..., d // 2:]) * np.exp(1j * (5 + np.arange(seq))[:, None, None] * inv_freq.astype(np.float64))
    ref = np.concatenate([z.real, z.imag], axis=-1)
    assert np.max(np.abs(y - ref)) < 4e-3                                        # f16 output, |x| up to ~4
    assert np.allclose(np.hypot(y[..., : d // 2], y[..., d // 2:]), np.abs(z), atol=6e-3)   # norms of pairs kept
    assert np.array_equal(oracle.rope_seq_f16(x[:1], inv_freq, 0), x[:1])      # position 0: identity
    # a quarter turn swaps and negates: theta = pi/2 -> (lo, hi) -> (-hi, lo)
    q = oracle.rope_seq_f16(f16(np.array([[[1.0, 2.0]]])), np.array([np.pi / 2], np.float32), 1)
    assert np.allclose(f32(q).ravel(), [-2.0, 1.0], atol=2e-3)


# ---- HIP kernels (GPU) -----------------------------------------------------------------------
def _dev(bits, dev):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.float16)).to(dev)


def _bits(t):
    return t.cpu().numpy().view(np.uint16)


@pytest.mark.gpu
@pytest.mark.parametrize("rows,n,variant", [(33, 128, None), (64, 4096, None), (16, 8192, "w4v4"), (7, 1000, None), (5, 96, "generic")])
def test_gpu_add_rms_norm(ct, dev, rows, n, variant):
    r, x = normal_f16_bits((rows, n), 641), normal_f16_bits((rows, n), 642)
    w = f16(oracle.uniform_f32((n,), 643, 0.5, 1.5))
    out, res = torch.zeros(rows, n, dtype=torch.float16, device=dev), torch.zeros(rows, n, dtype=torch.float16, device=dev)
    ct.add_rms_norm_f16(_dev(r, dev), _dev(x, dev), _dev(w, dev), ct.partition(out, [1, n]), ct.partition(res, [1, n]), 1e-6,
                        variant=variant)
    torch.cuda.synchronize()
    ref_out, ref_res = oracle.add_rms_norm_f16(r, x, w, 1e-6)
    assert np.array_equal(_bits(res), ref_res)                      # the rounded sum is exact
    assert np.max(f16_ulp_diff(_bits(out), ref_out)) <= 1


@pytest.mark.gpu
@pytest.mark.parametrize("n", [4096, 8192, 1000])
def test_gpu_add_rms_norm_decode_raw(ct, dev, n):
    """cutile-kernels/src/experimental/norms.rs:22-153: the one-row raw-pointer form is add_rms_norm_f16 on [1, N]"""
    r, x = normal_f16_bits((1, n), 671), normal_f16_bits((1, n), 672)
    w = f16(oracle.uniform_f32((n,), 673, 0.5, 1.5))
    out, res = torch.zeros(n, dtype=torch.float16, device=dev), torch.zeros(n, dtype=torch.float16, device=dev)
    ct.add_rms_norm_decode_raw_f16(_dev(r, dev), _dev(x, dev), _dev(w, dev), out, res, 1e-6, generics=[n])
    torch.cuda.synchronize()
    ref_out, ref_res = oracle.add_rms_norm_f16(r, x, w, 1e-6)
    assert np.array_equal(_bits(res), ref_res[0]) and np.max(f16_ulp_diff(_bits(out), ref_out[0])) <= 1


@pytest.mark.gpu
@pytest.mark.parametrize("n,variant,q_rows,k_rows", [
    (128, None, 40, 8), (64, None, 40, 8), (256, "w1v1", 40, 8), (120, None, 40, 8),
    # many workgroups, a ragged last one, the q/k boundary inside one pass of one wavefront
    (128, None, 1003, 251), (64, None, 1001, 77), (256, None, 2050, 513), (128, "s32", 333, 90),
])
def test_gpu_qk_norm(ct, dev, n, variant, q_rows, k_rows):
    q, k = normal_f16_bits((q_rows, n), 651), normal_f16_bits((k_rows, n), 652)
    qw, kw = f16(oracle.uniform_f32((n,), 653, 0.5, 1.5)), f16(oracle.uniform_f32((n,), 654, 0.5, 1.5))
    out = torch.zeros(q_rows + k_rows, n, dtype=torch.float16, device=dev)
    ct.qk_norm_f16(_dev(q, dev), _dev(k, dev), _dev(qw, dev), _dev(kw, dev), ct.partition(out, [1, n]), 1e-6, q_rows, variant=variant)
    torch.cuda.synchronize()
    assert np.max(f16_ulp_diff(_bits(out), oracle.qk_norm_f16(q, k, qw, kw, 1e-6))) <= 1


@pytest.mark.gpu
def test_gpu_pointwise(ct, dev):
    for shape, block in (((64, 4096), 1024), ((33, 200), 64)):
        a, b = normal_f16_bits(shape, 661, 3.0), normal_f16_bits(shape, 662, 3.0)
        out = torch.zeros(*shape, dtype=torch.float16, device=dev)
        ct.add_2d_f16(ct.partition(out, [1, block]), _dev(a, dev), _dev(b, dev), generics=[block])
        torch.cuda.synchronize()
        assert np.array_equal(_bits(out), oracle.add_f16(a, b))
        ct.silu_mul_2d_f16(ct.partition(out, [1, block]), _dev(a, dev), _dev(b, dev))
        torch.cuda.synchronize()
        assert np.max(f16_ulp_diff(_bits(out), oracle.silu_mul_f16(a, b))) <= 1
    with pytest.raises(ct.CutileError, match="BLOCK_SIZE"):
        ct.silu_mul_2d_f16(ct.partition(out, [1, 64]), _dev(a, dev), _dev(b, dev), generics=[128])


@pytest.mark.gpu
def test_gpu_rope_three_forms(ct, dev):
    seq, qh, kh, d = 37, 6, 2, 128
    inv_freq = (1.0 / 10000.0 ** (np.arange(d // 2) / (d // 2))).astype(np.float32)
    fr = torch.from_numpy(inv_freq).to(dev)
    q, k = normal_f16_bits((seq, qh, d), 671), normal_f16_bits((seq, kh, d), 672)
    # rope_seq_f16: start position by value
    out = torch.zeros(seq, qh, d, dtype=torch.float16, device=dev)
    ct.rope_f16(ct.partition(out, [1, 1, d // 2]), _dev(q, dev), fr, 11, generics=[d, d // 2])
    torch.cuda.synchronize()
    assert np.max(f16_ulp_diff(_bits(out), oracle.rope_seq_f16(q, inv_freq, 11))) <= 1
    # rope_seq_dynpos_f16: start position from device memory
    pos = torch.tensor([1000], dtype=torch.int32, device=dev)
    ct.rope_f16(ct.partition(out, [1, 1, d // 2]), _dev(q, dev), fr, pos)
    torch.cuda.synchronize()
    assert np.max(f16_ulp_diff(_bits(out), oracle.rope_seq_f16(q, inv_freq, 1000))) <= 1
    # qk_rope_dynpos_f16: q heads then k heads in one output
    out2 = torch.zeros(seq, qh + kh, d, dtype=torch.float16, device=dev)
    ct.rope_f16(ct.partition(out2, [1, 1, d // 2]), _dev(q, dev), fr, pos, k=_dev(k, dev), num_q_heads=qh)
    torch.cuda.synchronize()
    ref = np.concatenate([oracle.rope_seq_f16(q, inv_freq, 1000), oracle.rope_seq_f16(k, inv_freq, 1000)], axis=1)
    assert np.max(f16_ulp_diff(_bits(out2), ref)) <= 1
    # odd head dimension halves (scalar path) and a strided input view
    d2 = 24
    inv2 = (1.0 / 100.0 ** (np.arange(d2 // 2) / (d2 // 2))).astype(np.float32)
    x = normal_f16_bits((5, 3, d2), 673)
    wide = torch.zeros(5, 3, d2 + 8, dtype=torch.float16, device=dev)
    wide[..., :d2] = _dev(x, dev)
    out3 = torch.zeros(5, 3, d2, dtype=torch.float16, device=dev)
    ct.rope_f16(ct.partition(out3, [1, 1, d2 // 2]), wide[..., :d2], torch.from_numpy(inv2).to(dev), 3)
    torch.cuda.synchronize()
    assert np.max(f16_ulp_diff(_bits(out3), oracle.rope_seq_f16(x, inv2, 3))) <= 1
