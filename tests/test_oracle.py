"""Pins the CPU oracle (oracle/oracle.c) without the reference: against the known answers
the reference's own tests hold for this path, against library routines (numpy / torch /
scipy) and against what the mathematics fixes.  Each check is chosen so that a plausible
slip (dropped term, wrong sign or index, transposed operand, wrong rounding) fails it."""
import math
from fractions import Fraction

import numpy as np
import pytest
import torch

import oracle


# ---- codecs: exhaustive / library cross-checks ----------------------------------------------
def test_f16_decode_all_codes_vs_numpy():
    codes = np.arange(65536, dtype=np.uint16)
    ref = codes.view(np.float16).astype(np.float32)
    got = oracle.f16_bits_to_f32(codes)
    ok = ~np.isnan(ref)
    assert np.array_equal(got.view(np.uint32)[ok], ref.view(np.uint32)[ok]) and np.isnan(got[~ok]).all()


def test_f16_encode_rne_vs_numpy_including_ties_subnormals_overflow():
    x = np.concatenate([oracle.normal_f32(1 << 18, 1), oracle.normal_f32(1 << 18, 2, 0, 1e-6),
                        oracle.normal_f32(1 << 16, 3, 0, 3e4),
                        # exact ties and boundaries: halfway between representable halves
                        np.array([1.0 + 2 ** -11, 1.0 + 3 * 2 ** -11, 65504, 65519.99, 65520, 2 ** -24, 2 ** -25,
                                  1.5 * 2 ** -24, 2 ** -14, 2 ** -14 - 2 ** -25, 0.0, -0.0, np.inf, -np.inf], np.float32)])
    with np.errstate(over="ignore"):
        ref = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.f32_to_f16_bits(x), ref)


def test_bf16_encode_rne_vs_torch_and_decode_is_shift():
    x = np.concatenate([oracle.normal_f32(1 << 18, 4), np.array([1.0 + 2 ** -8, 1.0 + 3 * 2 ** -8, 3.3895314e38], np.float32)])
    ref = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = oracle.f32_to_bf16_bits(x)
    assert np.array_equal(got, ref)
    assert np.array_equal(oracle.bf16_bits_to_f32(got).view(np.uint32), got.astype(np.uint32) << 16)


def test_e4m3fn_and_e8m0_decode_all_256_codes_vs_torch():
    codes = torch.arange(256, dtype=torch.uint8)
    t8 = codes.view(torch.float8_e4m3fn).float().numpy()
    mine = np.array([oracle.e4m3fn_to_f32(i) for i in range(256)], np.float32)
    assert np.array_equal(np.isnan(t8), np.isnan(mine)) and np.array_equal(t8[~np.isnan(t8)], mine[~np.isnan(mine)])
    t0 = codes.view(torch.float8_e8m0fnu).float().numpy()
    mine0 = np.array([oracle.e8m0_to_f32(i) for i in range(256)], np.float32)
    assert np.array_equal(np.isnan(t0), np.isnan(mine0)) and np.array_equal(t0[~np.isnan(t0)], mine0[~np.isnan(mine0)])
    # cuda-core/src/dtype.rs:225-227: one() is 0x38 for e4m3fn and 0x7F for e8m0fnu
    assert oracle.e4m3fn_to_f32(0x38) == 1.0 and oracle.e8m0_to_f32(0x7F) == 1.0
    assert oracle.e4m3fn_to_f32(0x7E) == 448.0 and np.isnan(oracle.e4m3fn_to_f32(0x7F))


def test_e4m3fn_encode_vs_torch_in_range_and_saturation_by_spec():
    xs = np.concatenate([oracle.uniform_f32(20000, 5, -448, 448), oracle.normal_f32(20000, 6, 0, 0.01),
                         np.array([2 ** -9, 2 ** -10, 1.5 * 2 ** -9, 0.0, -0.0, 448.0, 464.0], np.float32)])
    ref = torch.from_numpy(xs).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = np.array([oracle.f32_to_e4m3fn(v) for v in xs], np.uint8)
    assert np.array_equal(got, ref)
    assert oracle.f32_to_e4m3fn(480.0) == 0x7E and oracle.f32_to_e4m3fn(-1e9) == 0xFE  # saturating, not NaN
    assert oracle.f32_to_e4m3fn(float("nan")) == 0x7F
    # round trip of every finite code is the identity
    for c in range(256):
        v = oracle.e4m3fn_to_f32(c)
        if not np.isnan(v) and c != 0x80:
            assert oracle.f32_to_e4m3fn(v) == c


# ---- seeded inputs --------------------------------------------------------------------------
def test_prng_is_deterministic_thread_independent_and_distributed():
    a = oracle.normal_f32(1 << 16, 42)
    oracle.set_num_threads(1)
    b = oracle.normal_f32(1 << 16, 42)
    oracle.set_num_threads(oracle.num_threads() or 1)
    assert np.array_equal(a, b)
    assert not np.array_equal(a, oracle.normal_f32(1 << 16, 43))
    u = oracle.uniform_f32(1 << 20, 7, -1, 1)
    assert -1 <= u.min() and u.max() < 1 and abs(u.mean()) < 5e-3 and abs(u.var() - 1 / 3) < 5e-3
    n = oracle.normal_f32(1 << 20, 7)
    assert abs(n.mean()) < 5e-3 and abs(n.std() - 1) < 5e-3 and abs(((n - n.mean()) ** 3).mean()) < 2e-2


# ---- K1 -------------------------------------------------------------------------------------
def test_saxpy_reference_vectors_and_fused_rounding():
    # cutile-examples/examples/saxpy.rs:27-53: arange(32), a = 2 -> 2*x + x, exact
    x = np.arange(32, dtype=np.float32)
    assert np.array_equal(oracle.saxpy_f32(2.0, x, x), 3 * x)
    # one rounding, not two: a*x is inexact in f32 for these, fma rounds once
    a, xv, yv = np.float32(1 + 2 ** -12), np.float32(1 + 2 ** -12), np.float32(-1.0)
    fused = np.float32(np.float64(a) * np.float64(xv) + np.float64(yv))
    unfused = np.float32(np.float32(a * xv) + yv)
    assert fused != unfused
    assert oracle.saxpy_f32(float(a), np.array([xv]), np.array([yv]))[0] == fused
    # cutile/tests/gpu/add_basic.rs:29-43
    assert np.array_equal(oracle.add_f32(np.ones(128, np.float32), np.ones(128, np.float32)), np.full(128, 2, np.float32))


# ---- K2 -------------------------------------------------------------------------------------
def test_rms_norm_closed_forms():
    n = 64
    ones = oracle.f32_to_f16_bits(np.ones(n, np.float32))
    # x == c  =>  out = sign(c) * w  (eps -> 0)
    for c in (3.0, -0.5):
        x = oracle.f32_to_f16_bits(np.full((2, n), c, np.float32))
        w = oracle.f32_to_f16_bits(oracle.uniform_f32(n, 1, 0.5, 1.5))
        out = oracle.f16_bits_to_f32(oracle.rms_norm_f16(x, w, 0.0))
        assert np.array_equal(out, np.sign(c) * oracle.f16_bits_to_f32(w)[None, :].repeat(2, 0))
    # w == 1  =>  mean(out^2) ~ 1, and scale equivariance: rms_norm(2x) == rms_norm(x)
    xb = oracle.f32_to_f16_bits(oracle.normal_f32((8, 256), 2))
    o1 = oracle.f16_bits_to_f32(oracle.rms_norm_f16(xb, oracle.f32_to_f16_bits(np.ones(256, np.float32)), 0.0))
    assert np.allclose((o1 ** 2).mean(axis=1), 1.0, atol=2e-3)
    x2 = oracle.f32_to_f16_bits(2 * oracle.f16_bits_to_f32(xb))
    o2 = oracle.f16_bits_to_f32(oracle.rms_norm_f16(x2, oracle.f32_to_f16_bits(np.ones(256, np.float32)), 0.0))
    assert np.array_equal(o1, o2)
    # eps matters and sits inside the rsqrt: x = 0 -> out = 0 (not NaN) for eps > 0
    z = oracle.rms_norm_f16(np.zeros((1, n), np.uint16), ones, 1e-6)
    assert not z.any()


def test_rms_norm_brute_force_tiny_and_float64_agreement():
    x = np.array([[1, 2, 3, 4, -1, -2, -3, -4], [0.5, 0, 0, 0, 0, 0, 0, 0]], np.float32)
    w = np.array([1, 2, 0.5, 1, 1, 1, 1, 3], np.float32)
    eps = 1e-3
    exp = np.empty_like(x)
    for r in range(2):          # python-loop restatement of the definition
        ss = sum(float(v) * float(v) for v in x[r])
        inv = 1.0 / np.sqrt(ss / 8 + eps)
        exp[r] = [np.float16(np.float32(v * inv) * wv) for v, wv in zip(x[r], w)]
    got = oracle.f16_bits_to_f32(oracle.rms_norm_f16(oracle.f32_to_f16_bits(x), oracle.f32_to_f16_bits(w), eps))
    assert np.allclose(got, exp, rtol=2 ** -10)
    # f32 body vs independent f64 evaluation, any chunk width: at most 1 f16 ulp apart
    xb = oracle.f32_to_f16_bits(oracle.normal_f32((16, 1024), 3))
    wb = oracle.f32_to_f16_bits(oracle.uniform_f32(1024, 4, 0.5, 1.5))
    ref = oracle.rms_norm_f16_f64(xb, wb, 1e-6).astype(np.int32)
    for block in (0, 128, 512):
        got = oracle.rms_norm_f16(xb, wb, 1e-6, block).astype(np.int32)
        assert np.abs(got - ref).max() <= 1


# ---- K3 -------------------------------------------------------------------------------------
def test_softmax_vs_scipy_and_invariants():
    from scipy.special import softmax as sp_softmax

    x = oracle.normal_f32((16, 96), 5, 0, 3)
    got = oracle.softmax_f32(x, 2, 96)
    assert np.allclose(got, sp_softmax(x.astype(np.float64), axis=1), rtol=1e-5, atol=1e-8)
    assert np.allclose(got.sum(axis=1), 1, atol=1e-5)                       # softmax.rs:55-60
    assert np.allclose(oracle.softmax_f32(x + 7.0, 2, 96), got, rtol=1e-4)   # shift invariance
    assert np.array_equal(got.argmax(axis=1), x.argmax(axis=1))
    # reference example input: arange(32) as [4, 8], tiles [2, 8]
    a = np.arange(32, dtype=np.float32).reshape(4, 8)
    assert np.allclose(oracle.softmax_f32(a, 2, 8), sp_softmax(a.astype(np.float64), axis=1), rtol=1e-6)


def test_softmax_chunk_tiles_and_zero_padding_rule():
    from scipy.special import softmax as sp_softmax

    x = oracle.normal_f32((4, 64), 6)
    got = oracle.softmax_f32(x, 1, 16)           # BN < N: every 16-column tile is normalised on its own
    exp = np.concatenate([sp_softmax(x[:, i:i + 16].astype(np.float64), axis=1) for i in range(0, 64, 16)], axis=1)
    assert np.allclose(got, exp, rtol=1e-5)
    # ragged last tile: the 6 missing lanes are zero padded and DO take part in max and sum
    xr = oracle.normal_f32((3, 10), 7)
    got = oracle.softmax_f32(xr, 1, 16)
    padded = np.concatenate([xr, np.zeros((3, 6), np.float32)], axis=1).astype(np.float64)
    assert np.allclose(got, sp_softmax(padded, axis=1)[:, :10], rtol=1e-5)
    # f16 version = f32 statistics on decoded inputs, rounded once
    xb = oracle.f32_to_f16_bits(x)
    g16 = oracle.f16_bits_to_f32(oracle.softmax_f16(xb, 1, 64))
    e16 = sp_softmax(oracle.f16_bits_to_f32(xb).astype(np.float64), axis=1)
    assert np.allclose(g16, e16, rtol=2 ** -10, atol=1e-7)


# ---- K4 -------------------------------------------------------------------------------------
def test_cpu_gemm_patterned_inputs_and_known_answers():
    # cutile-examples/examples/persistent_gemm.rs:89-94: patterned, non-uniform inputs
    m, n, k = 64, 48, 32
    x = np.fromfunction(lambda r, c: ((r % 7) - 3.0) * 0.25 + (c % 5) * 0.125, (m, k)).astype(np.float32)
    y = np.fromfunction(lambda r, c: ((r % 3) + 1.0) * 0.2 - (c % 11) * 0.05, (k, n)).astype(np.float32)
    got = oracle.cpu_gemm_f32(x, y)
    assert np.abs(got - x.astype(np.float64) @ y.astype(np.float64)).max() < 1e-3        # persistent_gemm.rs:111-118
    # a transposed-operand slip would change this non-symmetric product
    assert np.abs(got - (y.T.astype(np.float64) @ x.T.astype(np.float64)).T).max() < 1e-3
    assert not np.allclose(got[:32, :32], (x[:32] @ y[:, :32]).T, atol=1e-3)
    # ones x ones = K (cutile/tests/slice_non_divisible.rs:459-500), identity
    assert np.array_equal(oracle.cpu_gemm_f32(np.ones((5, 37), np.float32), np.ones((37, 3), np.float32)), np.full((5, 3), 37, np.float32))
    assert np.array_equal(oracle.cpu_gemm_f32(np.eye(16, dtype=np.float32), y[:16]), y[:16])


def test_gemm_bf16_is_cpu_gemm_on_decoded_inputs_with_rne_store_and_row_subsets():
    m, n, k = 24, 40, 64
    a, b = oracle.f32_to_bf16_bits(oracle.normal_f32((m, k), 8)), oracle.f32_to_bf16_bits(oracle.normal_f32((k, n), 9))
    full = oracle.gemm_bf16(a, b, f32out=True)
    assert np.array_equal(full, oracle.cpu_gemm_f32(oracle.bf16_bits_to_f32(a), oracle.bf16_bits_to_f32(b)))
    assert np.array_equal(oracle.gemm_bf16(a, b), oracle.f32_to_bf16_bits(full))
    rows = np.array([3, 17, 23])
    assert np.array_equal(oracle.gemm_bf16(a, b, rows=rows, f32out=True), full[rows])


# ---- K5 -------------------------------------------------------------------------------------
def _attention_f64(q, k, v, scale, causal, input_pos, group):
    b, h, m, d = q.shape
    out = np.zeros((b, h, m, d))
    for bi in range(b):
        for hi in range(h):
            kv = hi // group
            s = (q[bi, hi].astype(np.float64) @ k[bi, kv].astype(np.float64).T) * scale
            if causal:
                i, j = np.indices(s.shape)
                s = np.where(j > i + input_pos, -np.inf, s)
            p = np.exp(s - s.max(axis=1, keepdims=True))
            out[bi, hi] = (p / p.sum(axis=1, keepdims=True)) @ v[bi, kv].astype(np.float64)
    return out


@pytest.mark.parametrize("causal,input_pos,group", [(False, 0, 1), (True, 0, 1), (True, 5, 1), (True, 3, 2)])
def test_fmha_ref_cpu_vs_float64_matrix_form(causal, input_pos, group):
    # shape of the reference example: flash_attention_causal.rs:216-222
    b, h, m, d = 2, 8, 64, 32
    q = oracle.normal_f32((b, h, m, d), 10)
    k = oracle.normal_f32((b, h // group, m, d), 11)
    v = oracle.normal_f32((b, h // group, m, d), 12)
    scale = 1 / np.sqrt(d)
    got = oracle.fmha_ref_cpu(q, k, v, scale, input_pos, group, causal)
    exp = _attention_f64(q, k, v, scale, causal, input_pos, group)
    assert np.abs(got - exp).max() <= 2e-5          # the reference itself accepts 2e-3 (rs:277-278)
    rows = np.array([0, 63, 64 * 9 + 5, b * h * m - 1])
    assert np.array_equal(oracle.fmha_ref_cpu(q, k, v, scale, input_pos, group, causal, rows=rows), got.reshape(-1, d)[rows])


def test_fmha_invariants():
    b, h, m, d = 1, 2, 32, 16
    q, k, v = (oracle.normal_f32((b, h, m, d), 20 + i) for i in range(3))
    out = oracle.fmha_ref_cpu(q, k, v, 0.25, 0, 1, True)
    # causal row 0 with input_pos = 0 sees only key 0
    assert np.allclose(out[:, :, 0], v[:, :, 0], atol=1e-6)
    # convex combination: every output column within [min V, max V]
    assert (out <= v.max(axis=2, keepdims=True) + 1e-5).all() and (out >= v.min(axis=2, keepdims=True) - 1e-5).all()
    # Q == 0 -> uniform weights over the visible keys
    o0 = oracle.fmha_ref_cpu(np.zeros_like(q), k, v, 0.25, 0, 1, True)
    exp = np.cumsum(v, axis=2) / np.arange(1, m + 1)[None, None, :, None]
    assert np.allclose(o0, exp, atol=1e-5)


# ---- K6 -------------------------------------------------------------------------------------
def test_mx_all_ones_known_answer_and_formula():
    # cutile-examples/examples/mxfp8.rs:84-135: 0x38 data, 0x7F scales -> every output = K
    m = n = 16
    k = 128
    x = np.full((m, k), 0x38, np.uint8)
    s = np.full((m, k // 32), 0x7F, np.uint8)
    assert np.array_equal(oracle.mx_gemm_f32(x, x, s, s), np.full((m, n), float(k), np.float32))
    # z = alpha * (x*sx) @ (y*sy)^T with y stored [N, K]
    xf, yf = oracle.normal_f32((8, 64), 30), oracle.normal_f32((12, 64), 31) * 37.0
    xq, xs = oracle.mx_quantize_e4m3(xf)
    yq, ys = oracle.mx_quantize_e4m3(yf)
    got = oracle.mx_gemm_f32(xq, yq, xs, ys, 0.5)
    exp = 0.5 * oracle.mx_dequantize_e4m3(xq, xs).astype(np.float64) @ oracle.mx_dequantize_e4m3(yq, ys).astype(np.float64).T
    assert np.allclose(got, exp, rtol=1e-5, atol=1e-5)
    assert got.shape == (8, 12)


def test_mx_quantiser_follows_ocp_rule():
    x = oracle.normal_f32((64, 256), 32) * np.exp2(oracle.uniform_f32((64, 8), 33, -20, 20)).repeat(32, axis=1)
    q, s = oracle.mx_quantize_e4m3(x)
    amax = np.abs(x.reshape(64, 8, 32)).max(axis=2)
    assert np.array_equal(s.astype(np.int32) - 127, np.floor(np.log2(amax)).astype(np.int32) - 8)
    deq = oracle.mx_dequantize_e4m3(q, s)
    # 3 mantissa bits: relative error <= 2^-4 for normal values, except the saturated top (amax/scale in (448, 512))
    scale = np.exp2(s.astype(np.float32) - 127).repeat(32, axis=1)
    normal = np.abs(x) >= scale * 2 ** -6
    unsat = np.abs(x) <= 448 * scale
    sel = normal & unsat
    assert (np.abs(deq - x)[sel] <= np.abs(x)[sel] * 2 ** -4 + 1e-30).all()
    assert (np.abs(deq)[~unsat] == (448 * scale)[~unsat]).all()
    z, zs = oracle.mx_quantize_e4m3(np.zeros((1, 32), np.float32))
    assert not z.any() and zs[0, 0] == 127


def test_rms_norm_f32_example_rounds_its_square_root_down():
    """cutile-examples/examples/rms_norm.rs:17-61: scale = sqrt_rd(1 / (mean(x^2) + eps)); float64 fixes the scale as the
    largest f32 that does not exceed the exact square root of the f32 argument"""
    x, w = oracle.normal_f32((64, 512), 991), oracle.uniform_f32(512, 992, 0.5, 1.5)
    out = oracle.rms_norm_f32_example(x, w, 1e-6, 128)
    for r in range(64):
        acc = np.zeros(128, np.float32)
        for j in range(0, 512, 128):
            acc = acc + x[r, j:j + 128] * x[r, j:j + 128]
        width = 128                                        # the tile reduction: pairwise halves
        while width > 1:
            half = (width + 1) // 2
            acc[:width // 2] = acc[:width // 2] + acc[half:half + width // 2]
            width = half
        s = acc[0]
        arg = np.float32(np.float32(1.0) / np.float32(np.float32(s / np.float32(512)) + np.float32(1e-6)))
        exact = np.sqrt(np.float64(arg))
        scale = np.float32(exact)
        if np.float64(scale) > exact:
            scale = np.nextafter(scale, np.float32(0))
        assert np.float64(scale) <= exact < np.float64(np.nextafter(scale, np.float32(np.inf)))
        assert np.array_equal(out[r], x[r] * scale * w)
    # a constant row: mean(x^2) = c^2, so out = sign(c) w up to the eps and the downward rounding
    c = np.full((2, 256), -3.0, np.float32)
    got = oracle.rms_norm_f32_example(c, w[:256], 0.0)
    assert np.allclose(got, -w[:256], rtol=3e-7, atol=0) and np.all(np.abs(got) <= w[:256])
    # against float64 as a whole
    ref = x.astype(np.float64) / np.sqrt((x.astype(np.float64) ** 2).mean(axis=1, keepdims=True) + 1e-6) * w
    assert np.max(np.abs(out - ref) / np.abs(ref).max()) < 1e-6


# ---- the benchmark programs' all-f16 arithmetic ---------------------------------------------------------------
def _rn_f16(q: Fraction) -> Fraction:
    """round-to-nearest-even of a non-negative rational to the f16 grid (normal and subnormal range, no overflow)"""
    if q == 0:
        return Fraction(0)
    e = max(math.floor(math.log2(q)), -14)
    while Fraction(2) ** e > q and e > -14:
        e -= 1
    while Fraction(2) ** (e + 1) <= q:
        e += 1
    ulp = Fraction(2) ** (e - 10)
    k = q / ulp
    lo = math.floor(k)
    k = lo + 1 if (k - lo > Fraction(1, 2) or (k - lo == Fraction(1, 2) and lo % 2 == 1)) else lo
    return k * ulp


def test_f16_square_root_rounded_down_over_every_positive_f16():
    v = np.arange(0, 0x7C01, dtype=np.uint16).view(np.float16)          # +0 .. +inf
    r = oracle.sqrt_f16_toward_minus_infinity(v)
    fin = np.isfinite(v)
    r64, v64 = r.astype(np.float64)[fin], v.astype(np.float64)[fin]     # squares of f16 values are exact in f64
    up = np.nextafter(r, np.float16(np.inf)).astype(np.float64)[fin]
    assert (r64 ** 2 <= v64).all() and (up ** 2 > v64).all()
    assert np.isinf(r[-1]) and np.isnan(oracle.sqrt_f16_toward_minus_infinity(np.float16(-1.0)))


def test_all_f16_rms_norm_against_exact_rational_arithmetic_rounded_step_by_step():
    # A row of constants makes every step of cutile-benchmarks/benches/rmsnorm.rs:37-62 checkable with exact rationals:
    # lane sums, the tree, sum / N, + eps, 1 / x, the downward square root, x * rms * w.
    n, block = 2048, 512
    for xv, wv, eps in [(1.0, 1.0, 1e-5), (3.0, 0.5, 1e-5), (0.3330078125, 1.5, 1e-3), (5.25, 0.0999755859375, 1e-5)]:
        x = np.full((2, n), xv, np.float16)
        w = np.full(n, wv, np.float16)
        got = oracle.rms_norm_all_f16(x.view(np.uint16), w.view(np.uint16), eps, block).view(np.float16)
        fx, fw = Fraction(float(x[0, 0])), Fraction(float(w[0]))
        lane = Fraction(0)
        for _ in range(n // block):
            lane = _rn_f16(lane + _rn_f16(fx * fx))
        total, lanes = lane, block
        while lanes > 1:                       # equal lanes: every tree level doubles, rounded
            total, lanes = _rn_f16(total + total), lanes // 2
        mean = _rn_f16(total / _rn_f16(Fraction(n)))
        inv = _rn_f16(1 / _rn_f16(mean + Fraction(float(np.float16(eps)))))
        grid = [Fraction(float(h)) for h in np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16)]
        scale = max(h for h in grid if h * h <= inv)
        want = _rn_f16(_rn_f16(fx * scale) * fw)
        assert Fraction(float(got[0, 0])) == want and (got == got[0, 0]).all(), (xv, wv, float(got[0, 0]), float(want))
    # the f16 sum of squares overflows early (17.5^2 * 2048 > 65504): inf -> 1 / inf = 0 -> every output is 0
    x = np.full((1, n), 17.5, np.float16)
    assert (oracle.rms_norm_all_f16(x.view(np.uint16), np.ones(n, np.float16).view(np.uint16), 1e-5, block) == 0).all()


def test_all_f16_reduce_sum_is_the_stride_halving_tree():
    # brute force with scalar f16 additions in the stated order, on lanes chosen so that the order matters
    rng = np.random.default_rng(11)
    lanes = (rng.standard_normal(64) * np.exp2(rng.integers(-6, 7, 64))).astype(np.float16)
    a = [np.float16(v) for v in np.abs(lanes)]
    step = 32
    while step >= 1:
        for l in range(step):
            a[l] = np.float16(np.float32(a[l]) + np.float32(a[l + step]))
        step //= 2
    assert oracle._tree_sum_f16(np.abs(lanes)[None, :])[0] == a[0]
    # through rms_norm_all_f16: one tile, x = sqrt of the lanes would not be exact, so check the softmax denominator
    # instead: exp(0) = 1 everywhere -> the tree of ones is exact: every output is 1 / BN
    y = oracle.softmax_all_f16(np.zeros((3, 256), np.float16).view(np.uint16), 1, 256).view(np.float16)
    assert (y == np.float16(1 / 256)).all()


def test_all_f16_forms_stay_near_the_float64_functions():
    x = oracle.f32_to_f16_bits(oracle.normal_f32((16, 4096), 3))
    w = oracle.f32_to_f16_bits(oracle.normal_f32((4096,), 4))
    xf, wf = x.view(np.float16).astype(np.float64), w.view(np.float16).astype(np.float64)
    o = oracle.rms_norm_all_f16(x, w, 1e-5, 512).view(np.float16).astype(np.float64)
    ref = xf / np.sqrt((xf ** 2).mean(1, keepdims=True) + 1e-5) * wf
    assert np.abs(o - ref).max() <= 4e-3 * np.abs(ref).max()              # f16 accumulation of 4096 squares: ~2^-9 relative
    for bm, bn in [(1, 4096), (4, 1024), (2, 64)]:
        y = oracle.softmax_all_f16(x, bm, bn).view(np.float16).astype(np.float64)
        seg = xf.reshape(16, 4096 // bn, bn)
        e = np.exp(seg - seg.max(2, keepdims=True))
        sref = (e / e.sum(2, keepdims=True)).reshape(16, 4096)
        assert np.abs(y - sref).max() <= 3e-3 * sref.max()
    # ragged width: the last tile's missing columns read 0 and take part (exp(0 - max) joins the denominator)
    xr = x[:, :100]
    y = oracle.softmax_all_f16(xr, 1, 64).view(np.float16).astype(np.float64)
    seg = np.concatenate([xf[:, 64:100], np.zeros((16, 28))], axis=1)
    e = np.exp(seg - seg.max(1, keepdims=True))
    assert np.abs(y[:, 64:] - (e / e.sum(1, keepdims=True))[:, :36]).max() <= 2e-3


# ---- the example programs' small kernels: pinned by hand-worked cases, the reference programs' own checks and f64 sums ----
def test_relu_and_dropout_hand_worked_cases():
    assert oracle.relu_f32([-1.5, -0.0, 0.0, 2.25]).tolist() == [0.0, 0.0, 0.0, 2.25]
    # p = 0.5: values at or below p go, the rest double (exact in binary)
    assert oracle.dropout_f32(0.5, [0.25, 0.5, 0.75, 1.0]).tolist() == [0.0, 0.0, 1.5, 2.0]
    # a shorter keep tensor reads 0 beyond its end; a longer one is cut
    assert oracle.dropout_f32(0.5, [0.75], 3).tolist() == [1.5, 0.0, 0.0]
    assert oracle.dropout_f32(0.5, [0.75, 1.0, 0.625], 2).tolist() == [1.5, 2.0]
    # p = 0.4 as in cutile-examples/examples/dropout.rs:45: the quotient is the f32 division by the f32 value of 1 - p
    got = oracle.dropout_f32(0.4, [0.9])[0]
    assert got == np.float32(0.9) / (np.float32(1) - np.float32(0.4)) and abs(float(got) - 1.5) < 1e-6
    # the keep fraction of uniform samples is 1 - p
    keep = oracle.uniform_f32(100000, 5, 0.0, 1.0)
    assert abs(np.count_nonzero(oracle.dropout_f32(0.4, keep)) / keep.size - 0.6) < 0.01


def test_scale_is_the_reference_programs_own_check():
    # cutile-examples/examples/scale_ptr.rs:102-110: output[i] == input[i] * scale for arange(1024), scale 3
    x = np.arange(1024, dtype=np.float32)
    assert np.array_equal(oracle.scale_f32(x, 3.0), np.arange(1024) * 3)


def test_matvec_and_batch_matmul_against_f64_sums_and_closed_forms():
    x, y, z = oracle.normal_f32((37, 300), 1), oracle.normal_f32(300, 2), oracle.normal_f32(37, 3)
    want = z.astype(np.float64) + x.astype(np.float64) @ y.astype(np.float64)
    assert np.allclose(oracle.matvec_f32(z, x, y), want, rtol=0, atol=1e-4)
    # k / BK whole K tiles: the last 300 - 256 products are left out; a transposed operand or a dropped z would show
    cut = z.astype(np.float64) + x[:, :256].astype(np.float64) @ y[:256].astype(np.float64)
    assert np.allclose(oracle.matvec_f32(z, x, y, 300, 128), cut, rtol=0, atol=1e-4)
    assert not np.allclose(cut, want, atol=1e-2)
    # cutile-examples/examples/batch_matmul.rs:49-76: ones x ones = K everywhere
    assert np.array_equal(oracle.batch_matmul_f32(np.ones((4, 128, 64), np.float32), np.ones((4, 64, 256), np.float32)), np.full((4, 128, 256), 64, np.float32))
    a, b = oracle.normal_f32((3, 20, 40), 4), oracle.normal_f32((3, 40, 30), 5)
    assert np.allclose(oracle.batch_matmul_f32(a, b), np.einsum("bmk,bkn->bmn", a.astype(np.float64), b.astype(np.float64)), rtol=0, atol=1e-4)
    # batches stay apart: permuting the batches of both operands permutes the result
    perm = [2, 0, 1]
    assert np.array_equal(oracle.batch_matmul_f32(a[perm], b[perm]), oracle.batch_matmul_f32(a, b)[perm])
