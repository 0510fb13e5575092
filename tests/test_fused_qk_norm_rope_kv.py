"""Fused Q/K norm + rotary embedding + KV-cache update: qk_norm_rope_kv_prefill_raw_f16 and qk_norm_rope_kv_decode_raw_f16
(cutile-kernels/src/experimental/fused_transformer.rs:22-345, 356-625).

CPU: the oracle pinned by rms_norm at position 0 (no rotation), by the chain of the separate kernels' oracles (equal up
to the f16 rounding between them), a float64 evaluation, the norm-preserving rotation and exact copies of v.
GPU: within 1 f16 ulp of the oracle (rsqrt, cos / sin and the fused multiply-adds differ in the last f32 bit; where
the rotated terms cancel, within 4e-6 absolute), v rows and untouched cache rows bit-exact."""
import numpy as np
import pytest
import torch

import oracle
from util import f16_ulp_diff

f16b = lambda a: oracle.f32_to_f16_bits(np.asarray(a, np.float32))
f16v = lambda bits: oracle.f16_bits_to_f32(bits)


def _case(seq, nq, nkv, d, max_seq, seed):
    q, k, v = (f16b(oracle.normal_f32((seq, h, d), seed + i)) for i, h in enumerate((nq, nkv, nkv)))
    qw, kw = f16b(oracle.uniform_f32(d, seed + 3, 0.5, 1.5)), f16b(oracle.uniform_f32(d, seed + 4, 0.5, 1.5))
    inv_freq = (1.0 / 10000.0 ** (np.arange(d // 2) / (d // 2))).astype(np.float32)
    kc, vc = f16b(oracle.normal_f32((nkv, max_seq, d), seed + 5)), f16b(oracle.normal_f32((nkv, max_seq, d), seed + 6))
    return q, k, v, qw, kw, inv_freq, kc, vc


# ---- oracle (CPU) ---------------------------------------------------------------------------
def test_oracle_fused_reduces_to_rms_norm_and_matches_float64():
    q, k, v, qw, kw, inv_freq, kc, vc = _case(5, 4, 2, 64, 16, 901)
    # position 0 only: theta = 0, so every row is its RMS norm
    qo, kc1, vc1 = oracle.qk_norm_rope_kv_f16(q[:1], k[:1], v[:1], qw, kw, inv_freq, kc, vc, 1e-6, 0)
    assert np.array_equal(qo[0], oracle.rms_norm_f16(q[0], qw, 1e-6))
    assert np.array_equal(kc1[:, 0], oracle.rms_norm_f16(k[0], kw, 1e-6))
    assert np.array_equal(vc1[:, 0], v[0]) and np.array_equal(kc1[:, 1:], kc[:, 1:]) and np.array_equal(vc1[:, 1:], vc[:, 1:])
    # float64 evaluation at positions 7 .. 11
    qo, kc1, vc1 = oracle.qk_norm_rope_kv_f16(q, k, v, qw, kw, inv_freq, kc, vc, 1e-6, 7)
    half = 32
    for x, w, got in ((f16v(q), f16v(qw), f16v(qo)), (f16v(k), f16v(kw), f16v(kc1[:, 7:12]).transpose(1, 0, 2))):
        x64 = x.astype(np.float64)
        n = x64 / np.sqrt((x64 ** 2).mean(axis=-1, keepdims=True) + 1e-6) * w
        th = (7 + np.arange(5))[:, None, None] * inv_freq.astype(np.float64)[None, None, :]
        lo, hi = n[..., :half], n[..., half:]
        want = np.concatenate([lo * np.cos(th) - hi * np.sin(th), hi * np.cos(th) + lo * np.sin(th)], axis=-1)
        assert np.max(np.abs(got - want)) < 4e-3                                   # f16 output near magnitude 4
        # the rotation keeps every pair's length: |y|^2 = |n|^2 per row
        assert np.allclose((got.astype(np.float64) ** 2).sum(-1), (n ** 2).sum(-1), rtol=2e-3)
    assert np.array_equal(vc1[:, 7:12], v.transpose(1, 0, 2)) and np.array_equal(vc1[:, :7], vc[:, :7]) and np.array_equal(kc1[:, 12:], kc[:, 12:])


def test_oracle_fused_equals_the_chain_of_separate_kernels_up_to_one_rounding():
    q, k, v, qw, kw, inv_freq, kc, vc = _case(9, 6, 2, 128, 32, 911)
    qo, kc1, vc1 = oracle.qk_norm_rope_kv_f16(q, k, v, qw, kw, inv_freq, kc, vc, 1e-5, 3)
    normed = oracle.qk_norm_f16(q.reshape(-1, 128), k.reshape(-1, 128), qw, kw, 1e-5)        # rounded to f16 here ...
    qn, kn = normed[:9 * 6].reshape(9, 6, 128), normed[9 * 6:].reshape(9, 2, 128)
    q_chain, k_chain = oracle.rope_seq_f16(qn, inv_freq, 3), oracle.rope_seq_f16(kn, inv_freq, 3)   # ... and rotated from there
    # the chain rounds the normalised values (magnitude up to ~4: half an ulp is 2e-3) before rotating them
    assert np.max(np.abs(f16v(qo) - f16v(q_chain))) <= 6e-3
    assert np.max(np.abs(f16v(kc1[:, 3:12].transpose(1, 0, 2)) - f16v(k_chain))) <= 6e-3
    assert np.mean(f16_ulp_diff(qo, q_chain) <= 1) > 0.95
    kc2, vc2 = oracle.kv_cache_update_f16(k_chain, v, kc, vc, 3, 9)
    assert np.array_equal(vc1, vc2)


# ---- launcher on the recording runtime (CPU) ----------------------------------------------------
def test_fused_launcher_validation(fake_hip):
    ct = fake_hip
    from test_host_abi import _last
    h = torch.half
    q, k = torch.zeros(10, 4, 128, dtype=h), torch.zeros(10, 2, 128, dtype=h)
    w, inv = torch.zeros(128, dtype=h), torch.zeros(64)
    kc = torch.zeros(2, 32, 128, dtype=h)
    ct.qk_norm_rope_kv_prefill_raw_f16(q, k, k, w, w, inv, q, kc, kc.clone(), 1e-6, 5, 10, generics=[128, 64, 32])
    rec, _ = _last(ct)
    assert rec.symbol == b"qk_norm_rope_kv_entry__f16" and tuple(rec.grid) == (10, 1, 1)
    pos = torch.zeros(1, dtype=torch.int32)
    ct.qk_norm_rope_kv_decode_raw_f16(torch.zeros(8 * 128, dtype=h), w, w, inv, torch.zeros(4, 128, dtype=h), kc, kc.clone(), pos, 1e-6, 4, 2)
    assert tuple(_last(ct)[0].grid) == (1, 1, 1)
    n0 = ct.lib().cutile_testing_launch_count()
    cases = [
        (lambda: ct.qk_norm_rope_kv_prefill_raw_f16(q, k, k, w, w, inv, q, kc, kc.clone(), 1e-6, 25, 10), "do not fit the 32 rows"),
        (lambda: ct.qk_norm_rope_kv_prefill_raw_f16(q, k, k, w, w, inv, q, kc, kc.clone(), 1e-6, 5, 10, generics=[64, 32, 32]), "D"),
        (lambda: ct.qk_norm_rope_kv_prefill_raw_f16(q[:, :, 1:], k, k, w, w, inv, q, kc, kc.clone(), 1e-6, 5, 10), "contiguous"),
        (lambda: ct.qk_norm_rope_kv_prefill_raw_f16(torch.zeros(10, 4, 24, dtype=h), torch.zeros(10, 2, 24, dtype=h), torch.zeros(10, 2, 24, dtype=h),
                                                    w, w, inv, torch.zeros(10, 4, 24, dtype=h), torch.zeros(2, 32, 24, dtype=h),
                                                    torch.zeros(2, 32, 24, dtype=h), 1e-6, 0, 10), "multiple of 16"),
    ]
    for fn, msg in cases:
        with pytest.raises(ct.CutileError, match=msg):
            fn()
    assert ct.lib().cutile_testing_launch_count() == n0


# ---- HIP kernel (GPU) ---------------------------------------------------------------------------
def _dev16(bits, dev):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(dev).view(torch.half)


def _bits(t):
    return t.cpu().numpy().view(np.uint16)


def _close(got_bits, ref_bits):
    """within 1 f16 ulp, or within 4e-6 where the two rotated terms cancel (there the f32 rounding of rsqrt, cos and
    sin, 1e-7 relative on terms of magnitude ~1, is many ulps of a result near zero)"""
    return bool(np.all((f16_ulp_diff(got_bits, ref_bits) <= 1) | (np.abs(f16v(got_bits) - f16v(ref_bits)) <= 4e-6)))


@pytest.mark.gpu
@pytest.mark.parametrize("seq,nq,nkv,d,max_seq,start", [(37, 6, 2, 128, 64, 5), (64, 32, 8, 128, 128, 64), (19, 4, 4, 64, 32, 0), (8, 3, 1, 256, 16, 8),
                                                        (300, 5, 2, 32, 512, 100)])
def test_gpu_fused_prefill(ct, dev, seq, nq, nkv, d, max_seq, start):
    q, k, v, qw, kw, inv_freq, kc, vc = _case(seq, nq, nkv, d, max_seq, 921)
    q_out = torch.zeros(seq, nq, d, dtype=torch.half, device=dev)
    kcd, vcd = _dev16(kc, dev), _dev16(vc, dev)
    ct.qk_norm_rope_kv_prefill_raw_f16(_dev16(q, dev), _dev16(k, dev), _dev16(v, dev), _dev16(qw, dev), _dev16(kw, dev),
                                       torch.from_numpy(inv_freq).to(dev), q_out, kcd, vcd, 1e-6, start, seq, generics=[d, d // 2, max_seq])
    torch.cuda.synchronize()
    rq, rk, rv = oracle.qk_norm_rope_kv_f16(q, k, v, qw, kw, inv_freq, kc, vc, 1e-6, start)
    assert _close(_bits(q_out), rq)
    assert _close(_bits(kcd)[:, start:start + seq], rk[:, start:start + seq])
    assert np.array_equal(_bits(vcd), rv)                                                      # copies are exact
    assert np.array_equal(_bits(kcd)[:, :start], kc[:, :start]) and np.array_equal(_bits(kcd)[:, start + seq:], kc[:, start + seq:])


@pytest.mark.gpu
@pytest.mark.parametrize("pos", [0, 77])
def test_gpu_fused_decode_in_place(ct, dev, pos):
    nq, nkv, d, max_seq = 8, 2, 128, 128
    q, k, v, qw, kw, inv_freq, kc, vc = _case(1, nq, nkv, d, max_seq, 931)
    qkv = _dev16(np.concatenate([q.reshape(-1), k.reshape(-1), v.reshape(-1)]), dev)
    q_out = torch.zeros(nq, d, dtype=torch.half, device=dev)
    kcd, vcd = _dev16(kc, dev), _dev16(vc, dev)
    pos_dev = torch.tensor([pos], dtype=torch.int32, device=dev)
    ct.qk_norm_rope_kv_decode_raw_f16(qkv, _dev16(qw, dev), _dev16(kw, dev), torch.from_numpy(inv_freq).to(dev), q_out, kcd, vcd, pos_dev,
                                      1e-6, nq, nkv)
    torch.cuda.synchronize()
    rq, rk, rv = oracle.qk_norm_rope_kv_f16(q, k, v, qw, kw, inv_freq, kc, vc, 1e-6, pos)
    assert _close(_bits(q_out), rq[0]) and _close(_bits(kcd), rk) and np.array_equal(_bits(vcd), rv)
    # q_out may be the q rows themselves (the reference's decode graph rotates in place)
    ct.qk_norm_rope_kv_decode_raw_f16(qkv, _dev16(qw, dev), _dev16(kw, dev), torch.from_numpy(inv_freq).to(dev), qkv, kcd, vcd, pos_dev,
                                      1e-6, nq, nkv)
    torch.cuda.synchronize()
    assert _close(_bits(qkv)[:nq * d].reshape(nq, d), rq[0])
