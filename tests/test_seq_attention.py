"""Sequence-layout attention of cutile-kernels/src/attention.rs: flash_attn_causal_seq_f16 (:21-116),
flash_attn_causal_seq_dynpos_f16 (:128-231), fmha_prefill_causal (:242-391), fmha_prefill_gqa (:408-587) and
fmha_causal (:598-726).  q and out are [q_len, q_heads, D], k and v [kv_heads, max_seq, D], all f16.

CPU: the oracle (fmha_ref_cpu on the permuted layout) pinned by a float64 evaluation with an explicit mask and by
closed forms; the launcher on the recording runtime.  GPU: every reference form against the oracle, max-abs <= 2e-2
(observed ~1e-3: f16 inputs, f16 probabilities in the second product, f16 output)."""
import struct

import numpy as np
import pytest
import torch

import oracle

f16r = lambda a: np.asarray(a, np.float32).astype(np.float16).astype(np.float32)


def _inputs(q_len, q_heads, kv_heads, max_seq, d, seed):
    q = f16r(oracle.normal_f32((q_len, q_heads, d), seed))
    k = f16r(oracle.normal_f32((kv_heads, max_seq, d), seed + 1))
    v = f16r(oracle.normal_f32((kv_heads, max_seq, d), seed + 2))
    return q, k, v


def _float64(q, k, v, scale, group, kv_len, query_start, causal):
    q_len, q_heads, d = q.shape
    out = np.zeros((q_len, q_heads, d))
    for h in range(q_heads):
        kk, vv = k[h // group, :kv_len].astype(np.float64), v[h // group, :kv_len].astype(np.float64)
        s = q[:, h].astype(np.float64) @ kk.T * scale
        if causal:
            s = np.where(np.arange(kv_len)[None, :] <= query_start + np.arange(q_len)[:, None], s, -np.inf)
        p = np.exp(s - s.max(axis=1, keepdims=True))
        out[:, h] = (p / p.sum(axis=1, keepdims=True)) @ vv
    return out


# ---- oracle (CPU) ---------------------------------------------------------------------------
def test_oracle_seq_attention_is_masked_softmax_attention():
    q, k, v = _inputs(37, 8, 2, 96, 32, 701)
    for kv_len, start, causal in ((96, 0, True), (70, 33, True), (50, 0, False), (20, 40, True), (96, 59, True)):
        ref = oracle.attention_seq_ref(q, k, v, 0.17, 4, kv_len, start, causal)
        assert ref.shape == q.shape
        assert np.max(np.abs(ref - _float64(q, k, v, 0.17, 4, kv_len, start, causal))) < 2e-5


def test_oracle_seq_attention_reduces_to_the_example_reference():
    """with as many keys as queries the rule is fmha_ref_cpu's (cutile-examples/examples/flash_attention_causal.rs:140-210,
    input_pos = query_start) on the permuted layout"""
    q, k, v = _inputs(48, 6, 3, 48, 32, 705)
    for start, causal in ((0, True), (7, True), (0, False)):
        ref = oracle.attention_seq_ref(q, k, v, 0.21, 2, 48, start, causal)
        ex = oracle.fmha_ref_cpu(np.ascontiguousarray(q.transpose(1, 0, 2))[None], k[None], v[None], 0.21, start, 2, causal)
        assert np.max(np.abs(ref - ex[0].transpose(1, 0, 2))) < 1e-6


def test_oracle_seq_attention_closed_forms():
    q, k, v = _inputs(16, 4, 2, 40, 32, 711)
    ref = oracle.attention_seq_ref(q, k, v, 0.2, 2, 40, 0, True)
    assert np.allclose(ref[0], v[[0, 0, 1, 1], 0], atol=1e-6)                  # query 0 sees key 0 only, of its kv head
    z = oracle.attention_seq_ref(np.zeros_like(q), k, v, 0.2, 2, 25, 3, True)       # zero queries: mean of the visible rows
    for i in (0, 5, 15):
        n = min(25, 3 + i + 1)
        assert np.allclose(z[i, 3], v[1, :n].mean(axis=0), atol=1e-5)
    z = oracle.attention_seq_ref(np.zeros_like(q), k, v, 0.2, 2, 25, 0, False)
    assert np.allclose(z[7, 0], v[0, :25].mean(axis=0), atol=1e-5)
    assert not oracle.attention_seq_ref(q, k, v, 0.2, 2, 0, 0, True).any()         # no key at all: zeros


# ---- launcher on the recording runtime (CPU) ----------------------------------------------------
def _last(ct):
    import ctypes as C

    from test_host_abi import _last as last
    return last(ct)


def test_seq_attention_launcher_translates_the_layout(fake_hip):
    ct = fake_hip
    h = torch.half
    q = torch.zeros(300, 8, 128, dtype=h)
    kc = torch.zeros(2, 512, 128, dtype=h)
    out = torch.zeros(300, 8, 128, dtype=h)
    # prefill: 300 rows >= 256 -> the ping-pong kernel, one workgroup per (head, 256 rows)
    ct.fmha_seq_f16(q, kc, kc, ct.partition(out, [64, 1, 128]), 0.088, 4, kv_len=300, query_start=0, generics=[64, 64, 128])
    rec, args = _last(ct)
    assert rec.symbol == b"fmha_entry__f16_256x64x128_pp" and tuple(rec.grid) == (8, 2, 1) and tuple(rec.block) == (512, 1, 1)
    # out partition record: ptr, shape (heads, rows, d), strides (d, heads*d, 1), tile (1, 256, 128)
    ptr, = struct.unpack_from("<Q", args, 0)
    assert ptr == out.data_ptr()
    assert struct.unpack_from("<6i", args, 8) == (8, 300, 128, 128, 1024, 1)
    assert struct.unpack_from("<3i", args, 32) == (1, 256, 128)
    # q view (1, heads, rows, d) strides (0, d, heads*d, 1); k view (1, kv_heads, kv_len, d)
    assert struct.unpack_from("<8i", args, 56 + 8) == (1, 8, 300, 128, 0, 128, 1024, 1)
    assert struct.unpack_from("<8i", args, 56 + 40 + 8) == (1, 2, 300, 128, 0, 512 * 128, 128, 1)
    scale, start, group, causal = struct.unpack_from("<fiii", args, 56 + 3 * 40)
    assert abs(scale - 0.088) < 1e-7 and (start, group, causal) == (0, 4, 1)
    # decode-style call with the position on the device: BM = 1, one row -> the plain kernel of that D
    pos = torch.zeros(1, dtype=torch.int32)
    q1, o1 = torch.zeros(1, 8, 128, dtype=h), torch.zeros(1, 8, 128, dtype=h)
    ct.fmha_seq_f16(q1, kc, kc, ct.partition(o1, [1, 1, 128]), 0.088, 4, position_start=pos, kv_len_from_position=True)
    rec, args = _last(ct)
    assert rec.symbol == b"fmha_seq_entry__f16_128x64x128" and tuple(rec.grid) == (8, 1, 1) and tuple(rec.block) == (256, 1, 1)
    p, from_pos, group, causal = struct.unpack_from("<Qiii", args, 56 + 3 * 40 + 8)
    assert p == pos.data_ptr() and (from_pos, group, causal) == (1, 4, 1)
    assert struct.unpack_from("<8i", args, 56 + 40 + 8)[:4] == (1, 2, 512, 128)      # every cached row is reachable
    # the packed-heads form: tiles [BM, GROUP, D] cover the same outputs
    ct.fmha_seq_f16(q, kc, kc, ct.partition(out, [32, 4, 128]), 0.088, 4, kv_len=512, query_start=212, causal=False)
    assert tuple(_last(ct)[0].grid) == (8, 2, 1)
    n0 = ct.lib().cutile_testing_launch_count()
    cases = [
        (lambda: ct.fmha_seq_f16(q, kc, kc, ct.partition(out, [64, 1, 128]), 0.088, 2, kv_len=300), "do not agree"),
        (lambda: ct.fmha_seq_f16(q, kc, kc, ct.partition(out, [64, 3, 128]), 0.088, 4, kv_len=300), "G dividing query_group_size"),
        (lambda: ct.fmha_seq_f16(q, kc, kc, ct.partition(out, [64, 1, 128]), 0.088, 4, kv_len=513), "kv_len within the 512 rows"),
        (lambda: ct.fmha_seq_f16(q, kc, kc, ct.partition(out, [64, 1, 128]), 0.088, 4, kv_len=300, query_start=-1), "non-negative"),
        (lambda: ct.fmha_seq_f16(q, kc, kc, ct.partition(out, [64, 1, 128]), 0.088, 4, kv_len=300, generics=[32, 64, 128]), "BM"),
        (lambda: ct.fmha_seq_f16(q.float(), kc, kc, ct.partition(out, [64, 1, 128]), 0.088, 4, kv_len=300), "must be f16"),
        (lambda: ct.fmha_seq_f16(torch.zeros(300, 8, 96, dtype=h), torch.zeros(2, 512, 96, dtype=h), torch.zeros(2, 512, 96, dtype=h),
                                 ct.partition(torch.zeros(300, 8, 96, dtype=h), [64, 1, 96]), 0.088, 4, kv_len=300), "no precompiled sequence attention"),
    ]
    for fn, msg in cases:
        with pytest.raises(ct.CutileError, match=msg):
            fn()
    assert ct.lib().cutile_testing_launch_count() == n0


# ---- HIP kernels (GPU) --------------------------------------------------------------------------
def _dev(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev).half()


def _check(out, ref):
    got = out.float().cpu().numpy()
    assert np.all(np.isfinite(got))
    assert float(np.max(np.abs(got - ref))) <= 2e-2


@pytest.mark.gpu
@pytest.mark.parametrize("q_len,q_heads,kv_heads,max_seq,d,bm,kv_len,start", [
    (200, 8, 2, 512, 128, 64, 300, 100),          # ragged rows, queries behind a cached prefix
    (64, 4, 4, 64, 64, 32, 64, 0),                # D 64, no grouping
    (70, 6, 2, 100, 32, 16, 100, 30),             # D 32
    (300, 8, 8, 300, 128, 64, 300, 0),            # long enough for the ping-pong kernel, ragged
    (150, 4, 2, 256, 256, 32, 200, 50),           # D 256
])
def test_gpu_flash_attn_causal_seq(ct, dev, q_len, q_heads, kv_heads, max_seq, d, bm, kv_len, start):
    q, k, v = _inputs(q_len, q_heads, kv_heads, max_seq, d, 721)
    out = torch.full((q_len, q_heads, d), float("nan"), dtype=torch.half, device=dev)
    group = q_heads // kv_heads
    ct.fmha_seq_f16(_dev(q, dev), _dev(k, dev), _dev(v, dev), ct.partition(out, [bm, 1, d]), d ** -0.5, group,
                    kv_len=kv_len, query_start=start, generics=[bm, 32, d])
    torch.cuda.synchronize()
    _check(out, oracle.attention_seq_ref(q, k, v, d ** -0.5, group, kv_len, start, True))


@pytest.mark.gpu
@pytest.mark.parametrize("pos", [0, 137, 511])
def test_gpu_flash_attn_causal_seq_dynpos_and_fmha_causal(ct, dev, pos):
    """the decode forms: q_len = 1, BM = 1, the position in device memory"""
    q, k, v = _inputs(1, 8, 2, 512, 128, 731)
    pos_dev = torch.tensor([pos], dtype=torch.int32, device=dev)
    qd, kd, vd = _dev(q, dev), _dev(k, dev), _dev(v, dev)
    out = torch.full((1, 8, 128), float("nan"), dtype=torch.half, device=dev)
    ct.fmha_seq_f16(qd, kd, vd, ct.partition(out, [1, 1, 128]), 0.09, 4, position_start=pos_dev, kv_len_from_position=True)
    torch.cuda.synchronize()
    ref = oracle.attention_seq_ref(q, k, v, 0.09, 4, pos + 1, pos, True)
    _check(out, ref)
    # fmha_causal: every row of k is in range, the causal rule alone ends at the position
    out2 = torch.full_like(out, float("nan"))
    ct.fmha_seq_f16(qd, kd, vd, ct.partition(out2, [1, 1, 128]), 0.09, 4, position_start=pos_dev, causal=True)
    torch.cuda.synchronize()
    _check(out2, ref)
    # ... and without it (CAUSAL = 0) all 512 rows count
    ct.fmha_seq_f16(qd, kd, vd, ct.partition(out2, [1, 1, 128]), 0.09, 4, position_start=pos_dev, causal=False)
    torch.cuda.synchronize()
    _check(out2, oracle.attention_seq_ref(q, k, v, 0.09, 4, 512, pos, False))


@pytest.mark.gpu
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("q_len,kv_len,start,d,pack", [(512, 512, 0, 128, 1), (256, 640, 384, 128, 4), (96, 96, 0, 64, 2),
                                                        (130, 77, 0, 128, 1)])
def test_gpu_fmha_prefill_causal_and_gqa(ct, dev, causal, q_len, kv_len, start, d, pack):
    """fmha_prefill_causal (tiles [BM, 1, D]) and fmha_prefill_gqa (tiles [BM, GROUP, D]) write the same outputs"""
    q, k, v = _inputs(q_len, 8, 2, 640, d, 741)
    out = torch.full((q_len, 8, d), float("nan"), dtype=torch.half, device=dev)
    ct.fmha_seq_f16(_dev(q, dev), _dev(k, dev), _dev(v, dev), ct.partition(out, [32, pack, d]), d ** -0.5, 4, kv_len=kv_len,
                    query_start=start, causal=causal)
    torch.cuda.synchronize()
    _check(out, oracle.attention_seq_ref(q, k, v, d ** -0.5, 4, kv_len, start, causal))


@pytest.mark.gpu
def test_gpu_seq_attention_empty_key_range_and_prefix_coverage(ct, dev):
    q, k, v = _inputs(128, 4, 2, 64, 64, 751)
    qd, kd, vd = _dev(q, dev), _dev(k, dev), _dev(v, dev)
    out = torch.full((128, 4, 64), float("nan"), dtype=torch.half, device=dev)
    ct.fmha_seq_f16(qd, kd, vd, ct.partition(out, [32, 1, 64]), 0.125, 2, kv_len=0)
    torch.cuda.synchronize()
    assert torch.all(out == 0)                                       # l_safe: attention.rs:383-386
    out.fill_(7.0)
    ct.fmha_seq_f16(qd, kd, vd, ct.partition(out, [32, 1, 64], prefix=True), 0.125, 2, kv_len=64, grid=(2, 3, 1))
    torch.cuda.synchronize()
    ref = oracle.attention_seq_ref(q, k, v, 0.125, 2, 64, 0, True)
    got = out.float().cpu().numpy()
    assert np.max(np.abs(got[:64, :3] - ref[:64, :3])) <= 2e-2
    assert np.all(got[64:] == 7.0) and np.all(got[:, 3] == 7.0)     # rows and heads outside the launch stay untouched


@pytest.mark.gpu
@pytest.mark.parametrize("causal", [True, False])
def test_gpu_fmha_prefill_gqa_lpt_raw(ct, dev, causal):
    """cutile-kernels/src/experimental/attention.rs:22-377: the raw-pointer form with caller-chosen block order computes
    fmha_prefill_gqa; k and v hold exactly kv_len rows per head"""
    q, k, v = _inputs(200, 8, 2, 320, 128, 761)
    out = torch.full((200, 8, 128), float("nan"), dtype=torch.half, device=dev)
    ct.fmha_prefill_gqa_lpt_raw_f16(_dev(q, dev), _dev(k, dev), _dev(v, dev), out, 128 ** -0.5, 4, 320, 120, 4, causal=causal,
                                    generics=[64, 64, 128, 4])
    torch.cuda.synchronize()
    _check(out, oracle.attention_seq_ref(q, k, v, 128 ** -0.5, 4, 320, 120, causal))
