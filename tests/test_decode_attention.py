"""Decode-time kernels of cutile-kernels: kv_cache_update_seq(_dynpos)_f16 (kv_cache.rs:15-49, 58-97),
fmha_decode_gqa_split and splitk_reduce_merge (attention.rs:737-902, 917-1013).  The reference holds no
numeric test for them (cutile-kernels/tests/smoke.rs only compiles them), so the oracle's restatements
are pinned here by what the mathematics fixes: split + merge must equal softmax attention over keys
0..position evaluated in float64, whatever the number of splits; the merge has closed forms of its own;
the cache update is an exact copy.  Then the HIP kernels are checked against the oracle through the C ABI."""
import numpy as np
import pytest
import torch

import oracle
from util import f16_ulp_diff, normal_f16_bits

f16 = lambda a: oracle.f32_to_f16_bits(np.asarray(a, np.float32))
f32 = oracle.f16_bits_to_f32


def _attention_f64(q, k, v, scale, pos):
    """softmax(q k^T * scale) v over keys 0..pos, float64; q [H, G, D], k/v [H, S, D] (f16 bits)"""
    qf, kf, vf = (f32(t).astype(np.float64) for t in (q, k, v))
    s = np.einsum("hgd,hsd->hgs", qf, kf[:, : pos + 1]) * scale
    p = np.exp(s - s.max(axis=-1, keepdims=True))
    return np.einsum("hgs,hsd->hgd", p / p.sum(axis=-1, keepdims=True), vf[:, : pos + 1]), s


# ---- oracle (CPU) ---------------------------------------------------------------------------
@pytest.mark.parametrize("splits", [1, 3, 8])
def test_oracle_decode_split_then_merge_is_softmax_attention(splits):
    heads, group, d, max_seq, pos, bn = 3, 4, 64, 300, 212, 32
    q, k, v = normal_f16_bits((heads, group, d), 701), normal_f16_bits((heads, max_seq, d), 702), normal_f16_bits((heads, max_seq, d), 703)
    scale = float(np.float16(1.0 / np.sqrt(d)))
    att, lse = oracle.fmha_decode_gqa_split(q, k, v, scale, pos, bn, splits)
    out = f32(oracle.splitk_reduce_merge(att, lse, group)).astype(np.float64)
    ref, s = _attention_f64(q, k, v, scale, pos)
    assert np.max(np.abs(out - ref)) < 3e-3                      # f16 partials and output, |v| up to ~4
    # keys beyond pos must not matter: poison them
    k2, v2 = k.copy(), v.copy()
    k2[:, pos + 1:], v2[:, pos + 1:] = f16(100.0), f16(-100.0)
    att2, lse2 = oracle.fmha_decode_gqa_split(q, k2, v2, scale, pos, bn, splits)
    assert np.array_equal(att, att2) and np.array_equal(lse, lse2)
    # each split's lse is the base-2 log-sum-exp of its own scores
    tiles = -(-(pos + 1) // bn)
    per = -(-tiles // splits)
    for sp in range(splits):
        lo, hi = sp * per * bn, min(min((sp + 1) * per, tiles) * bn, pos + 1)
        got = lse[:, sp * group:(sp + 1) * group]
        if lo >= hi:                                             # no keys: the tile program's untouched state
            assert np.all(f32(att[:, sp * group:(sp + 1) * group]) == 0.0)
            assert np.allclose(got, -1.0e30 + np.log2(bn))
            continue
        z = s[:, :, lo:hi] * np.log2(np.e)
        want = np.log2(np.exp2(z - z.max(-1, keepdims=True)).sum(-1)) + z.max(-1)
        assert np.max(np.abs(got - want)) < 2e-3


def test_oracle_merge_closed_forms():
    heads, group, d, splits = 2, 2, 16, 4
    att = normal_f16_bits((heads, splits * group, d), 711)
    a = f32(att).astype(np.float64).reshape(heads, splits, group, d)
    # equal lse -> plain mean of the partials
    out = f32(oracle.splitk_reduce_merge(att, np.full((heads, splits * group), 3.25, np.float32), group))
    assert np.max(np.abs(out - a.mean(axis=1))) < 2e-3
    # one split 40 octaves above the rest -> that partial, exactly
    lse = np.zeros((heads, splits, group), np.float32)
    lse[:, 2] = 40.0
    out = oracle.splitk_reduce_merge(att, lse.reshape(heads, -1), group)
    assert np.array_equal(out, att.reshape(heads, splits, group, d)[:, 2])
    # general weights 2^lse / sum 2^lse, per (head, group) column
    lse = oracle.uniform_f32((heads, splits, group), 712, -3.0, 3.0)
    w = np.exp2(lse.astype(np.float64))
    w /= w.sum(axis=1, keepdims=True)
    out = f32(oracle.splitk_reduce_merge(att, lse.reshape(heads, -1), group))
    assert np.max(np.abs(out - (w[..., None] * a).sum(axis=1))) < 2e-3
    # an empty split (att 0, lse ~ -1e30) is ignored
    lse[:, 1] = -1.0e30
    w = np.exp2(np.where(lse < -1e29, -np.inf, lse).astype(np.float64))
    w /= w.sum(axis=1, keepdims=True)
    out = f32(oracle.splitk_reduce_merge(att, lse.reshape(heads, -1), group))
    assert np.max(np.abs(out - (w[..., None] * a).sum(axis=1))) < 2e-3


def test_oracle_decode_one_key_returns_its_value_row():
    q, k, v = normal_f16_bits((2, 8, 128), 721), normal_f16_bits((2, 10, 128), 722), normal_f16_bits((2, 10, 128), 723)
    att, lse = oracle.fmha_decode_gqa_split(q, k, v, 0.0884, 0, 64, 1)      # position 0: softmax over one key is 1
    assert np.array_equal(att, np.broadcast_to(v[:, :1], (2, 8, 128)))
    s = np.einsum("hgd,hd->hg", f32(q).astype(np.float64), f32(k[:, 0]).astype(np.float64)) * 0.0884 * np.log2(np.e)
    assert np.max(np.abs(lse - s)) < 1e-3


def test_oracle_kv_cache_update_is_an_exact_copy_of_the_new_rows():
    heads, max_seq, d, seq = 3, 20, 16, 5
    nk, nv = normal_f16_bits((seq, heads, d), 731), normal_f16_bits((seq, heads, d), 732)
    kc, vc = normal_f16_bits((heads, max_seq, d), 733), normal_f16_bits((heads, max_seq, d), 734)
    k2, v2 = oracle.kv_cache_update_f16(nk, nv, kc, vc, 7, 4)
    assert np.array_equal(k2[:, 7:11], nk[:4].transpose(1, 0, 2)) and np.array_equal(v2[:, 7:11], nv[:4].transpose(1, 0, 2))
    keep = np.ones(max_seq, bool)
    keep[7:11] = False
    assert np.array_equal(k2[:, keep], kc[:, keep]) and np.array_equal(v2[:, keep], vc[:, keep])
    k3, v3 = oracle.kv_cache_update_f16(nk, nv, kc, vc, 3, 0)                 # seq_len 0: nothing written
    assert np.array_equal(k3, kc) and np.array_equal(v3, vc)


# ---- HIP kernels (GPU) -----------------------------------------------------------------------
def _dev(bits, dev):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.float16)).to(dev)


def _bits(t):
    return t.cpu().numpy().view(np.uint16)


@pytest.mark.gpu
def test_gpu_kv_cache_update_both_forms(ct, dev):
    heads, max_seq, d, seq = 8, 96, 128, 33
    nk, nv = normal_f16_bits((seq, heads, d), 741), normal_f16_bits((seq, heads, d), 742)
    kc, vc = normal_f16_bits((heads, max_seq, d), 743), normal_f16_bits((heads, max_seq, d), 744)
    # prefill form: position by value (0), BM_S rows per tile block
    kd, vd = _dev(kc, dev), _dev(vc, dev)
    ct.kv_cache_update_f16(_dev(nk, dev), _dev(nv, dev), ct.partition(kd, [1, 16, 64]), ct.partition(vd, [1, 16, 64]), 0, seq,
                           generics=[d, 64, 16])
    torch.cuda.synchronize()
    k_ref, v_ref = oracle.kv_cache_update_f16(nk, nv, kc, vc, 0, seq)
    assert np.array_equal(_bits(kd), k_ref) and np.array_equal(_bits(vd), v_ref)
    with pytest.raises(ct.CutileError, match="position_start must be 0"):
        ct.kv_cache_update_f16(_dev(nk, dev), _dev(nv, dev), ct.partition(kd, [1, 16, 64]), ct.partition(vd, [1, 16, 64]), 4, seq)
    # decode form: position from device memory, one token and several
    pos = torch.tensor([57], dtype=torch.int32, device=dev)
    for n in (1, 5):
        kd, vd = _dev(kc, dev), _dev(vc, dev)
        ct.kv_cache_update_f16(_dev(nk, dev), _dev(nv, dev), ct.partition(kd, [1, max_seq, 128]), ct.partition(vd, [1, max_seq, 128]),
                               pos, n, generics=[d, 128, max_seq])
        torch.cuda.synchronize()
        k_ref, v_ref = oracle.kv_cache_update_f16(nk, nv, kc, vc, 57, n)
        assert np.array_equal(_bits(kd), k_ref) and np.array_equal(_bits(vd), v_ref)
    # a head dimension that rules out 16-byte accesses, strided cache view
    d2 = 12
    nk2, nv2 = normal_f16_bits((3, 2, d2), 745), normal_f16_bits((3, 2, d2), 746)
    wide_k = torch.zeros(2, 10, d2 + 4, dtype=torch.float16, device=dev)
    wide_v = torch.zeros(2, 10, d2 + 4, dtype=torch.float16, device=dev)
    pos2 = torch.tensor([6], dtype=torch.int32, device=dev)
    ct.kv_cache_update_f16(_dev(nk2, dev), _dev(nv2, dev), ct.partition(wide_k[..., :d2], [1, 10, d2]),
                           ct.partition(wide_v[..., :d2], [1, 10, d2]), pos2, 3)
    torch.cuda.synchronize()
    zero = np.zeros((2, 10, d2), np.uint16)
    k_ref, v_ref = oracle.kv_cache_update_f16(nk2, nv2, zero, zero, 6, 3)
    assert np.array_equal(_bits(wide_k[..., :d2].contiguous()), k_ref) and np.array_equal(_bits(wide_v[..., :d2].contiguous()), v_ref)
    assert torch.all(wide_k[..., d2:] == 0) and torch.all(wide_v[..., d2:] == 0)


def _run_decode(ct, dev, q, k, v, scale, pos, bn, splits, variant=None):
    heads, group, d = q.shape
    att = torch.full((heads, splits * group, d), float("nan"), dtype=torch.float16, device=dev)
    lse = torch.full((heads, splits * group), float("nan"), dtype=torch.float32, device=dev)
    out = torch.full((heads, group, d), float("nan"), dtype=torch.float16, device=dev)
    p = torch.tensor([pos], dtype=torch.int32, device=dev)
    ct.fmha_decode_gqa_split(_dev(q, dev), _dev(k, dev), _dev(v, dev), ct.partition(att, [1, group, d]),
                             ct.partition(lse, [1, group]), scale, p, generics=[group, bn, d, splits], variant=variant)
    ct.splitk_reduce_merge(att, lse, ct.partition(out, [1, group, d]), generics=[group, d, d, splits])
    torch.cuda.synchronize()
    return _bits(att), lse.cpu().numpy(), _bits(out)


@pytest.mark.gpu
@pytest.mark.parametrize("heads,group,d,max_seq,pos,bn,splits", [
    (8, 4, 128, 1024, 700, 64, 8),        # the reference's decode configuration shape (GROUP 4, D 128)
    (2, 8, 64, 300, 299, 32, 3),          # the last cache row is the newest key
    (4, 1, 256, 200, 0, 64, 4),           # one key: three of four splits are empty
    (3, 2, 128, 520, 130, 64, 16),        # more splits than tiles
    (1, 8, 256, 4100, 4099, 128, 5),
    (4, 16, 128, 1500, 1403, 64, 6),      # GROUP 16 exists on the matrix cores only
    (2, 16, 64, 90, 70, 16, 2),
])
def test_gpu_decode_split_and_merge(ct, dev, heads, group, d, max_seq, pos, bn, splits):
    q, k, v = normal_f16_bits((heads, group, d), 751), normal_f16_bits((heads, max_seq, d), 752), normal_f16_bits((heads, max_seq, d), 753)
    scale = float(np.float16(1.0 / np.sqrt(d)))
    att, lse, out = _run_decode(ct, dev, q, k, v, scale, pos, bn, splits)
    att_ref, lse_ref = oracle.fmha_decode_gqa_split(q, k, v, scale, pos, bn, splits)
    out_ref = oracle.splitk_reduce_merge(att_ref, lse_ref, group)
    if group <= 8:      # two variants up to GROUP 8 (vector ALUs, matrix cores): whichever is not the default must hold too
        for variant in (f"f16_g{group}_d{d}", f"f16_g{group}_d{d}_mfma"):
            att_v, lse_v, out_v = _run_decode(ct, dev, q, k, v, scale, pos, bn, splits, variant=variant)
            assert np.max(np.abs(f32(att_v) - f32(att_ref))) <= 2e-2 and np.max(np.abs(f32(out_v) - f32(out_ref))) <= 2e-2
            assert np.array_equal(lse_ref > -1e29, lse_v > -1e29) and np.allclose(lse_v, lse_ref, atol=2e-3)
    # tolerance: max-abs 2e-2 as for the prefill attention kernel; observed differences are a few f16 ulps
    # (the kernel sums each split's keys in a different order than the tile program does)
    assert np.max(np.abs(f32(att) - f32(att_ref))) <= 2e-2
    live = lse_ref > -1e29
    assert np.array_equal(live, lse > -1e29)
    assert np.max(np.abs(lse[live] - lse_ref[live])) <= 2e-3 and np.allclose(lse[~live], lse_ref[~live])
    assert np.max(np.abs(f32(out) - f32(out_ref))) <= 2e-2
    ref64, _ = _attention_f64(q, k, v, scale, pos)
    assert np.max(np.abs(f32(out) - ref64)) <= 2e-2
    # the merge kernel alone, on the oracle's partials: same inputs, so a few ulps at most
    o2 = torch.zeros(heads, group, d, dtype=torch.float16, device=dev)
    ct.splitk_reduce_merge(_dev(att_ref, dev), torch.from_numpy(lse_ref).to(dev), ct.partition(o2, [1, group, d // 2]))
    torch.cuda.synchronize()
    assert np.max(f16_ulp_diff(_bits(o2), out_ref)) <= 2


@pytest.mark.gpu
def test_gpu_decode_rejects_what_no_variant_covers(ct, dev):
    q = torch.zeros(2, 3, 128, dtype=torch.float16, device=dev)            # GROUP 3
    kv = torch.zeros(2, 64, 128, dtype=torch.float16, device=dev)
    att = torch.zeros(2, 6, 128, dtype=torch.float16, device=dev)
    lse = torch.zeros(2, 6, dtype=torch.float32, device=dev)
    p = torch.zeros(1, dtype=torch.int32, device=dev)
    with pytest.raises(ct.CutileError, match="no precompiled variant"):
        ct.fmha_decode_gqa_split(q, kv, kv, ct.partition(att, [1, 3, 128]), ct.partition(lse, [1, 3]), 0.1, p)
    q4 = torch.zeros(2, 4, 128, dtype=torch.float16, device=dev)
    att4 = torch.zeros(2, 8, 128, dtype=torch.float16, device=dev)
    lse4 = torch.zeros(2, 8, dtype=torch.float32, device=dev)
    with pytest.raises(ct.CutileError, match="NUM_KV_SPLITS"):
        ct.fmha_decode_gqa_split(q4, kv, kv, ct.partition(att4, [1, 4, 128]), ct.partition(lse4, [1, 4]), 0.1, p,
                                 generics=[4, 64, 128, 3])


@pytest.mark.gpu
def test_gpu_decode_step_replayed_from_a_captured_graph(ct, dev):
    """one decode step (cache update at the device position, split attention, merge) captured once and replayed with the
    program's own eager work between the replays: every replay must equal the eager step on the same inputs"""
    heads, group, d, max_seq, splits = 4, 4, 128, 512, 4
    rng = np.random.default_rng(77)
    half = lambda *shape: torch.from_numpy(rng.standard_normal(shape).astype(np.float16)).to(dev)
    q, new_k, new_v = half(heads, group, d), half(1, heads, d), half(1, heads, d)
    k_cache, v_cache = half(heads, max_seq, d), half(heads, max_seq, d)
    pos = torch.tensor([100], dtype=torch.int32, device=dev)
    att = torch.zeros(heads, splits * group, d, dtype=torch.float16, device=dev)
    lse = torch.zeros(heads, splits * group, device=dev)
    out = torch.zeros(heads, group, d, dtype=torch.float16, device=dev)

    def step(stream=None):
        ct.kv_cache_update_f16(new_k, new_v, ct.partition(k_cache, [1, max_seq, d]), ct.partition(v_cache, [1, max_seq, d]), pos, 1, stream=stream)
        ct.fmha_decode_gqa_split(q, k_cache, v_cache, ct.partition(att, [1, group, d]), ct.partition(lse, [1, group]), d ** -0.5, pos, stream=stream)
        ct.splitk_reduce_merge(att, lse, ct.partition(out, [1, group, d]), stream=stream)

    torch.cuda.synchronize()
    graph = ct.CapturedGraph().capture(step)
    try:
        for it in range(4):
            # new inputs through the same buffers, written by eager work on torch's stream
            q.copy_(half(heads, group, d)); new_k.copy_(half(1, heads, d)); new_v.copy_(half(1, heads, d))
            pos.fill_(100 + 37 * it)
            saved_k, saved_v = k_cache.clone(), v_cache.clone()
            torch.cuda.synchronize()
            graph.launch()
            graph.synchronize()
            got, got_k = out.clone(), k_cache.clone()
            k_cache.copy_(saved_k); v_cache.copy_(saved_v); out.zero_()
            step()
            torch.cuda.synchronize()
            assert torch.equal(got, out) and torch.equal(got_k, k_cache)
            assert torch.equal(k_cache[:, 100 + 37 * it], new_k[0])
    finally:
        graph.close()
