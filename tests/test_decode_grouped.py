"""attention_decode_kernel_grouped (cutile-kernels/src/experimental/attention.rs:385-846): the split-KV decode partial
in batched layouts.  The reference only compiles it (cutile-kernels/tests/smoke.rs:408-412), so the oracle's
restatement is pinned by what the mathematics fixes: every split's output is softmax attention over its own keys
and its lse their base-2 log-sum-exp, both against float64; merging the splits by their lse gives attention over
all s_kv keys; keys at or beyond s_kv do not matter; a split without keys yields zeros and -inf.  Then the HIP kernel
is checked against the oracle through the C ABI (max-abs 2e-2 on the outputs as for the other attention kernels,
2e-3 on lse; observed: a few f16 ulps)."""
import struct

import numpy as np
import pytest
import torch

import oracle
from util import normal_f16_bits

f16 = lambda a: oracle.f32_to_f16_bits(np.asarray(a, np.float32))
f32 = oracle.f16_bits_to_f32


def _inputs(batch, heads, group, d, s_max, seed):
    return (normal_f16_bits((batch, heads, group, d), seed), normal_f16_bits((batch, heads, s_max, d), seed + 1),
            normal_f16_bits((batch, heads, s_max, d), seed + 2))


def _check_against_f64(q, k, v, att, lse, scale, s_kv, klps, tol_att=3e-3, tol_lse=2e-3):
    """every split on its own, then the merge of all splits, in float64"""
    qf, kf, vf = (f32(t).astype(np.float64) for t in (q, k, v))
    splits = att.shape[3]
    a, l = f32(att).astype(np.float64), lse.astype(np.float64)
    for sp in range(splits):
        lo, hi = sp * klps, min((sp + 1) * klps, s_kv)
        if lo >= hi:
            assert np.all(a[:, :, :, sp] == 0.0) and np.all(np.isneginf(lse[:, :, :, sp]))
            continue
        z = np.einsum("bhgd,bhsd->bhgs", qf, kf[:, :, lo:hi]) * scale * np.log2(np.e)
        p = np.exp2(z - z.max(-1, keepdims=True))
        want = np.einsum("bhgs,bhsd->bhgd", p / p.sum(-1, keepdims=True), vf[:, :, lo:hi])
        assert np.max(np.abs(a[:, :, :, sp] - want)) < tol_att
        assert np.max(np.abs(l[:, :, :, sp] - (np.log2(p.sum(-1)) + z.max(-1)))) < tol_lse
    if s_kv > 0:
        wgt = np.exp2(l - l.max(-1, keepdims=True))
        merged = (wgt[..., None] * a).sum(3) / wgt.sum(-1)[..., None]
        z = np.einsum("bhgd,bhsd->bhgs", qf, kf[:, :, :s_kv]) * scale
        p = np.exp(z - z.max(-1, keepdims=True))
        full = np.einsum("bhgs,bhsd->bhgd", p / p.sum(-1, keepdims=True), vf[:, :, :s_kv])
        assert np.max(np.abs(merged - full)) < tol_att


# ---- oracle (CPU) ---------------------------------------------------------------------------
@pytest.mark.parametrize("s_kv,tile_n,klps,splits", [(212, 32, 64, 5), (256, 64, 64, 4), (100, 32, 96, 4), (1, 16, 16, 3), (0, 32, 32, 2)])
def test_oracle_grouped_decode_is_softmax_attention_per_split(s_kv, tile_n, klps, splits):
    batch, heads, group, d, s_max = 2, 3, 4, 64, 320
    q, k, v = _inputs(batch, heads, group, d, s_max, 901)
    scale = float(np.float16(1.0 / np.sqrt(d)))
    att, lse = oracle.attention_decode_grouped_f16(q, k, v, scale, s_kv, tile_n, klps, splits)
    assert att.shape == (batch, heads, group, splits, d) and lse.shape == (batch, heads, group, splits)
    _check_against_f64(q, k, v, att, lse, scale, min(s_kv, splits * klps), klps)
    k2, v2 = k.copy(), v.copy()                                  # keys at or beyond s_kv must not matter
    k2[:, :, s_kv:], v2[:, :, s_kv:] = f16(100.0), f16(-100.0)
    att2, lse2 = oracle.attention_decode_grouped_f16(q, k2, v2, scale, s_kv, tile_n, klps, splits)
    assert np.array_equal(att, att2) and np.array_equal(lse, lse2)


def test_oracle_grouped_decode_one_key_returns_its_value_row():
    q, k, v = _inputs(1, 2, 8, 32, 40, 911)
    att, lse = oracle.attention_decode_grouped_f16(q, k, v, 0.25, 17, 16, 16, 2)
    # split 1 holds key 16 alone: softmax over one key is 1, lse its scaled score in base 2
    assert np.array_equal(att[:, :, :, 1], np.broadcast_to(v[:, :, None, 16], att[:, :, :, 1].shape))
    z = np.einsum("bhgd,bhd->bhg", f32(q).astype(np.float64), f32(k[:, :, 16]).astype(np.float64)) * 0.25 * np.log2(np.e)
    assert np.max(np.abs(lse[:, :, :, 1] - z)) < 1e-4


# ---- launcher on the recording runtime (CPU) ----------------------------------------------------
def test_grouped_decode_launcher_records_and_validates(fake_hip):
    ct = fake_hip
    from test_host_abi import _last
    h = torch.half
    q, k, v = torch.zeros(2, 8, 4, 128, dtype=h), torch.zeros(2, 8, 1024, 128, dtype=h), torch.zeros(2, 8, 1024, 128, dtype=h)
    att, lse = torch.zeros(2, 8, 4, 16, 128, dtype=h), torch.zeros(2, 8, 4, 16)
    s_kv = torch.zeros(1, dtype=torch.int32)
    ct.attention_decode_kernel_grouped_f16(q, k, v, att, lse, 0.088, s_kv, tile_n=32, kv_len_per_split=64, query_group_tile_size=16,
                                           generics=[128, 32, 64, 4, 16, 16])
    rec, args = _last(ct)
    assert rec.symbol == b"attention_decode_grouped_entry__f16_g4_d128" and tuple(rec.grid) == (2, 8, 16) and tuple(rec.block) == (256, 1, 1)
    ptrs = struct.unpack_from("<6Q", args, 0)
    assert ptrs == (q.data_ptr(), k.data_ptr(), v.data_ptr(), att.data_ptr(), lse.data_ptr(), s_kv.data_ptr())
    ints = struct.unpack_from("<19i", args, 48)
    assert ints[:3] == q.stride()[:3] and ints[3:6] == k.stride()[:3] and ints[6:9] == v.stride()[:3]
    assert ints[9:13] == att.stride()[:4] and ints[13:16] == lse.stride()[:3] and ints[16:] == (1024, 1024, 64)
    assert abs(struct.unpack_from("<f", args, 124)[0] - 0.088) < 1e-7 and struct.unpack_from("<3I", args, 128) == (2, 8, 16)
    n0 = ct.lib().cutile_testing_launch_count()
    call = lambda **kw: ct.attention_decode_kernel_grouped_f16(
        kw.get("q", q), kw.get("k", k), v, kw.get("att", att), kw.get("lse", lse), 0.088, s_kv, tile_n=kw.get("tile_n", 32),
        kv_len_per_split=kw.get("klps", 64), query_group_tile_size=kw.get("qgts", 16), grid=kw.get("grid"), generics=kw.get("generics"))
    cases = [
        (dict(klps=80), "multiple of TILE_N"),
        (dict(k=torch.zeros(2, 4, 1024, 128, dtype=h)), "do not agree"),
        (dict(lse=torch.zeros(2, 8, 4, 8)), "do not agree"),
        (dict(qgts=2), "QUERY_GROUP_TILE_SIZE"),
        (dict(q=torch.zeros(2, 8, 3, 128, dtype=h), att=torch.zeros(2, 8, 3, 16, 128, dtype=h), lse=torch.zeros(2, 8, 3, 16)), "no precompiled variant"),
        (dict(q=torch.zeros(2, 8, 4, 129, dtype=h)[..., 1:]), "16-byte aligned"),
        (dict(grid=(8, 2, 16)), "launch grid"),
        (dict(generics=[128, 32, 64, 4, 16, 8]), "NUM_KV_SPLITS"),
    ]
    for kw, msg in cases:
        with pytest.raises(ct.CutileError, match=msg):
            call(**kw)
    assert ct.lib().cutile_testing_launch_count() == n0


# ---- HIP kernel (GPU) ---------------------------------------------------------------------------
def _dev16(bits, dev):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(dev).view(torch.half)


@pytest.mark.gpu
@pytest.mark.parametrize("batch,heads,group,d,s_max,s_kv,tile_n,klps,splits", [
    (2, 8, 4, 128, 1024, 700, 64, 128, 8),       # the last two splits are empty, one is cut by s_kv
    (1, 2, 8, 64, 300, 300, 32, 64, 5),          # s_kv = all rows, the last split is short
    (3, 1, 1, 256, 200, 1, 64, 64, 4),           # one key
    (2, 3, 2, 128, 520, 131, 16, 16, 16),        # one tile per split, more splits than needed
    (1, 2, 16, 64, 260, 257, 32, 96, 3),
    (2, 2, 4, 64, 128, 0, 32, 32, 2),            # nothing cached yet: every split is empty
    (1, 4, 8, 256, 2100, 2099, 128, 512, 5),
])
def test_gpu_grouped_decode(ct, dev, batch, heads, group, d, s_max, s_kv, tile_n, klps, splits):
    q, k, v = _inputs(batch, heads, group, d, s_max, 921)
    scale = float(np.float16(1.0 / np.sqrt(d)))
    att = torch.full((batch, heads, group, splits, d), float("nan"), dtype=torch.half, device=dev)
    lse = torch.full((batch, heads, group, splits), float("nan"), device=dev)
    count = torch.tensor([s_kv], dtype=torch.int32, device=dev)
    ct.attention_decode_kernel_grouped_f16(_dev16(q, dev), _dev16(k, dev), _dev16(v, dev), att, lse, scale, count, tile_n=tile_n,
                                           kv_len_per_split=klps, query_group_tile_size=max(group, 16))
    torch.cuda.synchronize()
    att_ref, lse_ref = oracle.attention_decode_grouped_f16(q, k, v, scale, s_kv, tile_n, klps, splits)
    got_att, got_lse = att.cpu().view(torch.int16).numpy().view(np.uint16), lse.cpu().numpy()
    live = np.isfinite(lse_ref)
    assert np.array_equal(live, np.isfinite(got_lse)) and np.all(np.isneginf(got_lse[~live]))
    assert np.max(np.abs(f32(got_att) - f32(att_ref))) <= 2e-2
    assert live.sum() == 0 or np.max(np.abs(got_lse[live] - lse_ref[live])) <= 2e-3
    _check_against_f64(q, k, v, got_att, got_lse, scale, min(s_kv, splits * klps), klps, tol_att=4e-3)


@pytest.mark.gpu
def test_gpu_grouped_decode_strided_views(ct, dev):
    """every tensor a view of a larger allocation: the strides the reference passes as scalars are honoured"""
    batch, heads, group, d, s_max, s_kv, tile_n, klps, splits = 2, 3, 4, 128, 192, 150, 32, 64, 3
    q, k, v = _inputs(batch, heads, group, d, s_max, 931)
    scale = float(np.float16(1.0 / np.sqrt(d)))
    big_q = torch.zeros(batch, heads + 1, group + 2, d + 8, dtype=torch.half, device=dev)
    big_k = torch.zeros(batch, heads, s_max + 5, 2 * d, dtype=torch.half, device=dev)
    big_v = torch.zeros(batch + 1, heads, s_max, d + 16, dtype=torch.half, device=dev)
    qv, kv, vv = big_q[:, :heads, :group, :d], big_k[:, :, :s_max, :d], big_v[:batch, :, :, :d]
    qv.copy_(_dev16(q, dev)); kv.copy_(_dev16(k, dev)); vv.copy_(_dev16(v, dev))
    big_att = torch.full((batch, heads, group + 1, splits + 2, d + 8), 7.0, dtype=torch.half, device=dev)
    big_lse = torch.full((batch, heads + 2, group, splits), 7.0, device=dev)
    attv, lsev = big_att[:, :, :group, :splits, :d], big_lse[:, :heads]
    count = torch.tensor([s_kv], dtype=torch.int32, device=dev)
    ct.attention_decode_kernel_grouped_f16(qv, kv, vv, attv, lsev, scale, count, tile_n=tile_n, kv_len_per_split=klps)
    torch.cuda.synchronize()
    att_ref, lse_ref = oracle.attention_decode_grouped_f16(q, k, v, scale, s_kv, tile_n, klps, splits)
    got = attv.contiguous().cpu().view(torch.int16).numpy().view(np.uint16)
    assert np.max(np.abs(f32(got) - f32(att_ref))) <= 2e-2 and np.max(np.abs(lsev.cpu().numpy() - lse_ref)) <= 2e-3
    # nothing outside the views was written
    big_att[:, :, :group, :splits, :d] = 7.0
    big_lse[:, :heads] = 7.0
    assert torch.all(big_att == 7.0) and torch.all(big_lse == 7.0)
