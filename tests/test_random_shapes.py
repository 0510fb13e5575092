"""Seeded sweeps over shapes nobody hand-picked: the hot kernels against the oracle at randomly drawn sizes, ragged
edges, strides, head groupings and causal offsets (fixed seeds, so a failure names its case and repeats)."""
import numpy as np
import pytest
import torch

import oracle
from util import (assert_rounded_close, f16_ulp_diff, from_dev_f16_bits, normal_bf16_bits, normal_f16_bits, rel_l2, to_dev_bf16,
                  to_dev_f16)

pytestmark = pytest.mark.gpu


def _cases(seed, n, draw):
    rng = np.random.default_rng(seed)
    return [draw(rng) for _ in range(n)]


GEMM_CASES = _cases(9001, 14, lambda r: (int(r.integers(1, 900)), int(r.integers(1, 900)), int(r.integers(1, 12)) * 64 + int(r.choice([0, 0, 8, 24, 40])),
                                         [(256, 256), (128, 128), (64, 128), (128, 256)][int(r.integers(0, 4))], bool(r.integers(0, 2))))


@pytest.mark.parametrize("m,n,k,tile,accumulate", GEMM_CASES)
def test_gemm_bf16_random_shapes(ct, dev, m, n, k, tile, accumulate):
    # N a multiple of 8 keeps the matrix-core variants eligible; every third case keeps an odd N for the any-layout kernel
    n8 = n if (m + n + k) % 3 == 0 else max(8, n // 8 * 8)
    a, b = normal_bf16_bits((m, k), 3000 + m, k ** -0.5), normal_bf16_bits((k, n8), 3001 + n, k ** -0.5)
    z0 = normal_bf16_bits((m, n8), 3002 + k, 0.5) if accumulate else np.zeros((m, n8), np.uint16)
    z = to_dev_bf16(z0, dev).clone()
    ct.gemm(ct.partition(z, list(tile)), to_dev_bf16(a, dev), to_dev_bf16(b, dev), k, accumulate=accumulate)
    torch.cuda.synchronize()
    k_used = k // 64 * 64                      # the tile program runs k / BK whole K tiles
    ref = oracle.gemm_bf16(a[:, :k_used], b[:k_used], f32out=True) + (oracle.bf16_bits_to_f32(z0) if accumulate else 0.0)
    got = z.float().cpu().numpy()
    assert rel_l2(got, ref) <= 1e-2
    assert_rounded_close(got, ref, tile, what=f"gemm {m}x{n8}x{k} {tile} acc={accumulate}")


FMHA_CASES = _cases(9002, 14, lambda r: (int(r.integers(1, 3)), [1, 2, 4][int(r.integers(0, 3))], int(r.integers(1, 3)), int(r.integers(1, 700)),
                                         [64, 128, 128, 256][int(r.integers(0, 4))], bool(r.integers(0, 2)), int(r.integers(0, 40)),
                                         [torch.bfloat16, torch.float16][int(r.integers(0, 2))]))


@pytest.mark.parametrize("b,group,hkv,s,d,causal,input_pos,dtype", FMHA_CASES)
def test_fmha_random_shapes(ct, dev, b, group, hkv, s, d, causal, input_pos, dtype):
    h = hkv * group
    bm = 256 if (d == 128 and s > 300) else 128        # tile heights both element types are precompiled for
    cast = (lambda x: oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(x))) if dtype == torch.bfloat16 else (
        lambda x: oracle.f16_bits_to_f32(oracle.f32_to_f16_bits(x)))
    q = cast(oracle.normal_f32((b, h, s, d), 4000 + s))
    k, v = cast(oracle.normal_f32((b, hkv, s, d), 4001 + s)), cast(oracle.normal_f32((b, hkv, s, d), 4002 + s))
    out = torch.full((b * h, s, d), float("nan"), dtype=dtype, device=dev)
    td = lambda t: torch.from_numpy(t).to(dev).to(dtype)
    pos = input_pos if causal else 0
    ct.fmha(ct.partition(out, [1, bm, d]), td(q), td(k), td(v), d ** -0.5, pos, group, causal=causal)
    torch.cuda.synchronize()
    ref = oracle.fmha_ref_cpu(q, k, v, d ** -0.5, pos, group, causal).reshape(b * h, s, d)
    got = out.float().cpu().numpy()
    assert np.isfinite(got).all()
    assert np.max(np.abs(got - ref)) <= 2e-2


ROW_CASES = _cases(9003, 12, lambda r: (int(r.integers(1, 200)), int(r.choice([int(r.integers(1, 40)) * 8, int(r.integers(9, 3000)), 1 << int(r.integers(6, 14))]))))


@pytest.mark.parametrize("rows,n", ROW_CASES)
def test_row_kernels_random_shapes(ct, dev, rows, n):
    x, w = normal_f16_bits((rows, n), 5000 + n), normal_f16_bits((n,), 5001 + n)
    out = torch.zeros(rows, n, dtype=torch.half, device=dev)
    ct.rms_norm_f16(to_dev_f16(x, dev), to_dev_f16(w, dev), ct.partition(out, [1, n]), 1e-6)
    torch.cuda.synchronize()
    assert f16_ulp_diff(from_dev_f16_bits(out), oracle.rms_norm_f16(x, w, 1e-6)).max() <= 1
    ct.softmax(to_dev_f16(x, dev), ct.partition(out, [1, n]))
    torch.cuda.synchronize()
    got, ref = from_dev_f16_bits(out), oracle.softmax_f16(x, 1, n)
    d = np.abs(oracle.f16_bits_to_f32(got) - oracle.f16_bits_to_f32(ref))
    assert np.all(d <= np.abs(oracle.f16_bits_to_f32(ref)) * 2.0 ** -10 + 1e-7)
    # a view with a padded row pitch takes the any-layout kernels: same answers
    wide = torch.zeros(rows, n + 5, dtype=torch.half, device=dev)
    xin = torch.zeros(rows, n + 3, dtype=torch.half, device=dev)
    xin[:, :n] = to_dev_f16(x, dev)
    ct.rms_norm_f16(xin[:, :n], to_dev_f16(w, dev), ct.partition(wide[:, :n], [1, n]), 1e-6)
    torch.cuda.synchronize()
    assert f16_ulp_diff(from_dev_f16_bits(wide[:, :n].contiguous()), oracle.rms_norm_f16(x, w, 1e-6)).max() <= 1
    assert torch.all(wide[:, n:] == 0)


MX_CASES = _cases(9004, 8, lambda r: (int(r.integers(1, 700)), int(r.integers(1, 700)), int(r.integers(1, 9)) * 128,
                                      [torch.float32, torch.bfloat16][int(r.integers(0, 2))]))


@pytest.mark.parametrize("m,n,k,out_dtype", MX_CASES)
def test_mxfp8_random_shapes(ct, dev, m, n, k, out_dtype):
    n = max(8, n // 8 * 8)
    xf = oracle.normal_f32((m, k), 6000 + m) * np.exp2(oracle.uniform_f32((m, k // 32), 6001 + m, -4, 4)).repeat(32, axis=1)
    yf = oracle.normal_f32((n, k), 6002 + n) * np.exp2(oracle.uniform_f32((n, k // 32), 6003 + n, -4, 4)).repeat(32, axis=1)
    xq, xs = oracle.mx_quantize_e4m3(xf)
    yq, ys = oracle.mx_quantize_e4m3(yf)
    z = torch.full((m, n), float("nan"), dtype=out_dtype, device=dev)
    td = lambda t: torch.from_numpy(t).to(dev)
    ct.linear_tile_mxfp8(ct.partition(z, [256, 256]), td(xq), td(yq), td(xs), td(ys), 1.25)
    torch.cuda.synchronize()
    ref = oracle.mx_gemm_f32(xq, yq, xs, ys, 1.25)
    mag = oracle.mx_gemm_f32(xq & 0x7F, yq & 0x7F, xs, ys, 1.25)
    got = z.float().cpu().numpy()
    assert np.isfinite(got).all() and rel_l2(got, ref) <= 3e-2
    assert_rounded_close(got, ref, (256, 256), rel_ulp=1e-5 if out_dtype == torch.float32 else 2.0 ** -7, atol_frac=1e-4, what="mxfp8", mag=mag)


DECODE_CASES = _cases(9005, 10, lambda r: (int(r.integers(1, 9)), [1, 2, 4, 8, 16][int(r.integers(0, 5))], [64, 128, 256][int(r.integers(0, 3))],
                                           int(r.integers(1, 3000)), [16, 32, 64, 128][int(r.integers(0, 4))], int(r.integers(1, 20))))


@pytest.mark.parametrize("heads,group,d,pos,bn,splits", DECODE_CASES)
def test_decode_attention_random_shapes(ct, dev, heads, group, d, pos, bn, splits):
    max_seq = pos + 1 + (pos * 7) % 50           # the cache holds rows past the newest key; they must not matter
    q, k, v = normal_f16_bits((heads, group, d), 7000 + pos), normal_f16_bits((heads, max_seq, d), 7001 + pos), normal_f16_bits((heads, max_seq, d), 7002 + pos)
    scale = float(np.float16(1.0 / np.sqrt(d)))
    dv = lambda bits: torch.from_numpy(np.ascontiguousarray(bits).view(np.float16)).to(dev)
    att = torch.full((heads, splits * group, d), float("nan"), dtype=torch.float16, device=dev)
    lse = torch.full((heads, splits * group), float("nan"), dtype=torch.float32, device=dev)
    out = torch.full((heads, group, d), float("nan"), dtype=torch.float16, device=dev)
    p = torch.tensor([pos], dtype=torch.int32, device=dev)
    ct.fmha_decode_gqa_split(dv(q), dv(k), dv(v), ct.partition(att, [1, group, d]), ct.partition(lse, [1, group]), scale, p,
                             generics=[group, bn, d, splits])
    ct.splitk_reduce_merge(att, lse, ct.partition(out, [1, group, d]), generics=[group, d, d, splits])
    torch.cuda.synchronize()
    att_ref, lse_ref = oracle.fmha_decode_gqa_split(q, k, v, scale, pos, bn, splits)
    out_ref = oracle.splitk_reduce_merge(att_ref, lse_ref, group)
    f32 = oracle.f16_bits_to_f32
    got = out.cpu().numpy().view(np.uint16)
    assert np.isfinite(f32(got)).all() and np.max(np.abs(f32(got) - f32(out_ref))) <= 2e-2
    live = lse_ref > -1e29
    assert np.array_equal(live, lse.cpu().numpy() > -1e29)
    assert np.max(np.abs(lse.cpu().numpy()[live] - lse_ref[live])) <= 2e-3
    # float64 softmax attention over keys 0..pos of each KV head
    qf, kf, vf = f32(q).astype(np.float64), f32(k).astype(np.float64)[:, :pos + 1], f32(v).astype(np.float64)[:, :pos + 1]
    sc = np.einsum("hgd,hkd->hgk", qf, kf) * scale
    w = np.exp(sc - sc.max(-1, keepdims=True))
    ref64 = np.einsum("hgk,hkd->hgd", w / w.sum(-1, keepdims=True), vf)
    assert np.max(np.abs(f32(got) - ref64)) <= 2e-2
