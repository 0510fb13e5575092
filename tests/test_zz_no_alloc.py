"""The decode-attention entry point that allocates nothing (cutile_launch_fmha_decode_gqa_noalloc): its partial results
live in the library's device-resident scratch array.  It must give what the split + merge entry points give with
caller-allocated partials, bit for bit (same kernels, same inputs), on calls in a row that share the scratch."""
import numpy as np
import pytest
import torch

import oracle
from util import normal_f16_bits

f32 = oracle.f16_bits_to_f32


def _dev(bits, dev):
    return torch.from_numpy(bits.view(np.float16)).to(dev)


def _reference_step(ct, dev, q, k, v, scale, pos, bn, splits):
    heads, group, d = q.shape
    att = torch.full((heads, splits * group, d), float("nan"), dtype=torch.float16, device=dev)
    lse = torch.full((heads, splits * group), float("nan"), dtype=torch.float32, device=dev)
    out = torch.full((heads, group, d), float("nan"), dtype=torch.float16, device=dev)
    ct.fmha_decode_gqa_split(q, k, v, ct.partition(att, [1, group, d]), ct.partition(lse, [1, group]), scale, pos,
                             generics=[group, bn, d, splits])
    ct.splitk_reduce_merge(att, lse, ct.partition(out, [1, group, d]))
    torch.cuda.synchronize()
    return out


@pytest.mark.gpu
def test_gpu_decode_noalloc_matches_split_and_merge_on_calls_in_a_row(ct, dev):
    # the second call is smaller in every extent, so it reuses a part of what the first left in the scratch
    cases = [(8, 4, 128, 2048, 1900, 64, 16, 761), (2, 8, 64, 300, 130, 32, 3, 771), (4, 1, 256, 200, 0, 64, 4, 781)]
    for heads, group, d, max_seq, pos, bn, splits, seed in cases:
        print(f"noalloc case heads={heads} group={group} d={d} pos={pos} splits={splits}", flush=True)
        qb, kb, vb = (normal_f16_bits((heads, group, d), seed), normal_f16_bits((heads, max_seq, d), seed + 1),
                      normal_f16_bits((heads, max_seq, d), seed + 2))
        q, k, v = _dev(qb, dev), _dev(kb, dev), _dev(vb, dev)
        p = torch.tensor([pos], dtype=torch.int32, device=dev)
        scale = float(np.float16(1.0 / np.sqrt(d)))
        want = _reference_step(ct, dev, q, k, v, scale, p, bn, splits)
        got = torch.full((heads, group, d), float("nan"), dtype=torch.float16, device=dev)
        # the once-per-device-and-shape work (side library, scratch address, code objects) happens here, not in the call
        ct.fmha_decode_gqa_noalloc_prepare(q, k, v, ct.partition(got, [1, group, d]), p, splits, bn)
        torch.cuda.synchronize()
        before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
        ct.fmha_decode_gqa_noalloc(q, k, v, ct.partition(got, [1, group, d]), scale, p, splits, bn)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert torch.cuda.mem_get_info()[0] == free_before      # the driver's own count of free device memory: nothing was taken
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))        # bit for bit
        att_ref, lse_ref = oracle.fmha_decode_gqa_split(qb, kb, vb, scale, pos, bn, splits)
        out_ref = oracle.splitk_reduce_merge(att_ref, lse_ref, group)
        assert np.max(np.abs(got.float().cpu().numpy() - f32(out_ref))) <= 2e-2   # max-abs, as for the split + merge pair


@pytest.mark.gpu
def test_gpu_decode_noalloc_rejects_what_the_scratch_cannot_hold(ct, dev):
    heads, group, d, splits = 64, 16, 256, 64                  # 64 * 64 * 16 rows of 516 bytes = 32 MiB
    assert heads * splits * group * (d * 2 + 4) > ct.scratch_capacity()
    q = torch.zeros(heads, group, d, dtype=torch.float16, device=dev)
    kv = torch.zeros(heads, 64, d, dtype=torch.float16, device=dev)
    out = torch.zeros(heads, group, d, dtype=torch.float16, device=dev)
    p = torch.zeros(1, dtype=torch.int32, device=dev)
    with pytest.raises(ct.CutileError, match="device-resident scratch holds"):
        ct.fmha_decode_gqa_noalloc(q, kv, kv, ct.partition(out, [1, group, d]), 0.1, p, splits)


@pytest.mark.gpu
def test_gpu_decode_noalloc_captured_after_warm_up_and_replayed(ct, dev):
    """what the entry point is for: after the warm-up call it runs inside a stream capture, and every replay of the graph,
    with the program's own eager work between the replays, equals split + merge with caller memory bit for bit"""
    heads, group, d, max_seq, bn, splits = 4, 4, 128, 1024, 64, 8
    q, k, v = (_dev(normal_f16_bits(shape, seed), dev) for shape, seed in
               (((heads, group, d), 801), ((heads, max_seq, d), 802), ((heads, max_seq, d), 803)))
    p = torch.tensor([500], dtype=torch.int32, device=dev)
    scale = float(np.float16(1.0 / np.sqrt(d)))
    got = torch.full((heads, group, d), float("nan"), dtype=torch.float16, device=dev)
    gp = ct.partition(got, [1, group, d])
    ct.fmha_decode_gqa_noalloc_prepare(q, k, v, gp, p, splits, bn)
    torch.cuda.synchronize()
    graph = ct.CapturedGraph().capture(lambda stream: ct.fmha_decode_gqa_noalloc(q, k, v, gp, scale, p, splits, bn, stream=stream))
    try:
        for it in range(4):
            print(f"noalloc replay {it}", flush=True)
            q.copy_(_dev(normal_f16_bits((heads, group, d), 810 + it), dev))      # new inputs through the same buffers
            p.fill_(500 - 111 * it)
            got.fill_(float("nan"))
            torch.cuda.synchronize()
            graph.launch()
            graph.synchronize()
            want = _reference_step(ct, dev, q, k, v, scale, p, bn, splits)
            assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    finally:
        graph.close()
