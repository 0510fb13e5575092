"""The two benchmark programs with their own arithmetic (cutile-benchmarks/benches/rmsnorm.rs:20-66,
benches/softmax.rs:19-35): every operation an f16 operation.  RMSNorm has no transcendental step, so the device
result must equal the oracle's bit for bit; the softmax evaluates exp in f32 (hardware exp2 on the device, libm's exp
in the oracle) and rounds it to f16, so a few numerators sit one f16 step apart and the bar is 2 f16 steps."""
import numpy as np
import pytest
import torch

import oracle
from util import f16_ulp_diff, from_dev_f16_bits, normal_f16_bits, to_dev_f16


def _last(ct):
    import ctypes as C

    n = ct.lib().cutile_testing_launch_count()
    rec = ct.LaunchRecord()
    ct.check(ct.lib().cutile_testing_get_launch(n - 1, C.byref(rec)))
    return rec


def test_all_f16_launchers_choose_the_kernel_by_tile_width_and_validate(fake_hip):
    ct = fake_hip
    h = torch.half
    x, w, o = torch.zeros(10, 4096, dtype=h), torch.zeros(4096, dtype=h), torch.zeros(10, 4096, dtype=h)
    for block, sym in [(512, b"rms_norm_all_f16_entry__v8"), (1024, b"rms_norm_all_f16_entry__v16"), (64, b"rms_norm_all_f16_entry__v1"),
                       (16, b"rms_norm_all_f16_entry__v1"), (128, b"rms_norm_all_f16_entry__v2")]:
        ct.rms_norm_all_f16(x, w, ct.partition(o, [1, 4096]), 1e-5, generics=[4096, block])
        rec = _last(ct)
        assert rec.symbol == sym and tuple(rec.grid) == (3, 1, 1) and tuple(rec.block) == (256, 1, 1)     # 4 rows per workgroup
    for bn, sym, grid in [(4096, b"softmax_all_f16_entry__c8v8", 3), (512, b"softmax_all_f16_entry__c1v8", 20),
                          (256, b"softmax_all_f16_entry__c1v4", 40), (32, b"softmax_all_f16_entry__c1v1", 320)]:
        ct.softmax_all_f16(x, ct.partition(o, [1, bn]))
        rec = _last(ct)
        assert rec.symbol == sym and tuple(rec.grid) == (grid, 1, 1)
    n = ct.lib().cutile_testing_launch_count()
    bad = [
        (lambda: ct.rms_norm_all_f16(x, w, ct.partition(o, [1, 4096]), 1e-5, generics=[4096]), "BLOCK_SIZE"),
        (lambda: ct.rms_norm_all_f16(x, w, ct.partition(o, [1, 4096]), 1e-5, generics=[4096, 96]), "power of two"),
        (lambda: ct.rms_norm_all_f16(x, w, ct.partition(o, [1, 4096]), 1e-5, generics=[4096, 2048]), "at most 1024"),
        (lambda: ct.rms_norm_all_f16(x, w, ct.partition(o, [1, 4096]), 1e-5, generics=[2048, 512]), "generic N"),
        (lambda: ct.rms_norm_all_f16(x.float(), w, ct.partition(o, [1, 4096]), 1e-5, generics=[4096, 512]), "must be f16"),
        (lambda: ct.rms_norm_all_f16(x[:, ::2], w[::2], ct.partition(o[:, :2048], [1, 2048]), 1e-5, generics=[2048, 512]), "contiguous"),
        (lambda: ct.softmax_all_f16(x, ct.partition(o, [1, 96])), "power of two"),
        (lambda: ct.softmax_all_f16(torch.zeros(4, 32768, dtype=h), ct.partition(torch.zeros(4, 32768, dtype=h), [1, 32768])), "at most 16384"),
        (lambda: ct.softmax_all_f16(x.float(), ct.partition(o, [1, 512])), "must be f16"),
    ]
    for fn, msg in bad:
        with pytest.raises(ct.CutileError, match=msg):
            fn()
    assert ct.lib().cutile_testing_launch_count() == n


@pytest.mark.gpu
@pytest.mark.parametrize("m,n,block", [(64, 1024, 512), (37, 4096, 512), (16, 8192, 512), (9, 32768, 512),      # the benchmark's tile width
                                        (33, 2048, 1024), (20, 1024, 256), (12, 512, 128), (7, 256, 64), (5, 64, 16), (3, 8, 8)])
def test_gpu_rms_norm_all_f16_is_bit_exact(ct, dev, m, n, block):
    x = normal_f16_bits((m, n), 1201)
    w = normal_f16_bits((n,), 1202)
    out = torch.zeros(m, n, dtype=torch.half, device=dev)
    ct.rms_norm_all_f16(to_dev_f16(x, dev), to_dev_f16(w, dev), ct.partition(out, [1, n]), 1e-5, generics=[n, block])
    torch.cuda.synchronize()
    ref = oracle.rms_norm_all_f16(x, w, 1e-5, block)
    assert np.array_equal(from_dev_f16_bits(out), ref)


@pytest.mark.gpu
def test_gpu_rms_norm_all_f16_overflowing_sum_and_row_subset(ct, dev):
    # 17.5^2 * 2048 overflows the f16 sum: inf -> 1 / inf = 0 -> zeros, exactly as the f16 arithmetic says
    x = np.full((4, 2048), 17.5, np.float16).view(np.uint16)
    w = np.ones(2048, np.float16).view(np.uint16)
    out = torch.full((4, 2048), 7.0, dtype=torch.half, device=dev)
    ct.rms_norm_all_f16(to_dev_f16(x, dev), to_dev_f16(w, dev), ct.partition(out, [1, 2048]), 1e-5, generics=[2048, 512])
    torch.cuda.synchronize()
    assert np.array_equal(from_dev_f16_bits(out), oracle.rms_norm_all_f16(x, w, 1e-5, 512)) and torch.all(out == 0)
    # a prefix launch over the first 3 rows leaves the rest alone
    xs = normal_f16_bits((8, 1024), 1203)
    ws = normal_f16_bits((1024,), 1204)
    out = torch.full((8, 1024), 7.0, dtype=torch.half, device=dev)
    ct.rms_norm_all_f16(to_dev_f16(xs, dev), to_dev_f16(ws, dev), ct.partition(out, [1, 1024], prefix=True), 1e-5, generics=[1024, 512],
                        grid=(3, 1, 1))
    torch.cuda.synchronize()
    got = from_dev_f16_bits(out)
    assert np.array_equal(got[:3], oracle.rms_norm_all_f16(xs, ws, 1e-5, 512)[:3]) and torch.all(out[3:] == 7.0)


@pytest.mark.gpu
@pytest.mark.parametrize("m,n,bm,bn", [(64, 1024, 1, 1024), (33, 4096, 1, 4096), (16, 8192, 1, 8192), (5, 16384, 1, 16384),
                                       (24, 4096, 4, 1024), (16, 2048, 2, 256), (8, 512, 1, 64), (6, 256, 2, 32), (4, 128, 1, 8),
                                       (9, 1000, 1, 256), (3, 100, 1, 64), (7, 520, 4, 512)])
def test_gpu_softmax_all_f16(ct, dev, m, n, bm, bn):
    x = oracle.f32_to_f16_bits(oracle.normal_f32((m, n), 1211, 0, 2.0))
    y = torch.zeros(m, n, dtype=torch.half, device=dev)
    ct.softmax_all_f16(to_dev_f16(x, dev), ct.partition(y, [bm, bn]), generics=[bm, bn])
    torch.cuda.synchronize()
    got = from_dev_f16_bits(y)
    ref = oracle.softmax_all_f16(x, bm, bn)
    d = f16_ulp_diff(got, ref)
    assert d.max() <= 2 and (d > 0).mean() <= 0.10, (int(d.max()), float((d > 0).mean()))
    # and the segments are distributions: each sums to 1 within the f16 arithmetic's own error
    g = got.view(np.float16).astype(np.float64)
    tiles = -(-n // bn)
    pad = np.zeros((m, tiles * bn))
    pad[:, :n] = g
    sums = pad.reshape(m, tiles, bn).sum(2)
    full = np.ones((m, tiles), bool)
    if n % bn:
        full[:, -1] = False                   # a ragged last tile shares its denominator with the zero padding
    assert np.abs(sums[full] - 1.0).max() <= 2e-2
