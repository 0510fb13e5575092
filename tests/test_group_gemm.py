"""f16 operands on the pipelined GEMM kernels, and the grouped GEMM over descriptor tables
(cutile-kernels/src/experimental/moe.rs:67-128): C_g = A_g . B_g per group, f16 with f32 accumulation, NUM_SM
persistent tile blocks over the tiles of all groups.

The oracle is cpu_gemm (cutile-examples/examples/persistent_gemm.rs:140-152, pinned elsewhere) on the f16-decoded
operands, rounded to f16 like the kernel's store; tolerance rel-L2 <= 1e-2 as for the bf16 GEMM (observed ~3e-4:
f16 rounding of the output), products with the identity bit-exact."""
import numpy as np
import pytest
import torch

import oracle
from util import rel_l2

f16b = lambda a: oracle.f32_to_f16_bits(np.asarray(a, np.float32))
f16v = lambda bits: oracle.f16_bits_to_f32(bits)


def _dev16(bits, dev):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(dev).view(torch.half)


def _tables(tensors, dev):
    ptrs = torch.tensor([t.data_ptr() for t in tensors], dtype=torch.int64, device=dev)
    metas = torch.zeros(len(tensors), 8, dtype=torch.int32)
    for i, t in enumerate(tensors):
        metas[i, 0], metas[i, 1], metas[i, 2] = t.shape[0], t.shape[1], t.stride(0)
    return ptrs, metas.to(dev)


# ---- launcher on the recording runtime (CPU) ----------------------------------------------------
def test_group_gemm_launcher_takes_its_grid_from_num_sm(fake_hip):
    ct = fake_hip
    from test_host_abi import _last
    ptrs = torch.zeros(4, dtype=torch.int64)
    metas = torch.zeros(4, 8, dtype=torch.int32)
    ct.group_gemm_f16_nt_desc(ptrs, ptrs, ptrs, metas, metas, metas, 4, generics=[128, 128, 64, 96])
    rec, _ = _last(ct)
    assert rec.symbol == b"group_gemm_nt_desc_entry__f16_128x128x64_d2x2" and tuple(rec.grid) == (96, 1, 1) and tuple(rec.block) == (256, 1, 1)
    ct.group_gemm_f16_nt_desc(ptrs, ptrs, ptrs, metas, metas, metas, 3, generics=[256, 256, 64], grid=(40, 1, 1))
    rec, _ = _last(ct)
    assert rec.symbol == b"group_gemm_nt_desc_entry__f16_256x256x64_q2x4" and tuple(rec.grid) == (40, 1, 1) and tuple(rec.block) == (512, 1, 1)
    n0 = ct.lib().cutile_testing_launch_count()
    cases = [
        (lambda: ct.group_gemm_f16_nt_desc(ptrs, ptrs, ptrs, metas, metas, metas, 4), "Launch grid required"),
        (lambda: ct.group_gemm_f16_nt_desc(ptrs, ptrs, ptrs, metas, metas, metas, 4, generics=[128, 128, 64, 96], grid=(64, 1, 1)), "must equal NUM_SM"),
        (lambda: ct.group_gemm_f16_nt_desc(ptrs, ptrs, ptrs, metas, metas, metas, 5, generics=[128, 128, 64, 8]), "at least 5 entries"),
        (lambda: ct.group_gemm_f16_nt_desc(ptrs, ptrs, ptrs, metas[:, :4], metas, metas, 4, generics=[128, 128, 64, 8]), "i32 tensor"),
        (lambda: ct.group_gemm_f16_nt_desc(ptrs.int(), ptrs, ptrs, metas, metas, metas, 4, generics=[128, 128, 64, 8]), "i64 tensor"),
        (lambda: ct.group_gemm_f16_nt_desc(ptrs, ptrs, ptrs, metas, metas, metas, 4, generics=[64, 64, 64, 8]), "no precompiled variant"),
    ]
    for fn, msg in cases:
        with pytest.raises(ct.CutileError, match=msg):
            fn()
    assert ct.lib().cutile_testing_launch_count() == n0
    # f16 operands now pick a pipelined kernel of their own
    z = torch.zeros(512, 512, dtype=torch.half)
    a = torch.zeros(512, 256, dtype=torch.half)
    b = torch.zeros(256, 512, dtype=torch.half)
    ct.gemm(ct.partition(z, [256, 256]), a, b, 256, accumulate=False)
    assert _last(ct)[0].symbol == b"gemm_entry__f16_256x256x64_d4x2"
    ct.gemm_persistent(ct.mapped(ct.partition(z, [128, 128]), [4, 1], 7), a, b)
    assert _last(ct)[0].symbol == b"gemm_persistent_entry__f16_128x128x64_d2x2"


# ---- HIP kernels (GPU) --------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("m,n,k,tile,accumulate", [(512, 768, 1024, 256, False), (300, 264, 192, 256, True), (128, 128, 64, 128, False),
                                                   (1000, 520, 320, 128, True)])
def test_gpu_gemm_f16(ct, dev, m, n, k, tile, accumulate):
    ab, bb = f16b(oracle.normal_f32((m, k), 861, 0, k ** -0.5)), f16b(oracle.normal_f32((k, n), 862, 0, k ** -0.5))
    z0 = f16b(oracle.normal_f32((m, n), 863))
    z = _dev16(z0, dev).clone()
    ct.gemm(ct.partition(z, [tile, tile]), _dev16(ab, dev), _dev16(bb, dev), k, accumulate=accumulate)
    torch.cuda.synchronize()
    ref = oracle.cpu_gemm_f32(f16v(ab), f16v(bb)) + (f16v(z0) if accumulate else 0.0)
    assert rel_l2(z.float().cpu().numpy(), ref) <= 1e-2
    eye = torch.eye(k, n, dtype=torch.half, device=dev)
    zi = torch.zeros(m, n, dtype=torch.half, device=dev)
    ct.gemm(ct.partition(zi, [tile, tile]), _dev16(ab, dev), eye, k, accumulate=False)
    torch.cuda.synchronize()
    w = min(k, n)
    assert torch.equal(zi[:, :w], _dev16(ab, dev)[:, :w]) and not zi[:, w:].any()      # A . I = A, bit for bit
    zm = torch.zeros(m, n, dtype=torch.half, device=dev)
    blocks = min(5, ct.partition(zm, [tile, tile]).grid()[0] * ct.partition(zm, [tile, tile]).grid()[1])
    ct.gemm_persistent(ct.mapped(ct.partition(zm, [tile, tile]), [2, 1], blocks), _dev16(ab, dev), _dev16(bb, dev))
    torch.cuda.synchronize()
    assert rel_l2(zm.float().cpu().numpy(), oracle.cpu_gemm_f32(f16v(ab), f16v(bb))) <= 1e-2


@pytest.mark.gpu
@pytest.mark.parametrize("variant", ["f16_256x256x64_q2x4", "f16_256x256x64_r4x2", "f16_256x256x64_r2x4", "f16_256x256x64_d4x2"])
@pytest.mark.parametrize("m,n,k,accumulate", [(512, 768, 1024, False), (300, 264, 448, True), (256, 256, 64, False)])
def test_gpu_gemm_f16_pipelined_variants(ct, dev, variant, m, n, k, accumulate):
    """every f16 variant of the 256 x 256 tile, the ring-pipelined ones included (whole K tiles), against cpu_gemm"""
    ab, bb = f16b(oracle.normal_f32((m, k), 864, 0, k ** -0.5)), f16b(oracle.normal_f32((k, n), 865, 0, k ** -0.5))
    z0 = f16b(oracle.normal_f32((m, n), 866))
    z = _dev16(z0, dev).clone()
    ct.gemm(ct.partition(z, [256, 256]), _dev16(ab, dev), _dev16(bb, dev), k, accumulate=accumulate, variant=variant)
    torch.cuda.synchronize()
    ref = oracle.cpu_gemm_f32(f16v(ab), f16v(bb)) + (f16v(z0) if accumulate else 0.0)
    assert rel_l2(z.float().cpu().numpy(), ref) <= 1e-2
    eye = torch.eye(k, n, dtype=torch.half, device=dev)
    zi = torch.zeros(m, n, dtype=torch.half, device=dev)
    ct.gemm(ct.partition(zi, [256, 256]), _dev16(ab, dev), eye, k, accumulate=False, variant=variant)
    torch.cuda.synchronize()
    w = min(k, n)
    assert torch.equal(zi[:, :w], _dev16(ab, dev)[:, :w]) and not zi[:, w:].any()


@pytest.mark.gpu
@pytest.mark.parametrize("tile,num_sm", [(128, 8), (128, 256), (256, 3), (256, 64)])
def test_gpu_group_gemm_desc(ct, dev, tile, num_sm):
    shapes = [(128, 256, 64), (48, 16, 32), (0, 64, 64), (400, 272, 192), (16, 528, 16), (256, 256, 256)]   # (m, n, k)
    a_t, b_t, c_t, refs = [], [], [], []
    for i, (m, n, k) in enumerate(shapes):
        ab, bb = f16b(oracle.normal_f32((max(m, 1), k), 871 + i, 0, k ** -0.5)), f16b(oracle.normal_f32((k, n), 881 + i, 0, k ** -0.5))
        a_t.append(_dev16(ab, dev)[:m])
        # B_3 is a column slice of a wider matrix: its row stride differs from its width
        b_full = _dev16(np.concatenate([bb, bb], axis=1), dev) if i == 3 else _dev16(bb, dev)
        b_t.append(b_full[:, :n])
        c_t.append(torch.full((m, n), float("nan"), dtype=torch.half, device=dev))
        refs.append(oracle.cpu_gemm_f32(f16v(ab[:m]), f16v(bb)) if m else np.zeros((0, n), np.float32))
    ap, am = _tables(a_t, dev)
    bp, bmeta = _tables(b_t, dev)
    cp, cm = _tables(c_t, dev)
    ct.group_gemm_f16_nt_desc(ap, bp, cp, am, bmeta, cm, len(shapes), generics=[tile, tile, 64, num_sm])
    torch.cuda.synchronize()
    for c, ref in zip(c_t, refs):
        got = c.float().cpu().numpy()
        assert np.all(np.isfinite(got))
        if ref.size:
            assert rel_l2(got, ref) <= 1e-2
    # fewer groups than table rows: the rest stays untouched
    for c in c_t:
        c.fill_(5.0)
    ct.group_gemm_f16_nt_desc(ap, bp, cp, am, bmeta, cm, 2, generics=[tile, tile, 64, num_sm])
    torch.cuda.synchronize()
    assert rel_l2(c_t[1].float().cpu().numpy(), refs[1]) <= 1e-2 and torch.all(c_t[3] == 5.0) and torch.all(c_t[5] == 5.0)
