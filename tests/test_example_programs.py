"""GPU parity tests of the small kernels of the reference's example programs — relu and matvec
(cutile-examples/examples/async_mlp.rs), dropout (dropout.rs), scale_ptr (scale_ptr.rs), batch_matmul
(batch_matmul.rs) — through the C ABI against the CPU oracle.  relu, dropout and scale_ptr are bit exact;
matvec and the f32 batch_matmul are sums of f32 products in an order the tile program leaves open: each output
within 1e-5 of the sum of the magnitudes of its products; the 16-bit batch_matmul to the GEMM's bar (rel-L2 <= 1e-2,
and every element within one unit in the last place of the output type plus the accumulation slack)."""
import numpy as np
import pytest
import torch

import oracle
from util import assert_rounded_close, from_dev_bf16_bits, from_dev_f16_bits, normal_bf16_bits, normal_f16_bits, rel_l2, to_dev_bf16, to_dev_f16

pytestmark = pytest.mark.gpu


def sync():
    torch.cuda.synchronize()


# ---- relu -------------------------------------------------------------------------------------
@pytest.mark.parametrize("n,tile", [(16, 4), (1 << 20, 1024), (1000003, 128), (5, 8)])
def test_relu_in_place_bit_exact(ct, dev, n, tile):
    x = oracle.normal_f32(n, 401)
    x[::7] = -0.0
    xd = torch.from_numpy(x.copy()).to(dev)
    ct.relu(ct.partition(xd, [tile]), generics=[tile])
    sync()
    got = xd.cpu().numpy()
    assert np.array_equal(got, oracle.relu_f32(x))
    assert not np.signbit(got).any()          # max(0, -0) and max(0, negative) are +0


def test_relu_on_a_strided_view_and_a_prefix_grid(ct, dev):
    base = torch.from_numpy(oracle.normal_f32(4096, 402)).to(dev)
    want = base.clone()
    view = base[1::2]                          # stride 2, not 16-byte aligned
    ct.relu(ct.partition(view, [64]))
    sync()
    want[1::2] = torch.clamp_min(want[1::2], 0.0)
    assert torch.equal(base, want)
    t = torch.from_numpy(oracle.normal_f32(1000, 403)).to(dev)
    want = t.clone()
    ct.relu(ct.partition(t, [100], prefix=True), grid=(3, 1, 1))
    sync()
    want[:300] = torch.clamp_min(want[:300], 0.0)
    assert torch.equal(t, want)                # elements past the third tile are untouched


# ---- dropout ----------------------------------------------------------------------------------
def test_dropout_example_shape(ct, dev):
    # cutile-examples/examples/dropout.rs:39-50: m = 16, tiles of 4, p = 0.4, x_keep uniform in [0, 1)
    keep = oracle.uniform_f32(16, 411, 0.0, 1.0)
    keep[3] = np.float32(0.4)                  # exactly p: not kept (strictly greater)
    out = torch.zeros(16, device=dev)
    x = torch.from_numpy(oracle.normal_f32(16, 412)).to(dev)
    ct.dropout(0.4, x, torch.from_numpy(keep).to(dev), ct.partition(out, [4]), generics=[4])
    sync()
    got = out.cpu().numpy()
    assert np.array_equal(got, oracle.dropout_f32(0.4, keep))
    assert got[3] == 0.0
    assert np.array_equal(got != 0, keep > np.float32(0.4))


@pytest.mark.parametrize("n,n_keep,tile,p", [(1 << 20, 1 << 20, 1024, 0.1), (1000003, 900001, 128, 0.5), (37, 64, 8, 0.0)])
def test_dropout_bit_exact_with_a_shorter_keep_tensor(ct, dev, n, n_keep, tile, p):
    keep = oracle.uniform_f32(n_keep, 413, 0.0, 1.0)
    out = torch.full((n,), 7.0, device=dev)
    x = torch.zeros(1, device=dev)             # never read
    ct.dropout(p, x, torch.from_numpy(keep).to(dev), ct.partition(out, [tile]))
    sync()
    assert np.array_equal(out.cpu().numpy(), oracle.dropout_f32(p, keep, n))


# ---- scale_ptr ----------------------------------------------------------------------------------
@pytest.mark.parametrize("grid", [(4, 1, 1), (1, 1, 1), (1000, 1, 1)])
def test_scale_ptr_reference_program(ct, dev, grid):
    # cutile-examples/examples/scale_ptr.rs:86-110: arange(1024) * 3 with 4 blocks striding over the data
    x = torch.arange(1024, dtype=torch.float32, device=dev)
    out = torch.zeros(1024, device=dev)
    ct.scale_ptr(out.data_ptr(), x.data_ptr(), 3.0, 1024, grid=grid)
    sync()
    assert torch.equal(out, x * 3.0)


@pytest.mark.parametrize("n,offset", [(1 << 20, 0), (1000003, 1), (5, 3), (0, 0)])
def test_scale_ptr_lengths_and_unaligned_pointers(ct, dev, n, offset):
    x = oracle.normal_f32(n + offset + 8, 421)
    xd = torch.from_numpy(x).to(dev)
    out = torch.full((n + offset + 8,), -1.0, device=dev)
    ct.scale_ptr(out.data_ptr() + 4 * offset, xd.data_ptr() + 4 * offset, 0.37, n, grid=(8, 1, 1))
    sync()
    got = out.cpu().numpy()
    assert np.array_equal(got[offset:offset + n], oracle.scale_f32(x[offset:offset + n], 0.37))
    assert (got[:offset] == -1.0).all() and (got[offset + n:] == -1.0).all()


def test_scale_ptr_needs_a_grid(ct, dev):
    x = torch.zeros(128, device=dev)
    with pytest.raises(ct.CutileError, match="Launch grid required."):
        ct.scale_ptr(x.data_ptr(), x.data_ptr(), 2.0, 128)


# ---- matvec -------------------------------------------------------------------------------------
def _mag_matvec(x, y, kt):
    return np.abs(x[:, :kt].astype(np.float64)) @ np.abs(y[:kt].astype(np.float64))


@pytest.mark.parametrize("m,k,bm,bk", [(16, 16, 4, 4), (4096, 4096, 64, 64), (1000, 777, 8, 1), (33, 8200, 16, 100)])
def test_matvec_accumulates_onto_z(ct, dev, m, k, bm, bk):
    x, y, z = oracle.normal_f32((m, k), 431), oracle.normal_f32(k, 432), oracle.normal_f32(m, 433)
    zd = torch.from_numpy(z.copy()).to(dev)
    ct.matvec(ct.partition(zd, [bm]), torch.from_numpy(x).to(dev), torch.from_numpy(y).to(dev), k, generics=[bm, bk, k])
    sync()
    kt = (k // bk) * bk
    want = oracle.matvec_f32(z, x, y, k, bk)
    err = np.abs(zd.cpu().numpy().astype(np.float64) - want)
    assert (err <= 1e-5 * (_mag_matvec(x, y, kt) + np.abs(z))).all(), err.max()


def test_matvec_strided_operands_and_rows_x_does_not_have(ct, dev):
    m, k = 70, 300
    xb = oracle.normal_f32((k, 64), 434)       # x = transposed view: unit stride along rows, not along K
    y2 = oracle.normal_f32(2 * k, 435)
    z = np.zeros(m, np.float32)
    zd = torch.from_numpy(z.copy()).to(dev)
    xd = torch.from_numpy(xb).to(dev).t()      # [64, k]: rows 64..69 of z see no x row -> unchanged
    yd = torch.from_numpy(y2).to(dev)[::2]
    ct.matvec(ct.partition(zd, [7]), xd, yd, k)
    sync()
    want = np.zeros(m, np.float32)
    want[:64] = oracle.matvec_f32(z[:64], xb.T.copy(), y2[::2].copy(), k)
    err = np.abs(zd.cpu().numpy().astype(np.float64) - want)
    assert (err[:64] <= 1e-5 * _mag_matvec(xb.T, y2[::2], k)).all() and (zd.cpu().numpy()[64:] == 0).all()


def test_async_mlp_chain(ct, dev):
    # cutile-examples/examples/async_mlp.rs:124-137: gemm(data, w0) -> matvec(., w1) -> relu, dim 16, tiles of 4
    dim, bd = 16, 4
    data, w0, w1 = oracle.normal_f32((dim, dim), 441), oracle.normal_f32((dim, dim), 442), oracle.normal_f32(dim, 443)
    out0 = torch.zeros(dim, dim, device=dev)
    ct.gemm(ct.partition(out0, [bd, bd]), torch.from_numpy(data).to(dev), torch.from_numpy(w0).to(dev), dim, generics=["f32", bd, bd, bd])
    out1 = torch.zeros(dim, device=dev)
    ct.matvec(ct.partition(out1, [bd]), out0, torch.from_numpy(w1).to(dev), dim, generics=[bd, bd, dim])
    ct.relu(ct.partition(out1, [bd]), generics=[bd])
    sync()
    h = oracle.cpu_gemm_f32(data, w0)
    want = oracle.relu_f32(oracle.matvec_f32(np.zeros(dim, np.float32), h, w1))
    assert np.allclose(out1.cpu().numpy(), want, rtol=1e-4, atol=1e-4)


# ---- batch_matmul -------------------------------------------------------------------------------
def test_batch_matmul_reference_program(ct, dev):
    # cutile-examples/examples/batch_matmul.rs:49-76: ones [4,128,64] x ones [4,64,256], tiles (64, 64, 32): every output = K
    batch, m, n, k = 4, 128, 256, 64
    a, b = torch.ones(batch, m, k, device=dev), torch.ones(batch, k, n, device=dev)
    c = torch.zeros(batch, m, n, device=dev)
    ct.batch_matmul(ct.partition(c, [1, 64, 64]), a, b, k, generics=["f32", 64, 64, 32, k])
    sync()
    assert torch.equal(c, torch.full_like(c, float(k)))
    assert ct.last_resolved()["variant"] == "f32_generic"


@pytest.mark.parametrize("batch,m,n,k,bm,bn,bk", [(3, 100, 90, 72, 32, 16, 8), (2, 64, 64, 50, 64, 64, 16), (5, 17, 129, 33, 8, 8, 1)])
def test_batch_matmul_f32_ragged(ct, dev, batch, m, n, k, bm, bn, bk):
    a, b = oracle.normal_f32((batch, m, k), 451), oracle.normal_f32((batch, k, n), 452)
    c = torch.full((batch, m, n), 3.0, device=dev)      # overwritten: accumulators start at zero
    ct.batch_matmul(ct.partition(c, [1, bm, bn]), torch.from_numpy(a).to(dev), torch.from_numpy(b).to(dev), k, generics=["f32", bm, bn, bk, k])
    sync()
    kt = (k // bk) * bk
    want = oracle.batch_matmul_f32(a, b, k, bk)
    mag = np.einsum("bmk,bkn->bmn", np.abs(a[:, :, :kt]).astype(np.float64), np.abs(b[:, :kt, :]).astype(np.float64))
    err = np.abs(c.cpu().numpy().astype(np.float64) - want)
    assert (err <= 1e-5 * mag + 1e-30).all(), err.max()


@pytest.mark.parametrize("dtype,tile,variant", [("bf16", 256, "bf16_256x256x64_q2x4"), ("bf16", 256, "bf16_256x256x64_r2x4"), ("bf16", 256, "bf16_256x256x64_d2x4"),
                                                ("bf16", 128, "bf16_128x128x64_d2x2"), ("f16", 256, "f16_256x256x64_q2x4"), ("f16", 256, "f16_256x256x64_r2x4"),
                                                ("f16", 256, "f16_256x256x64_d4x2"), ("f16", 128, "f16_128x128x64_d2x2"),
                                                ("bf16", 128, "bf16_generic"), ("f16", 64, "f16_generic")])
def test_batch_matmul_16_bit_against_the_gemm_oracle(ct, dev, dtype, tile, variant):
    batch, m, n, k = 3, 384, 512, 256
    mk = normal_bf16_bits if dtype == "bf16" else normal_f16_bits
    to_dev = to_dev_bf16 if dtype == "bf16" else to_dev_f16
    from_bits = from_dev_bf16_bits if dtype == "bf16" else from_dev_f16_bits
    to_f32 = oracle.bf16_bits_to_f32 if dtype == "bf16" else oracle.f16_bits_to_f32
    a_bits, b_bits = mk((batch, m, k), 461, 1.0), mk((batch, k, n), 462, k ** -0.5)
    c = torch.full((batch, m, n), 5.0, device=dev).to(torch.bfloat16 if dtype == "bf16" else torch.half)
    ct.batch_matmul(ct.partition(c, [1, tile, tile]), to_dev(a_bits, dev), to_dev(b_bits, dev), k, generics=[dtype, tile, tile, 64, k], variant=variant)
    sync()
    assert ct.last_resolved()["variant"] == variant
    a, b = to_f32(a_bits), to_f32(b_bits)
    want = oracle.batch_matmul_f32(a, b)
    got = to_f32(from_bits(c))
    assert rel_l2(got, want) <= 1e-2
    mag = np.einsum("bmk,bkn->bmn", np.abs(a).astype(np.float64), np.abs(b).astype(np.float64))
    for i in range(batch):
        assert_rounded_close(got[i], want[i], (tile, tile), rel_ulp=2.0 ** -7 if dtype == "bf16" else 2.0 ** -10, what=f"batch {i}", mag=mag[i])


def test_batch_matmul_default_variants(ct, dev):
    # the ring on 16 x 16 x 32 whatever K is (it masks a ragged last K tile)
    for k, want in ((128, "bf16_256x256x64_q2x4"), (96, "bf16_256x256x64_q2x4")):
        a_bits, b_bits = normal_bf16_bits((2, 256, k), 465), normal_bf16_bits((2, k, 256), 466, k ** -0.5)
        c = torch.zeros(2, 256, 256, device=dev, dtype=torch.bfloat16)
        ct.batch_matmul(ct.partition(c, [1, 256, 256]), to_dev_bf16(a_bits, dev), to_dev_bf16(b_bits, dev), k, generics=["bf16", 256, 256, 32, k])
        sync()
        assert ct.last_resolved()["variant"] == want
        ref = oracle.batch_matmul_f32(oracle.bf16_bits_to_f32(a_bits), oracle.bf16_bits_to_f32(b_bits))
        assert rel_l2(oracle.bf16_bits_to_f32(from_dev_bf16_bits(c)), ref) <= 1e-2


def test_batch_matmul_batches_are_independent_and_strided(ct, dev):
    # batch stride larger than one matrix (a view into a wider allocation), batches distinguishable
    batch, m, n, k = 4, 256, 256, 128
    a_bits, b_bits = normal_bf16_bits((batch, 2, m, k), 471), normal_bf16_bits((batch, k, n), 472, k ** -0.5)
    ad = to_dev_bf16(a_bits, dev)[:, 1]          # [batch, m, k] with batch stride 2 * m * k
    c = torch.zeros(batch, m, n, device=dev, dtype=torch.bfloat16)
    ct.batch_matmul(ct.partition(c, [1, 128, 128]), ad, to_dev_bf16(b_bits, dev), k)
    sync()
    assert ct.last_resolved()["variant"] == "bf16_128x128x64_d2x2"
    want = oracle.batch_matmul_f32(oracle.bf16_bits_to_f32(a_bits[:, 1]), oracle.bf16_bits_to_f32(b_bits))
    assert rel_l2(oracle.bf16_bits_to_f32(from_dev_bf16_bits(c)), want) <= 1e-2
    for i in range(batch):
        assert rel_l2(oracle.bf16_bits_to_f32(from_dev_bf16_bits(c[i])), want[i]) <= 1e-2


def test_batch_matmul_prefix_grid_and_missing_batches(ct, dev):
    # a has fewer batches than c: the missing ones read as zeros; a prefix grid leaves the rest of c alone
    batch, m, n, k = 4, 128, 128, 64
    a_bits, b_bits = normal_f16_bits((2, m, k), 481), normal_f16_bits((batch, k, n), 482, k ** -0.5)
    c = torch.full((batch, m, n), 9.0, device=dev, dtype=torch.half)
    ct.batch_matmul(ct.partition(c, [1, 128, 128], prefix=True), to_dev_f16(a_bits, dev), to_dev_f16(b_bits, dev), k, grid=(3, 1, 1))
    sync()
    assert ct.last_resolved()["variant"] == "f16_generic"
    want = oracle.batch_matmul_f32(oracle.f16_bits_to_f32(a_bits), oracle.f16_bits_to_f32(b_bits[:2]))
    got = oracle.f16_bits_to_f32(from_dev_f16_bits(c))
    assert rel_l2(got[:2], want) <= 1e-2
    assert (got[2] == 0).all() and (got[3] == 9.0).all()


def test_batch_matmul_rejects_what_the_tile_program_would(ct, dev):
    a, b = torch.ones(2, 64, 32, device=dev), torch.ones(2, 32, 64, device=dev)
    c = torch.zeros(2, 64, 64, device=dev)
    with pytest.raises(ct.CutileError, match=r"partitioned \[1, BM, BN\]"):
        ct.batch_matmul(ct.partition(c, [2, 32, 32]), a, b, 32)
    with pytest.raises(ct.CutileError, match="generic K"):
        ct.batch_matmul(ct.partition(c, [1, 32, 32]), a, b, 32, generics=["f32", 32, 32, 8, 64])
    with pytest.raises(ct.CutileError, match="share one element type"):
        ct.batch_matmul(ct.partition(c, [1, 32, 32]), a.half(), b, 32)
