"""Device random fills behind api::randn / api::rand (the reference binds cuRAND: cuda-core/src/api.rs:214-293,
cutile/src/api.rs:683-719).  The generator here is Philox4x32-10; cuRAND's value stream cannot be reproduced, so parity
with the reference's stream is unpinned and what is checked is (a) the generator against the published Random123
known-answer vectors, (b) the fill layout (an element depends on seed and stream position only), (c) the
distributions, and (d) the HIP kernels against the CPU restatement on the same (seed, offset)."""
import numpy as np
import pytest
import scipy.stats

import oracle


def test_philox4x32_10_known_answer_vectors():
    # Random123 kat_vectors, philox4x32 with 10 rounds: counter, key -> output
    kat = [
        ([0, 0, 0, 0], [0, 0], [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]),
        ([0xffffffff] * 4, [0xffffffff] * 2, [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]),
        ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0], [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]),
    ]
    for counter, key, want in kat:
        assert list(oracle.philox4x32_10(counter, key)) == want


def test_philox_rounds_follow_the_published_round_function():
    """ten rounds of (hi(M1 c2) ^ c1 ^ k0, lo(M1 c2), hi(M0 c0) ^ c3 ^ k1, lo(M0 c0)) with Weyl key steps, in plain Python"""
    def philox(c, k):
        c, k = list(c), list(k)
        for _ in range(10):
            p0, p1 = 0xD2511F53 * c[0], 0xCD9E8D57 * c[2]
            c = [(p1 >> 32) ^ c[1] ^ k[0], p1 & 0xffffffff, (p0 >> 32) ^ c[3] ^ k[1], p0 & 0xffffffff]
            k = [(k[0] + 0x9E3779B9) & 0xffffffff, (k[1] + 0xBB67AE85) & 0xffffffff]
        return c
    rng = np.random.default_rng(5)
    for _ in range(20):
        c, k = rng.integers(0, 2 ** 32, 4), rng.integers(0, 2 ** 32, 2)
        assert list(oracle.philox4x32_10(c, k)) == philox([int(x) for x in c], [int(x) for x in k])


def test_fill_layout_depends_on_seed_and_position_only():
    a = oracle.rng_fill(64, 11)
    # f32: four values per block, so a fill that starts three blocks in continues the same stream
    assert np.array_equal(a[12:], oracle.rng_fill(52, 11, offset=3))
    assert np.array_equal(a[:13], oracle.rng_fill(13, 11))                    # a ragged count is a prefix
    assert not np.array_equal(a, oracle.rng_fill(64, 12))
    d = oracle.rng_fill(64, 11, dtype=np.float64)
    assert np.array_equal(d[10:], oracle.rng_fill(54, 11, offset=5, dtype=np.float64))   # two values per block
    # word w of block b is exactly (philox(b, seed)[w] >> 8) * 2^-24
    blk = oracle.philox4x32_10([2, 0, 0, 0], [11, 0])
    assert np.array_equal(a[8:12], (blk >> 8).astype(np.float32) * np.float32(2.0 ** -24))
    # a 64-bit seed uses both key words, a position beyond 2^32 the second counter word
    blk = oracle.philox4x32_10([1, 1, 0, 0], [0x9abcdef0, 0x12345678])
    u = oracle.rng_fill(4, 0x123456789abcdef0, offset=(1 << 32) + 1)
    assert np.array_equal(u, (blk >> 8).astype(np.float32) * np.float32(2.0 ** -24))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_distributions_of_the_cpu_restatement(dtype):
    n = 1 << 20
    u = oracle.rng_fill(n, 3, dtype=dtype)
    assert u.min() >= 0.0 and u.max() < 1.0
    assert scipy.stats.kstest(u[: 1 << 17], "uniform").pvalue > 1e-3
    assert abs(u.mean() - 0.5) < 2e-3 and abs(u.var() - 1 / 12) < 1e-3
    z = oracle.rng_fill(n, 4, kind="normal", mean=-1.5, std=0.75, dtype=dtype)
    assert abs(z.mean() + 1.5) < 4e-3 and abs(z.std() - 0.75) < 3e-3
    s = (z[: 1 << 17].astype(np.float64) + 1.5) / 0.75
    assert scipy.stats.kstest(s, "norm").pvalue > 1e-3
    assert abs(scipy.stats.skew(s)) < 0.03 and abs(scipy.stats.kurtosis(s)) < 0.06
    # the two members of a Box-Muller pair are uncorrelated, and so are neighbouring pairs
    assert abs(np.corrcoef(s[0::2], s[1::2])[0, 1]) < 0.01 and abs(np.corrcoef(s[:-2:2], s[2::2])[0, 1]) < 0.01


# ---- HIP kernels through the C ABI ----------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "float64"])
def test_gpu_uniform_fill_is_the_restatement_bit_for_bit(ct, dev, dtype):
    import torch

    td, nd = getattr(torch, dtype), getattr(np, dtype)
    for n, seed in ((1 << 20, 0), (4099, 0xfeedface12345678), (1, 9), (7, 9)):
        rng = ct.Rng(seed)
        t = torch.full((n,), -1.0, dtype=td, device=dev)
        rng.uniform_(t)
        torch.cuda.synchronize()
        assert np.array_equal(t.cpu().numpy(), oracle.rng_fill(n, seed, dtype=nd)), (n, seed)
        rng.close()
    # a destination that is not 16-byte aligned, and neighbours left alone
    rng = ct.Rng(21)
    buf = torch.full((1030,), -1.0, dtype=td, device=dev)
    rng.uniform_(buf[1:1028])
    torch.cuda.synchronize()
    got = buf.cpu().numpy()
    assert got[0] == -1.0 and np.all(got[1028:] == -1.0) and np.array_equal(got[1:1028], oracle.rng_fill(1027, 21, dtype=nd))
    rng.close()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "float64"])
def test_gpu_normal_fill_matches_the_restatement_and_the_distribution(ct, dev, dtype):
    import torch

    td, nd = getattr(torch, dtype), getattr(np, dtype)
    n = 1 << 22
    rng = ct.Rng(1234)
    t = torch.empty(n, dtype=td, device=dev)
    rng.normal_(t, 2.0, 3.0)
    torch.cuda.synchronize()
    got = t.cpu().numpy()
    ref = oracle.rng_fill(n, 1234, kind="normal", mean=2.0, std=3.0, dtype=nd)
    # same uniforms on both sides; log / sqrt / sincos differ by a few ulps between the device and libm.
    # tolerance: 3 * 2^-20 relative to the largest sample for f32 (observed ~1e-6), 1e-12 for f64
    tol = 3.0 * 3.0 * 6.0 * (2.0 ** -20 if dtype == "float32" else 1e-13)
    assert np.max(np.abs(got - ref)) <= tol
    assert abs(got.mean() - 2.0) < 6e-3 and abs(got.std() - 3.0) < 5e-3
    assert scipy.stats.kstest((got[: 1 << 17].astype(np.float64) - 2.0) / 3.0, "norm").pvalue > 1e-3
    rng.close()


@pytest.mark.gpu
def test_gpu_stream_position_and_seed(ct, dev):
    import torch

    rng = ct.Rng(77)
    a, b = torch.empty(1000, device=dev), torch.empty(500, device=dev)
    rng.uniform_(a)
    assert rng.offset == 250
    rng.uniform_(b)                                     # continues where the first fill stopped
    torch.cuda.synchronize()
    whole = oracle.rng_fill(1500, 77)
    assert np.array_equal(a.cpu().numpy(), whole[:1000]) and np.array_equal(b.cpu().numpy(), whole[1000:])
    rng.set_seed(77)                                    # the same seed rewinds: the same values again
    assert rng.offset == 0
    c = torch.empty(1000, device=dev)
    rng.uniform_(c)
    torch.cuda.synchronize()
    assert torch.equal(a, c)
    rng.set_seed(78)
    rng.uniform_(c)
    torch.cuda.synchronize()
    assert not torch.equal(a, c)
    rng.offset = 1 << 33                                # far positions use the second counter word
    rng.uniform_(b)
    torch.cuda.synchronize()
    assert np.array_equal(b.cpu().numpy(), oracle.rng_fill(500, 78, offset=1 << 33))
    rng.close()
