"""Greedy sampling and row gathers of cutile-kernels: argmax_blocks_f16, lm_head_argmax_blocks_f16,
argmax_reduce_blocks_to_u32 (src/argmax.rs:21-71, 88-158, 173-213), embedding_batch_f16 (src/embeddings.rs:21-41)
and gather_row_f16 (src/pointwise.rs:86-99).

CPU: the oracle pinned by numpy.argmax (first index of the maximum), the composition blocks -> reduce, a float64
matrix-vector product and numpy indexing.  GPU: indices and gathered bits exact; the fused LM head sums its f32
products in another order than the tile program, so its block maxima agree to 1e-4 relative and its indices
wherever the two best logits of a block are further apart than that."""
import numpy as np
import pytest
import torch

import oracle

f16b = lambda a: oracle.f32_to_f16_bits(np.asarray(a, np.float32))
f16v = lambda bits: oracle.f16_bits_to_f32(bits)


# ---- oracle (CPU) ---------------------------------------------------------------------------
def test_oracle_argmax_blocks_and_reduce_compose_to_numpy_argmax():
    n, bs = 5000, 512
    for seed, length in ((801, 5000), (802, 4321), (803, 513), (804, 1)):
        bits = f16b(oracle.normal_f32(n, seed))
        vals = f16v(bits)
        bm, bi = oracle.argmax_blocks_f16(bits, bs, length)
        for b in range(len(bm)):
            lo, hi = b * bs, min((b + 1) * bs, length)
            if lo < hi:
                assert bm[b] == vals[lo:hi].max() and bi[b] == lo + int(np.argmax(vals[lo:hi]))
            else:                                      # nothing valid: the masked value at the block's first position
                assert bm[b] == np.float32(-1e30) and bi[b] == lo
        used = -(-length // bs)
        assert oracle.argmax_reduce_blocks_to_u32(bm, bi, used) == int(np.argmax(vals[:length]))
    # ties go to the smallest index, inside a block and across blocks
    bits = f16b(np.zeros(2048))
    bits[[700, 300, 1900]] = f16b([5.0])[0]
    bm, bi = oracle.argmax_blocks_f16(bits, 1024, 2048)
    assert list(bi) == [300, 1900] and oracle.argmax_reduce_blocks_to_u32(bm, bi, 2) == 300
    # a logits tile that runs past the tensor reads zeros there; they count while index < len (argmax.rs:30-43)
    neg = f16b(np.full(100, -3.0))
    bm, bi = oracle.argmax_blocks_f16(neg, 128, 120)
    assert bm[0] == 0.0 and bi[0] == 100


def test_oracle_lm_head_is_a_matrix_vector_product_then_argmax():
    rows, k = 1000, 256
    w, h = f16b(oracle.normal_f32((rows, k), 811)), f16b(oracle.normal_f32(k, 812))
    logits = f16v(w).astype(np.float64) @ f16v(h).astype(np.float64)
    bm, bi = oracle.lm_head_argmax_blocks_f16(w, h, 990)
    assert len(bm) == 16
    for b in range(16):
        lo, hi = b * 64, min((b + 1) * 64, 990)
        assert bi[b] == lo + int(np.argmax(logits[lo:hi])) and abs(bm[b] - logits[lo:hi].max()) < 1e-4
    assert oracle.argmax_reduce_blocks_to_u32(bm, bi, 16) == int(np.argmax(logits[:990]))


def test_oracle_gathers_are_numpy_indexing():
    table = f16b(oracle.normal_f32((50, 24), 821))
    ids = np.array([3, 49, 0, 3, 77], np.uint32)
    out = oracle.embedding_batch_f16(ids, table)
    assert np.array_equal(out[:4], table[[3, 49, 0, 3]]) and not out[4].any()
    assert np.array_equal(oracle.gather_row_f16(table, 17), table[17])
    assert np.array_equal(oracle.gather_row_f16(table, 17, 30)[:24], table[17]) and not oracle.gather_row_f16(table, 17, 30)[24:].any()


# ---- launchers on the recording runtime (CPU) ---------------------------------------------------
def test_sampling_launchers_validate_before_any_launch(fake_hip):
    ct = fake_hip
    from test_host_abi import _last
    h = torch.half
    logits = torch.zeros(5000, dtype=h)
    bm, bi = torch.zeros(5), torch.zeros(5, dtype=torch.int32)
    ct.argmax_blocks_f16(logits, ct.partition(bm, [1]), ct.partition(bi, [1]), 5000, generics=[1024])
    rec, _ = _last(ct)
    assert rec.symbol == b"argmax_blocks_entry__f16" and tuple(rec.grid) == (5, 1, 1)
    w, hid = torch.zeros(320, 256, dtype=h), torch.zeros(1, 256, dtype=h)
    ct.lm_head_argmax_blocks_f16(w, hid, ct.partition(bm, [1]), ct.partition(bi, [1]), 300, generics=[256])
    rec, _ = _last(ct)
    assert rec.symbol == b"lm_head_argmax_blocks_entry__f16" and tuple(rec.grid) == (5, 1, 1) and rec.shared_mem_bytes == 512
    out = torch.zeros(1, dtype=torch.int32)
    ct.argmax_reduce_blocks_to_u32(bm, bi, ct.partition(out, [1]), 5)
    assert _last(ct)[0].symbol == b"argmax_reduce_blocks_entry__u32" and tuple(_last(ct)[0].grid) == (1, 1, 1)
    ids, table, emb = torch.zeros(7, dtype=torch.int32), torch.zeros(100, 64, dtype=h), torch.zeros(7, 64, dtype=h)
    ct.embedding_batch_f16(ids, table, ct.partition(emb, [1, 32]), generics=[64, 32])
    assert _last(ct)[0].symbol == b"embedding_batch_entry__f16" and tuple(_last(ct)[0].grid) == (7, 1, 1)
    row = torch.zeros(64, dtype=h)
    ct.gather_row_f16(table, ct.partition(row, [16]), 3)
    assert _last(ct)[0].symbol == b"gather_row_entry__f16"
    n0 = ct.lib().cutile_testing_launch_count()
    cases = [
        (lambda: ct.argmax_blocks_f16(logits.float(), ct.partition(bm, [1]), ct.partition(bi, [1]), 5000), "logits must be f16"),
        (lambda: ct.argmax_blocks_f16(logits, ct.partition(bm, [2]), ct.partition(bi, [1]), 5000), "partitioned \\[1\\]"),
        (lambda: ct.argmax_blocks_f16(logits, ct.partition(bm, [1]), ct.partition(bi[:4], [1]), 5000), "does not match the inferred partition grid"),
        (lambda: ct.lm_head_argmax_blocks_f16(w, torch.zeros(1, 128, dtype=h), ct.partition(bm, [1]), ct.partition(bi, [1]), 300), "expected \\[1, 256\\]"),
        (lambda: ct.lm_head_argmax_blocks_f16(torch.zeros(320, 48, dtype=h), torch.zeros(1, 48, dtype=h), ct.partition(bm, [1]), ct.partition(bi, [1]), 300), "multiple of 32"),
        (lambda: ct.argmax_reduce_blocks_to_u32(bm, bi, ct.partition(torch.zeros(2, dtype=torch.int32), [1]), 5), "one u32"),
        (lambda: ct.embedding_batch_f16(ids, table, ct.partition(torch.zeros(7, 32, dtype=h), [1, 32])), "D = 64"),
        (lambda: ct.embedding_batch_f16(ids, table, ct.partition(emb, [1, 32]), generics=[64, 16]), "BLOCK_SIZE"),
        (lambda: ct.gather_row_f16(table, ct.partition(row, [16]), -1), "non-negative"),
    ]
    for fn, msg in cases:
        with pytest.raises(ct.CutileError, match=msg):
            fn()
    assert ct.lib().cutile_testing_launch_count() == n0


# ---- HIP kernels (GPU) --------------------------------------------------------------------------
def _dev16(bits, dev):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(dev).view(torch.half)


@pytest.mark.gpu
@pytest.mark.parametrize("n,bs,length", [(128256, 1024, 128256), (5000, 512, 4321), (100, 128, 120), (3000, 4096, 3000), (2048, 256, 0)])
def test_gpu_argmax_blocks_and_reduce(ct, dev, n, bs, length):
    bits = f16b(oracle.normal_f32(n, 831))
    if n == 5000:
        bits[[4000, 600, 610]] = f16b([30.0])[0]                # equal maxima: the smallest index wins
    nb = -(-max(n, length) // bs)
    bm = torch.full((nb,), float("nan"), device=dev)
    bi = torch.full((nb,), -1, dtype=torch.int32, device=dev)
    ct.argmax_blocks_f16(_dev16(bits, dev), ct.partition(bm, [1]), ct.partition(bi, [1]), length, generics=[bs])
    out = torch.full((1,), -1, dtype=torch.int32, device=dev)
    ct.argmax_reduce_blocks_to_u32(bm, bi, ct.partition(out, [1]), nb)
    torch.cuda.synchronize()
    rm, ri = oracle.argmax_blocks_f16(bits, bs, length, nb)
    assert np.array_equal(bm.cpu().numpy(), rm) and np.array_equal(bi.cpu().numpy().view(np.uint32), ri)
    assert int(out.item()) == oracle.argmax_reduce_blocks_to_u32(rm, ri, nb)
    if length == n and n > 0:
        assert int(out.item()) == int(np.argmax(f16v(bits)))


@pytest.mark.gpu
@pytest.mark.parametrize("rows,k,vocab", [(4096, 1024, 4096), (1000, 256, 990), (130, 4096, 130), (640, 96, 640), (200, 8192, 150),
                                            (40000, 2080, 39990), (70016, 64, 70016)])
def test_gpu_lm_head_argmax(ct, dev, rows, k, vocab):
    w, h = f16b(oracle.normal_f32((rows, k), 841)), f16b(oracle.normal_f32(k, 842))
    nb = -(-rows // 64)
    bm = torch.full((nb,), float("nan"), device=dev)
    bi = torch.full((nb,), -1, dtype=torch.int32, device=dev)
    ct.lm_head_argmax_blocks_f16(_dev16(w, dev), _dev16(h.reshape(1, k), dev), ct.partition(bm, [1]), ct.partition(bi, [1]), vocab, generics=[k])
    out = torch.full((1,), -1, dtype=torch.int32, device=dev)
    ct.argmax_reduce_blocks_to_u32(bm, bi, ct.partition(out, [1]), nb)
    torch.cuda.synchronize()
    rm, ri = oracle.lm_head_argmax_blocks_f16(w, h, vocab)
    got_m, got_i = bm.cpu().numpy(), bi.cpu().numpy().view(np.uint32)
    logits = f16v(w).astype(np.float64) @ f16v(h).astype(np.float64)
    tol = 1e-4 * np.sqrt(k)
    assert np.all(np.abs(got_m - rm) <= tol)
    for b in range(nb):
        lo, hi = b * 64, min((b + 1) * 64, vocab)
        if lo >= hi:
            assert got_i[b] == ri[b] == lo and got_m[b] == np.float32(-1e30)
            continue
        assert lo <= got_i[b] < hi and logits[got_i[b]] >= logits[lo:hi].max() - tol      # a maximiser up to rounding
        top = np.sort(logits[lo:hi])[-2:]
        if len(top) < 2 or top[1] - top[0] > 2 * tol:
            assert got_i[b] == ri[b]
    best = int(out.item())
    assert logits[best] >= logits[:vocab].max() - tol


@pytest.mark.gpu
def test_gpu_embedding_and_gather_row(ct, dev):
    table = f16b(oracle.normal_f32((1000, 4096), 851))
    ids = np.array([3, 999, 0, 3, 512, 1000, 77], np.uint32)             # 1000 is beyond the table: zeros
    td = _dev16(table, dev)
    out = torch.full((7, 4096), 9.0, dtype=torch.half, device=dev)
    ct.embedding_batch_f16(torch.from_numpy(ids.view(np.int32)).to(dev), td, ct.partition(out, [1, 1024]), generics=[4096, 1024])
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint16), oracle.embedding_batch_f16(ids, table))
    # a narrow table through the element path, fewer output rows than ids
    small = f16b(oracle.normal_f32((20, 12), 852))
    o2 = torch.zeros(5, 12, dtype=torch.half, device=dev)
    ct.embedding_batch_f16(torch.from_numpy(ids.view(np.int32)).to(dev), _dev16(small, dev), ct.partition(o2, [1, 4]))
    torch.cuda.synchronize()
    assert np.array_equal(o2.cpu().numpy().view(np.uint16), oracle.embedding_batch_f16(ids[:5], small))
    row = torch.zeros(4096, dtype=torch.half, device=dev)
    ct.gather_row_f16(td, ct.partition(row, [256]), 512)
    torch.cuda.synchronize()
    assert np.array_equal(row.cpu().numpy().view(np.uint16), oracle.gather_row_f16(table, 512))
    wide = torch.full((5000,), 1.0, dtype=torch.half, device=dev)
    ct.gather_row_f16(td, ct.partition(wide, [1000]), 999)
    torch.cuda.synchronize()
    assert np.array_equal(wide.cpu().numpy().view(np.uint16), oracle.gather_row_f16(table, 999, 5000))
