"""KV block layout conversion: copy_stacked_to_contiguous_f16 / copy_contiguous_to_stacked_f16
(cutile-kernels/src/experimental/kvbm.rs:112-187, 283-352; layouts and index maps :358-400).

A block holds nh heads x nl layers x no offsets x nt tokens x hd values.  Stacked: one tensor per (block, layer, offset),
[nt, nh, hd] (NHD) or [nh, nt, hd] (HND).  Contiguous: one tensor per block, operational ([nl, no] + the stacked inner
order) or universal [nh, nl, no, nt, hd].  CPU: the oracle (a transpose by the reference's index map) against element-by-
element definitions of the layouts.  GPU: copies are bit-exact, both directions, every supported pair."""
import numpy as np
import pytest
import torch

import oracle

PAIRS = [("nhd", "universal"), ("hnd", "universal"), ("nhd", "operational_nhd"), ("hnd", "operational_hnd")]
S_ID = {"nhd": 0, "hnd": 1}
C_ID = {"operational_nhd": 0, "operational_hnd": 1, "universal": 2}


def _stacked(blocks, nh, nl, no, nt, hd, layout, seed):
    inner = (nt, nh, hd) if layout == "nhd" else (nh, nt, hd)
    return np.random.default_rng(seed).integers(0, 65536, (blocks, nl, no) + inner).astype(np.uint16)


# ---- oracle (CPU) ---------------------------------------------------------------------------
@pytest.mark.parametrize("stacked_layout,contiguous_layout", PAIRS)
def test_oracle_kvbm_layouts_element_by_element(stacked_layout, contiguous_layout):
    blocks, nh, nl, no, nt, hd = 2, 3, 2, 2, 4, 5
    st = _stacked(blocks, nh, nl, no, nt, hd, stacked_layout, 951)
    ct = oracle.kvbm_stacked_to_contiguous(st, stacked_layout, contiguous_layout)
    for b in range(blocks):
        for h in range(nh):
            for l in range(nl):
                for o in range(no):
                    for t in range(nt):
                        src = st[b, l, o, t, h] if stacked_layout == "nhd" else st[b, l, o, h, t]
                        if contiguous_layout == "universal":
                            dst = ct[b, h, l, o, t]                     # [heads, layers, offsets, tokens, head_dim] (:371-376)
                        elif contiguous_layout == "operational_nhd":
                            dst = ct[b, l, o, t, h]                     # [layers, offsets, tokens * heads * head_dim], NHD inner order
                        else:
                            dst = ct[b, l, o, h, t]
                        assert np.array_equal(src, dst)
    assert np.array_equal(oracle.kvbm_contiguous_to_stacked(ct, stacked_layout, contiguous_layout), st)
    # the reference derives the shapes with remap(src, map)[i] = src[map[i]] (:403-409)
    universal = [nh, nl, no, nt, hd]
    stacked_shape = [universal[i] for i in oracle.KVBM_UNIVERSAL_TO_STACKED[stacked_layout]]
    contiguous_shape = [stacked_shape[i] for i in oracle.KVBM_STACKED_TO_CONTIGUOUS[(stacked_layout, contiguous_layout)]]
    assert list(st.shape[1:]) == stacked_shape and list(ct.shape[1:]) == contiguous_shape


def test_kvbm_launcher_validation(fake_hip):
    ct = fake_hip
    from test_host_abi import _last
    stacked, contiguous = torch.zeros(2 * 3 * 2, dtype=torch.int64), torch.zeros(2, dtype=torch.int64)
    ct.kvbm_copy_f16(False, ct.KVBM_STACKED_NHD, ct.KVBM_UNIVERSAL, 2, stacked, contiguous, 4, 3, 2, 16, 128)
    rec, _ = _last(ct)
    assert rec.symbol == b"kvbm_copy_entry__f16" and tuple(rec.block) == (256, 1, 1)
    n0 = ct.lib().cutile_testing_launch_count()
    cases = [
        (lambda: ct.kvbm_copy_f16(False, ct.KVBM_STACKED_NHD, ct.KVBM_OPERATIONAL_HND, 2, stacked, contiguous, 4, 3, 2, 16, 128), "unsupported KVBM stacked-to-contiguous layout map"),
        (lambda: ct.kvbm_copy_f16(True, ct.KVBM_STACKED_HND, ct.KVBM_OPERATIONAL_NHD, 2, stacked, contiguous, 4, 3, 2, 16, 128), "unsupported KVBM contiguous-to-stacked layout map"),
        (lambda: ct.kvbm_copy_f16(False, ct.KVBM_STACKED_NHD, ct.KVBM_UNIVERSAL, 3, stacked, contiguous, 4, 3, 2, 16, 128), "pointer tables"),
        (lambda: ct.kvbm_copy_f16(False, ct.KVBM_STACKED_NHD, ct.KVBM_UNIVERSAL, 2, stacked.int(), contiguous, 4, 3, 2, 16, 128), "pointer tables"),
        (lambda: ct.kvbm_copy_f16(False, ct.KVBM_STACKED_NHD, ct.KVBM_UNIVERSAL, 2, stacked, contiguous, 4, 0, 2, 16, 128), "extents positive"),
    ]
    for fn, msg in cases:
        with pytest.raises(ct.CutileError, match=msg):
            fn()
    ct.kvbm_copy_f16(False, ct.KVBM_STACKED_NHD, ct.KVBM_UNIVERSAL, 0, stacked, contiguous, 4, 3, 2, 16, 128)     # nothing to do
    assert ct.lib().cutile_testing_launch_count() == n0


# ---- HIP kernel (GPU) ---------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("stacked_layout,contiguous_layout", PAIRS)
@pytest.mark.parametrize("blocks,nh,nl,no,nt,hd", [(3, 8, 4, 2, 16, 128), (2, 3, 2, 2, 5, 24), (1, 2, 1, 2, 7, 10)])
def test_gpu_kvbm_round_trip(ct, dev, stacked_layout, contiguous_layout, blocks, nh, nl, no, nt, hd):
    st = _stacked(blocks, nh, nl, no, nt, hd, stacked_layout, 961)
    ref = oracle.kvbm_stacked_to_contiguous(st, stacked_layout, contiguous_layout)
    to_dev = lambda a: torch.from_numpy(a.view(np.int16)).to(dev).view(torch.half)
    # one device tensor per (block, layer, offset), deliberately not adjacent in memory
    chunks = [[[to_dev(st[b, l, o]).clone() for o in range(no)] for l in range(nl)] for b in range(blocks)]
    outs = [torch.full(ref.shape[1:], float("nan"), dtype=torch.half, device=dev) for _ in range(blocks)]
    s_table = torch.tensor([chunks[b][l][o].data_ptr() for b in range(blocks) for l in range(nl) for o in range(no)], dtype=torch.int64, device=dev)
    c_table = torch.tensor([t.data_ptr() for t in outs], dtype=torch.int64, device=dev)
    ct.kvbm_copy_f16(False, S_ID[stacked_layout], C_ID[contiguous_layout], blocks, s_table, c_table, nh, nl, no, nt, hd)
    torch.cuda.synchronize()
    for b in range(blocks):
        assert np.array_equal(outs[b].cpu().numpy().view(np.uint16), ref[b])
    # and back into fresh stacked tensors
    back = [[[torch.zeros_like(chunks[b][l][o]) for o in range(no)] for l in range(nl)] for b in range(blocks)]
    b_table = torch.tensor([back[b][l][o].data_ptr() for b in range(blocks) for l in range(nl) for o in range(no)], dtype=torch.int64, device=dev)
    ct.kvbm_copy_f16(True, S_ID[stacked_layout], C_ID[contiguous_layout], blocks, b_table, c_table, nh, nl, no, nt, hd)
    torch.cuda.synchronize()
    for b in range(blocks):
        for l in range(nl):
            for o in range(no):
                assert np.array_equal(back[b][l][o].cpu().numpy().view(np.uint16), st[b, l, o])
