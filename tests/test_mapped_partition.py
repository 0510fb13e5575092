"""Mapped partitions (`partition.map(map_shape, num_tile_blocks)`, cutile/src/tensor.rs:314-401) and the
persistent GEMM over them (cutile-examples/examples/persistent_gemm.rs).

CPU: the host validation against the reference's own unit-test cases (golden fixtures), the oracle's
constructive schedule pinned by what the definition fixes (a permutation of the tile grid; row-major and
column-major special cases; band structure), and the library's host-visible schedule against the oracle.
GPU: the reference's coverage matrix (every tile written exactly once, by the tile block the schedule
names) and the persistent GEMM against the oracle.  The reference asserts coverage only, never the visiting
order, so the ORDER is pinned by the mathematics alone; results do not depend on it."""
import itertools
import json
import os

import numpy as np
import pytest
import torch

import oracle
from util import normal_bf16_bits, to_dev_bf16, rel_l2

CASES = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_cases.json")))["mapped_partition"]


def _logical(grid, tile):
    """a CPU tensor whose partition by `tile` has the logical grid `grid` (metadata only)"""
    dims = [g * t for g, t in zip(grid, tile)]
    return torch.zeros(dims, dtype=torch.int32), dims


# ---- oracle (CPU) ---------------------------------------------------------------------------
@pytest.mark.parametrize("grid,mp", [((4, 4), (1, 1)), ((3, 5), (2, 1)), ((3, 5), (2, 2)), ((3, 5), (3, 2)), ((7, 5), (4, 3)),
                                     ((2, 3, 2), (1, 2, 2)), ((2, 3, 2), (1, 3, 2)), ((5,), (1,)), ((4, 6), (0, 1)), ((4, 6), (1, 0))])
def test_oracle_schedule_is_a_permutation_of_the_streamed_grid(grid, mp):
    order = oracle.mapped_schedule(grid, mp)
    streamed = [range(g) if m != 0 else range(1) for g, m in zip(grid, mp)]
    assert sorted(order) == sorted(itertools.product(*streamed)) and len(set(order)) == len(order)


def test_oracle_schedule_special_cases():
    # (1, 1): row-major
    assert oracle.mapped_schedule((3, 4), (1, 1)) == [(m, n) for m in range(3) for n in range(4)]
    # one band holding every row: column-major
    assert oracle.mapped_schedule((3, 4), (3, 1)) == [(m, n) for n in range(4) for m in range(3)]
    assert oracle.mapped_schedule((3, 4), (8, 1)) == [(m, n) for n in range(4) for m in range(3)]
    # bands of GM rows: the first GM * num_n items stay inside rows 0..GM-1, and the short last band follows
    order = oracle.mapped_schedule((5, 3), (2, 1))
    assert [m for m, _ in order] == [0, 1] * 3 + [2, 3] * 3 + [4] * 3
    assert [n for _, n in order] == [0, 0, 1, 1, 2, 2] * 2 + [0, 1, 2]
    # groups of GN columns inside a band; a group is walked column by column
    order = oracle.mapped_schedule((2, 5), (2, 2))
    assert order == [(0, 0), (1, 0), (0, 1), (1, 1), (0, 2), (1, 2), (0, 3), (1, 3), (0, 4), (1, 4)]
    order = oracle.mapped_schedule((4, 3), (2, 2))
    assert order[:8] == [(0, 0), (1, 0), (0, 1), (1, 1), (0, 2), (1, 2), (2, 0), (3, 0)]
    # rank 3: the leading axis is the slowest, the trailing pair is scheduled inside it
    o3 = oracle.mapped_schedule((2, 3, 2), (1, 2, 1))
    assert [c[0] for c in o3] == [0] * 6 + [1] * 6
    assert [c[1:] for c in o3[:6]] == oracle.mapped_schedule((3, 2), (2, 1))
    # an owned axis is not streamed: its coordinate stays 0
    assert oracle.mapped_schedule((3, 4), (1, 0)) == [(0, 0), (1, 0), (2, 0)]


# ---- host library (CPU) -----------------------------------------------------------------------
@pytest.mark.parametrize("case", CASES["validate"], ids=lambda c: c["name"])
def test_validate_matches_the_reference_unit_tests(ct, case):
    grid = case["partition_grid"]
    rank = 3 if grid[2] != 1 else 2 if grid[1] != 1 else 1
    z, _ = _logical(grid[:rank], [4] * rank)
    mp = ct.mapped(ct.partition(z, [4] * rank), case["map_shape"], case["num_tile_blocks"])
    if "launch_grid" in case:
        assert list(mp.grid()) == case["launch_grid"]
    else:
        with pytest.raises(ct.CutileError, match=case["error_contains"].replace("(", r"\(").replace(")", r"\)")):
            mp.grid()


def test_prefix_partitions_cannot_be_mapped(ct):
    z = torch.zeros(8, 8, dtype=torch.int32)
    with pytest.raises(ct.CutileError, match="partial-coverage .* cannot be mapped"):      # tensor.rs:319-323
        ct.mapped(ct.partition(z, [4, 4], prefix=True), [1, 1], 2).grid()
    with pytest.raises(ct.CutileError, match="leading map axis must be 1"):                 # compile_intrinsic.rs:2806-2815
        ct.mapped(ct.partition(torch.zeros(2, 4, 4, dtype=torch.int32), [1, 2, 2]), [2, 1, 1], 2).grid()
    with pytest.raises(ct.CutileError, match=r"rank-1 mapped partition maps must be \[1\]"):  # :2826-2835
        ct.mapped(ct.partition(torch.zeros(8, dtype=torch.int32), [2]), [2], 2).grid()
    with pytest.raises(ct.CutileError, match=r"rank-1 mapped partition maps must be \[1\]"):  # one streamed axis left
        ct.mapped(ct.partition(torch.zeros(8, 12, dtype=torch.int32), [2, 2]), [2, 0], 2).grid()


@pytest.mark.parametrize("grid,mp", [((4, 4), (1, 1)), ((3, 5), (2, 1)), ((3, 5), (2, 2)), ((3, 5), (3, 2)), ((7, 5), (4, 3)),
                                     ((9, 2), (8, 1)), ((2, 3, 2), (1, 1, 1)), ((2, 3, 2), (1, 2, 2)), ((2, 3, 2), (1, 3, 2)),
                                     ((5,), (1,)), ((4, 6), (0, 1)), ((4, 6), (1, 0)), ((3, 4, 5), (1, 0, 1)), ((3, 4, 5), (0, 2, 2))])
def test_host_schedule_equals_the_oracle(ct, grid, mp):
    z, _ = _logical(grid, [2] * len(grid))
    m = ct.mapped(ct.partition(z, [2] * len(grid)), mp, 1)
    order = oracle.mapped_schedule(grid, mp)
    assert m.num_items() == len(order)
    assert [m.index(t) for t in range(len(order))] == order
    with pytest.raises(ct.CutileError, match="outside"):
        m.index(len(order))


@pytest.mark.parametrize("grid,mp,ranges", [((4, 4), (1, 1), [(1, 2), (0, -1)]), ((4, 4), (2, 1), [(1, 2), (0, -1)]),
                                            ((4, 4), (2, 2), [(0, 3), (0, -1)]), ((7, 5), (4, 3), [(2, -1), (1, 3)]),
                                            ((5,), (1,), [(2, 2)]), ((2, 6, 5), (1, 2, 2), [(1, 1), (1, 4), (0, -1)]),
                                            ((4, 4), (1, 1), [(1, 0), (0, -1)]), ((4, 4), (1, 1), [(4, -1), (0, -1)])])
def test_subrange_schedule_is_the_schedule_of_the_lengths_shifted_by_the_starts(ct, grid, mp, ranges):
    """iter_indices_within (cutile/src/_core.rs:912-930): 'the schedule runs over the effective lengths and the axis
    starts are added to the minted coordinates' (cutile-compiler/src/compiler/compile_expression.rs:1403-1405)"""
    z, _ = _logical(grid, [2] * len(grid))
    m = ct.mapped(ct.partition(z, [2] * len(grid)), mp, 1)
    starts = [s for s, _ in ranges]
    lens = [g - s if n == -1 else n for g, (s, n) in zip(grid, ranges)]
    want = [] if 0 in lens else [tuple(c + s for c, s in zip(idx, starts)) for idx in oracle.mapped_schedule(lens, mp)]
    got = ct.mapped_indices_within(m, ranges)
    assert got == want
    assert len(set(got)) == len(got) and all(s <= c < s + n for idx in got for c, s, n in zip(idx, starts, lens))
    if all(s == 0 for s in starts) and lens == list(grid):
        assert got == [m.index(t) for t in range(m.num_items())]


def test_subrange_over_the_whole_grid_is_the_plain_schedule(ct):
    z, _ = _logical((5, 3), [2, 2])
    m = ct.mapped(ct.partition(z, [2, 2]), (2, 2), 3)
    assert ct.mapped_indices_within(m, [(0, -1), (0, -1)]) == [m.index(t) for t in range(m.num_items())]
    assert ct.mapped_indices_within(m, [(0, 5), (0, 3)]) == [m.index(t) for t in range(m.num_items())]


def test_subrange_rejects_what_the_reference_rejects(ct):
    z, _ = _logical((4, 4), [2, 2])
    m = ct.mapped(ct.partition(z, [2, 2]), (1, 1), 2)
    for ranges, msg in [([(-1, 2), (0, -1)], "start -1 is negative"),                # partition_index_schedules.rs:553
                        ([(0, -2), (0, -1)], "length -2 is negative"),
                        ([(3, 2), (0, -1)], "exceeds the 4 tiles"), ([(5, -1), (0, -1)], "exceeds the 4 tiles")]:
        with pytest.raises(ct.CutileError, match=msg):
            ct.mapped_indices_within(m, ranges)
    owned = ct.mapped(ct.partition(z, [2, 2]), (1, 0), 2)
    with pytest.raises(ct.CutileError, match="OWNED axes is not supported"):         # compile_expression.rs:1279-1284
        ct.mapped_indices_within(owned, [(0, -1), (0, -1)])
    with pytest.raises(ValueError, match="expects 2"):
        ct.mapped_indices_within(m, [(0, -1)])


# ---- HIP kernels (GPU) -----------------------------------------------------------------------
def _expected_flat_index(dims, tile):
    grid = [-(-d // t) for d, t in zip(dims, tile)]
    idx = np.indices(dims)
    flat = np.zeros(dims, np.int64)
    for a in range(len(dims)):
        flat = flat * grid[a] + idx[a] // tile[a]
    return flat.astype(np.int32)


@pytest.mark.gpu
def test_gpu_schedule_matrix_covers_every_tile_exactly_once(ct, dev):
    m = CASES["schedule_matrix"]
    for c in m["cases"]:
        z = torch.full(c["dims"], m["poison"], dtype=torch.int32, device=dev)
        ct.mapped_tile_index(ct.mapped(ct.partition(z, c["tile"]), c["map_shape"], c["num_tile_blocks"]))
        torch.cuda.synchronize()
        assert np.array_equal(z.cpu().numpy(), _expected_flat_index(c["dims"], c["tile"])), c
    # grids the tile shape does not divide, an owned axis, and a strided view
    for dims, tile, mp, ntb in [([30, 21], [8, 8], [3, 2], 4), ([5, 70], [1, 16], [1, 0], 5), ([37], [8], [1], 2),
                                ([3, 10, 9], [1, 4, 4], [1, 2, 2], 7), ([3, 10, 9], [1, 4, 4], [0, 1, 1], 9)]:
        wide = torch.full(dims[:-1] + [dims[-1] + 3], m["poison"], dtype=torch.int32, device=dev)
        z = wide[..., : dims[-1]]
        ct.mapped_tile_index(ct.mapped(ct.partition(z, tile), mp, ntb))
        torch.cuda.synchronize()
        assert np.array_equal(z.cpu().numpy(), _expected_flat_index(dims, tile)), (dims, tile, mp, ntb)
        assert torch.all(wide[..., dims[-1]:] == m["poison"])


@pytest.mark.gpu
def test_gpu_subrange_writes_exactly_the_range(ct, dev):
    """the reference's subrange_edge_cases_write_exactly_the_range (mapped_partition_schedule_matrix.rs:354-369), then
    ranges on both axes, rank 1 and 3 and ragged edges"""
    sr = CASES["subrange"]
    whole = _expected_flat_index(sr["dims"], sr["tile"])
    for c in sr["cases"]:
        z = torch.full(sr["dims"], sr["poison"], dtype=torch.int32, device=dev)
        ct.mapped_tile_index_within(ct.mapped(ct.partition(z, sr["tile"]), c["map_shape"], sr["num_tile_blocks"]),
                                    [(c["start"], c["len"]), (0, -1)])
        torch.cuda.synchronize()
        want = np.full(sr["dims"], sr["poison"], np.int32)
        lo, hi = c["expect_lo"] * sr["tile"][0], c["expect_hi"] * sr["tile"][0]
        want[lo:hi] = whole[lo:hi]
        assert np.array_equal(z.cpu().numpy(), want), c
    for dims, tile, mp, ntb, ranges in [([30, 21], [8, 8], [3, 2], 4, [(1, 2), (1, -1)]), ([37], [8], [1], 2, [(2, 3)]),
                                        ([3, 10, 9], [1, 4, 4], [1, 2, 2], 7, [(1, -1), (0, 2), (2, 1)])]:
        z = torch.full(dims, -7, dtype=torch.int32, device=dev)
        ct.mapped_tile_index_within(ct.mapped(ct.partition(z, tile), mp, ntb), ranges)
        torch.cuda.synchronize()
        grid = [-(-d // t) for d, t in zip(dims, tile)]
        want = np.full(dims, -7, np.int32)
        box = tuple(slice(s * t, (g if n == -1 else s + n) * t) for (s, n), t, g in zip(ranges, tile, grid))
        want[box] = _expected_flat_index(dims, tile)[box]
        assert np.array_equal(z.cpu().numpy(), want), (dims, tile, mp, ranges)


def test_shared_mapped_partitions_need_equal_shapes_and_grids(ct):
    """iter_indices_with (cutile/src/_core.rs:904-911; cutile-compiler/src/compiler/compile_expression.rs:1318-1397)"""
    a = torch.zeros(2, 8, 16)
    part = lambda t, tile=(1, 1, 16), mp=(1, 1, 1), n=4: ct.mapped(ct.partition(t, list(tile)), list(mp), n)
    ct.mapped_partitions_shared(part(a), part(torch.zeros(2, 8, 16)))
    ct.mapped_partitions_shared(part(a), part(torch.zeros(2, 8, 9)))                 # the same (2, 8, 1) grid
    with pytest.raises(ct.CutileError, match="equal logical partition grids: axis 1 has 8 vs 9 tiles"):
        ct.mapped_partitions_shared(part(a), part(torch.zeros(2, 9, 16)))
    with pytest.raises(ct.CutileError, match="share tile and map shapes"):
        ct.mapped_partitions_shared(part(a), part(torch.zeros(2, 16, 16), tile=(1, 2, 16)))
    with pytest.raises(ct.CutileError, match="share tile and map shapes"):
        ct.mapped_partitions_shared(part(a), part(torch.zeros(2, 8, 16), mp=(1, 2, 1)))


@pytest.mark.gpu
def test_gpu_two_caches_through_one_shared_stream(ct, dev):
    """dynpos_shared_rank3_updates_only_the_device_read_range and
    prefill_shared_rank3_bounds_the_source_by_the_subrange_not_the_cache (mapped_partition_schedule_matrix.rs:372-476)"""
    c = CASES["shared_rank3"]
    h, max_seq, d, poison = c["heads"], c["max_seq"], c["d"], c["poison"]

    def caches(n_blocks):
        k, v = (torch.full((h, max_seq, d), poison, device=dev) for _ in range(2))
        mk = lambda t: ct.mapped(ct.partition(t, c["tile"]), c["map_shape"], n_blocks)
        return k, v, mk(k), mk(v)

    # start read from device memory; source [heads, seq, d]
    dp = c["dynpos"]
    src = (np.arange(np.prod(dp["source_shape"]), dtype=np.float32) * dp["source_scale"] + 1.0).reshape(dp["source_shape"])
    k, v, mk, mv = caches(dp["num_tile_blocks"])
    pos = torch.tensor([dp["position"]], dtype=torch.int32, device=dev)
    ct.mapped_shared_cache_update_f32(mk, mv, torch.from_numpy(src).to(dev), dp["n_tiles"], position=pos)
    torch.cuda.synchronize()
    want = np.full((h, max_seq, d), poison, np.float32)
    want[:, dp["position"]:dp["position"] + dp["n_tiles"]] = src
    want_v = np.where(want == poison, want, 2 * want)
    assert np.array_equal(k.cpu().numpy(), want) and np.array_equal(v.cpu().numpy(), want_v)
    # the same start by value
    k, v, mk, mv = caches(dp["num_tile_blocks"])
    ct.mapped_shared_cache_update_f32(mk, mv, torch.from_numpy(src).to(dev), dp["n_tiles"], start_tile=dp["position"])
    torch.cuda.synchronize()
    assert np.array_equal(k.cpu().numpy(), want) and np.array_equal(v.cpu().numpy(), want_v)
    # a device start that does not fit the axis writes nothing; a host one is an error
    k, v, mk, mv = caches(dp["num_tile_blocks"])
    ct.mapped_shared_cache_update_f32(mk, mv, torch.from_numpy(src).to(dev), dp["n_tiles"],
                                      position=torch.tensor([max_seq - 1], dtype=torch.int32, device=dev))
    torch.cuda.synchronize()
    assert torch.all(k == poison) and torch.all(v == poison)
    with pytest.raises(ct.CutileError, match="exceeds the 8 tiles"):
        ct.mapped_shared_cache_update_f32(mk, mv, torch.from_numpy(src).to(dev), dp["n_tiles"], start_tile=max_seq - 1)
    # prefill: source [seq, heads, d], rows 0..seq_len of a longer cache
    pf = c["prefill"]
    src = (np.arange(np.prod(pf["source_shape"]), dtype=np.float32) * pf["source_scale"] + 1.0).reshape(pf["source_shape"])
    k, v, mk, mv = caches(pf["num_tile_blocks"])
    ct.mapped_shared_cache_update_f32(mk, mv, torch.from_numpy(src).to(dev), pf["seq_len"], source_seq_major=True)
    torch.cuda.synchronize()
    want = np.full((h, max_seq, d), poison, np.float32)
    want[:, :pf["seq_len"]] = src.transpose(1, 0, 2)
    assert np.array_equal(k.cpu().numpy(), want) and np.array_equal(v.cpu().numpy(), np.where(want == poison, want, 2 * want))
    # larger, ragged: tiles [1, 4, 8] over caches [3, 22, 20] (grid (3, 6, 3)), grouped trailing axes, 7 tile blocks
    hh, ms, dd, start, n = 3, 22, 20, 2, 3
    src = np.random.default_rng(5).standard_normal((hh, n * 4, dd)).astype(np.float32)
    k, v = (torch.full((hh, ms, dd), poison, device=dev) for _ in range(2))
    mk, mv = (ct.mapped(ct.partition(t, [1, 4, 8]), [1, 2, 2], 7) for t in (k, v))
    ct.mapped_shared_cache_update_f32(mk, mv, torch.from_numpy(src).to(dev), n, start_tile=start)
    torch.cuda.synchronize()
    want = np.full((hh, ms, dd), poison, np.float32)
    want[:, start * 4:(start + n) * 4] = src
    assert np.array_equal(k.cpu().numpy(), want) and np.array_equal(v.cpu().numpy(), np.where(want == poison, want, 2 * want))


@pytest.mark.gpu
def test_gpu_explicit_grid_is_a_checked_override(ct, dev):
    # an explicit .grid() must equal (num_tile_blocks, 1, 1)
    grid, mp = (5, 4), (2, 2)
    z = torch.full((5 * 4, 4 * 4), -1, dtype=torch.int32, device=dev)
    part = ct.mapped(ct.partition(z, [4, 4]), mp, 20)
    ct.mapped_tile_index(part, grid=(20, 1, 1))
    with pytest.raises(ct.CutileError, match="does not match the inferred partition grid"):
        ct.mapped_tile_index(part, grid=(10, 1, 1))
    torch.cuda.synchronize()
    assert np.array_equal(z.cpu().numpy(), _expected_flat_index([20, 16], [4, 4]))


def _persistent_inputs(case):
    m, n, k = case["m"], case["n"], case["k"]
    r, c = np.meshgrid(np.arange(m), np.arange(k), indexing="ij")
    x = ((r % 7).astype(np.float32) - 3.0) * np.float32(0.25) + (c % 5).astype(np.float32) * np.float32(0.125)
    r, c = np.meshgrid(np.arange(k), np.arange(n), indexing="ij")
    y = ((r % 3).astype(np.float32) + 1.0) * np.float32(0.2) - (c % 11).astype(np.float32) * np.float32(0.05)
    return x.astype(np.float32), y.astype(np.float32)


@pytest.mark.gpu
def test_gpu_persistent_gemm_reference_example(ct, dev):
    """persistent_gemm.rs as written: f32, 16x16x8 tiles, M = N = 64, K = 32, map [4, 1], four tile blocks"""
    all_cases = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_cases.json")))
    p, launch = all_cases["persistent_gemm_patterned"], CASES["persistent_gemm_launch"]
    x, y = _persistent_inputs(p)
    z = torch.full((p["m"], p["n"]), float("nan"), dtype=torch.float32, device=dev)
    bm, bn, bk = p["tile"]
    ct.gemm_persistent(ct.mapped(ct.partition(z, [bm, bn]), launch["map_shape"], launch["num_tile_blocks"]),
                       torch.from_numpy(x).to(dev), torch.from_numpy(y).to(dev),
                       generics=["f32", bm, bn, bk, launch["map_shape"][0], launch["map_shape"][1]])
    torch.cuda.synchronize()
    got = z.cpu().numpy()
    for s in p["samples"]:
        assert abs(got[s["row"], s["col"]] - s["num"] / s["den"]) < p["abs_tol"]
    assert np.max(np.abs(got - oracle.cpu_gemm_f32(x, y))) < p["abs_tol"]
    with pytest.raises(ct.CutileError, match="MAP_SHAPE"):
        ct.gemm_persistent(ct.mapped(ct.partition(z, [bm, bn]), [4, 1], 4), torch.from_numpy(x).to(dev),
                           torch.from_numpy(y).to(dev), generics=["f32", bm, bn, bk, 2, 1])


@pytest.mark.gpu
@pytest.mark.parametrize("m,n,k,tile,mp,ntb,variant", [
    (1024, 1024, 512, 256, (8, 1), 16, None),                   # full grid: one item per tile block
    (1024, 768, 256, 256, (2, 1), 5, "bf16_256x256x64_d2x4"),   # a non-divisor number of tile blocks
    (1024, 768, 256, 256, (2, 1), 5, "bf16_256x256x64_q2x4"),   # the same on the 16 x 16 x 32 ring (whole K tiles of 64)
    (1000, 520, 192, 256, (3, 2), 1, "bf16_256x256x64_q2x4"),   # ragged edges, one tile block walks everything
    (1000, 520, 200, 256, (3, 2), 1, None),                     # ragged edges, K tail, one tile block walks everything
    (640, 384, 128, 128, (4, 1), 7, None),
    (300, 200, 96, 64, (2, 2), 6, None),                        # no matrix-core variant for 64x64 tiles: any-layout kernel
])
def test_gpu_persistent_gemm_bf16(ct, dev, m, n, k, tile, mp, ntb, variant):
    a, b = normal_bf16_bits((m, k), 801, k ** -0.5), normal_bf16_bits((k, n), 802)
    z = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
    ct.gemm_persistent(ct.mapped(ct.partition(z, [tile, tile]), mp, ntb), to_dev_bf16(a, dev), to_dev_bf16(b, dev), variant=variant)
    torch.cuda.synchronize()
    ref = oracle.bf16_bits_to_f32(oracle.gemm_bf16(a, b))
    got = z.float().cpu().numpy()
    assert np.all(np.isfinite(got))
    assert rel_l2(got, ref) <= 1e-2        # the bf16 GEMM tolerance
