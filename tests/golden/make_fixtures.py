"""Writes tests/golden/reference_cases.json: the known-answer cases that the reference's own
tests and examples hold for the kernels on the hot path, as data.

Nothing of the reference is imported or executed.  Every case below is the INPUT DEFINITION and
the EXPECTED OUTPUT that a reference test states in its text (file:line cited per case).  Where a
reference test computes its expectation with its own CPU loop on patterned inputs
(persistent_gemm.rs), the expected values stored here are evaluated in exact rational arithmetic
from the same input definition, so they do not depend on any floating-point summation order and
are independent of this repository's oracle.

Run:  python tests/golden/make_fixtures.py        (rewrites the JSON next to this file)
"""
from __future__ import annotations

import json
import os
from fractions import Fraction

HERE = os.path.dirname(os.path.abspath(__file__))


def persistent_gemm_case():
    # cutile-examples/examples/persistent_gemm.rs:70-75 (M, N, K), :89-94 (input patterns), :111-118 (|err| < 1e-3)
    m, n, k = 64, 64, 32
    x = lambda r, c: Fraction((r % 7) - 3, 4) + Fraction(c % 5, 8)
    y = lambda r, c: Fraction((r % 3) + 1, 5) - Fraction(c % 11, 20)
    samples = []
    for (i, j) in [(0, 0), (1, 1), (6, 10), (7, 11), (13, 27), (31, 5), (40, 63), (63, 0), (63, 63), (22, 44)]:
        v = sum(x(i, t) * y(t, j) for t in range(k))
        samples.append({"row": i, "col": j, "num": v.numerator, "den": v.denominator, "value": float(v)})
    # whole-matrix invariant: sum of all outputs, exact
    total = sum(sum(x(i, t) for i in range(m)) * sum(y(t, j) for j in range(n)) for t in range(k))
    return {
        "cite": "cutile-examples/examples/persistent_gemm.rs:70-75,89-94,111-118",
        "m": m, "n": n, "k": k, "tile": [16, 16, 8], "abs_tol": 1e-3,
        "x_pattern": "((row % 7) - 3) * 0.25 + (col % 5) * 0.125",
        "y_pattern": "((row % 3) + 1) * 0.2 - (col % 11) * 0.05",
        "samples": samples,
        "sum_of_outputs": {"num": total.numerator, "den": total.denominator, "value": float(total)},
    }


def mapped_partition_cases():
    # cutile/src/tensor.rs:2203-2350: MappedLaunchPartition::validate(partition_grid, num_tile_blocks)
    ok = lambda name, line, grid, mp, ntb: {"name": name, "cite": f"cutile/src/tensor.rs:{line}", "partition_grid": grid,
                                            "map_shape": mp, "num_tile_blocks": ntb, "launch_grid": [ntb, 1, 1]}
    err = lambda name, line, grid, mp, ntb, msg: {"name": name, "cite": f"cutile/src/tensor.rs:{line}", "partition_grid": grid,
                                                  "map_shape": mp, "num_tile_blocks": ntb, "error_contains": msg}
    validate = [
        ok("swizzle_accepts_tile_block_count", "2203-2212", [2, 3, 1], [4, 1], 3),
        err("swizzle_rejects_tile_block_count_larger_than_logical_grid", "2214-2226", [2, 3, 1], [4, 1], 7,
            "num_tile_blocks cannot exceed the streamed logical tile count"),
        ok("owned_axis_excluded_from_streamed_tile_count", "2228-2239", [2, 3, 1], [1, 0], 2),
        err("owned_axis_excluded_from_streamed_tile_count_over", "2240-2249", [2, 3, 1], [1, 0], 3,
            "num_tile_blocks cannot exceed the streamed logical tile count"),
        err("owned_axis_rejects_all_owned_map", "2251-2262", [2, 3, 1], [0, 0], 1, "at least one streamed (non-OWNED) map axis"),
        ok("owned_axis_accepts_leading_owned", "2264-2274", [2, 3, 1], [0, 1], 3),
        err("swizzle_rejects_zero_tile_blocks", "2276-2285", [2, 3, 1], [4, 1], 0, "num_tile_blocks > 0"),
        err("swizzle_rejects_grid_rank_above_map_rank", "2287-2298", [2, 3, 4], [4, 1], 3,
            "map rank must match the logical partition grid rank"),
        ok("swizzle_accepts_rank1_map", "2300-2309", [8, 1, 1], [1], 4),
        ok("swizzle_accepts_rank3_map", "2311-2320", [2, 3, 4], [1, 4, 1], 6),
        err("swizzle_rejects_rank1_map_with_2d_grid", "2322-2333", [2, 3, 1], [1], 2,
            "map rank must match the logical partition grid rank"),
        err("swizzle_rejects_map_rank_above_3", "2335-2345", [2, 3, 4], [1, 1, 1, 1], 2, "rank-1 through rank-3 map shape"),
    ]
    # cutile/tests/gpu/mapped_partition_schedule_matrix.rs:219-300: every (dims, tile, map, num_tile_blocks) of the
    # coverage matrix; the expectation is that every element ends up holding its tile's row-major index.
    matrix = [{"dims": [64], "tile": [16], "map_shape": [1], "num_tile_blocks": ntb} for ntb in (1, 3, 4)]
    for rows, cols in ((4, 4), (3, 5)):
        total = rows * cols
        for mp in ([1, 1], [2, 1], [2, 2], [3, 2]):
            for ntb in (1, min(5, total), total):
                matrix.append({"dims": [rows * 8, cols * 8], "tile": [8, 8], "map_shape": mp, "num_tile_blocks": ntb})
    for mp in ([1, 1, 1], [1, 2, 1], [1, 2, 2], [1, 3, 2]):
        for ntb in (1, 5, 12):
            matrix.append({"dims": [2, 12, 16], "tile": [1, 4, 8], "map_shape": mp, "num_tile_blocks": ntb})
    # cutile/tests/gpu/mapped_partition_schedule_matrix.rs:320-369: iter_indices_within([(start, len), (0, -1)]) on a
    # 64 x 64 tensor in 16 x 16 tiles, 4 tile blocks; rows of tiles [lo, hi) receive their flat index, the rest keep
    # the poison.
    sub = lambda mp, start, length, lo, hi: {"map_shape": mp, "start": start, "len": length, "expect_lo": lo, "expect_hi": hi}
    subrange = {"cite": "cutile/tests/gpu/mapped_partition_schedule_matrix.rs:320-369", "dims": [64, 64], "tile": [16, 16],
                "num_tile_blocks": 4, "poison": -0x5EAD,
                "cases": [sub([1, 1], 1, 0, 0, 0), sub([1, 1], 3, 1, 3, 4), sub([1, 1], 2, -1, 2, 4), sub([1, 1], 0, -1, 0, 4),
                          sub([2, 1], 1, 2, 1, 3), sub([2, 2], 0, 3, 0, 3)]}
    # the same file :372-476: two caches [heads, max_seq, d] written through one shared stream over the sequence sub-range
    shared = {"cite": "cutile/tests/gpu/mapped_partition_schedule_matrix.rs:372-476", "heads": 2, "max_seq": 8, "d": 16,
              "tile": [1, 1, 16], "map_shape": [1, 1, 1], "poison": -333.25,
              "dynpos": {"source_shape": [2, 2, 16], "source_scale": 0.5, "position": 3, "n_tiles": 2, "num_tile_blocks": 4},
              "prefill": {"source_shape": [2, 2, 16], "source_scale": 0.25, "seq_len": 2, "num_tile_blocks": 4}}
    return {"validate": validate, "subrange": subrange, "shared_rank3": shared,
            "schedule_matrix": {"cite": "cutile/tests/gpu/mapped_partition_schedule_matrix.rs:219-300",
                                                      "poison": -0x5EAD, "cases": matrix},
            "persistent_gemm_launch": {"cite": "cutile-examples/examples/persistent_gemm.rs:70-79",
                                       "map_shape": [4, 1], "num_tile_blocks": 4}}


def main():
    cases = {
        "mapped_partition": mapped_partition_cases(),
        "saxpy_example": {
            "cite": "cutile-examples/examples/saxpy.rs:28-53",
            "a": 2.0, "shape": [4, 8], "partition": [2, 2],
            "x": [float(i) for i in range(32)], "y": [float(i) for i in range(32)],
            "expected": [3.0 * i for i in range(32)], "comparison": "exact",
        },
        "async_saxpy": {
            "cite": "cutile/tests/gpu/async_saxpy_unsafe.rs:124-127",
            "a": 2.0, "n": 1024, "x_is": "arange", "y_is": "arange", "expected_is": "a * i + i", "comparison": "exact",
        },
        "add_ones": {
            "cite": "cutile/tests/gpu/add_basic.rs:29-43",
            "n": 32, "partition": [4], "grid": [8, 1, 1], "x_fill": 1.0, "y_fill": 1.0, "expected_fill": 2.0, "abs_tol": 1e-6,
        },
        "gemm_ones_non_divisible": {
            "cite": "cutile/tests/slice_non_divisible.rs:458-497",
            "m": 100, "n": 100, "k": 64, "reference_tile": [16, 16, 8], "fill": 1.0, "expected_fill": 64.0, "abs_tol": 1e-3,
        },
        "persistent_gemm_patterned": persistent_gemm_case(),
        "softmax_rows_sum_to_one": {
            "cite": "cutile-examples/examples/softmax.rs:55-60; cutile/tests/gpu/book_snippets.rs:241-248",
            "abs_tol": 1e-4,
        },
        "fmha_example": {
            "cite": "cutile-examples/examples/flash_attention_causal.rs:216-222,277-281",
            "batch": 2, "heads": 8, "heads_kv": 8, "seq_len": 64, "head_dim": 32, "tile": [32, 32],
            "atol": 2e-3, "rtol": 2e-3, "expectation": "fmha_ref_cpu on the same inputs",
        },
        "mxfp8_all_ones": {
            "cite": "cutile-examples/examples/mxfp8.rs:84-135",
            "m": 16, "n": 16, "k": 128, "reference_tile": [16, 16, 64], "e4m3_code": 0x38, "e8m0_code": 0x7F, "alpha": 1.0,
            "expected_fill": 128.0, "abs_tol": 1e-3,
        },
    }
    with open(os.path.join(HERE, "reference_cases.json"), "w") as f:
        json.dump(cases, f, indent=1)
        f.write("\n")


if __name__ == "__main__":
    main()
