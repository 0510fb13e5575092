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


def main():
    cases = {
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
