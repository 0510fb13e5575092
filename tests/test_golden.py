"""The reference's own known-answer cases for the hot path (tests/golden/reference_cases.json,
written by tests/golden/make_fixtures.py from the reference tests' text), checked twice:
against the CPU oracle (no GPU needed) and against the HIP kernels through the C ABI."""
import json
import os

import numpy as np
import pytest
import torch

import oracle
from util import to_dev_bf16

CASES = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_cases.json")))


def _patterned(case):
    m, n, k = case["m"], case["n"], case["k"]
    r, c = np.meshgrid(np.arange(m), np.arange(k), indexing="ij")
    x = ((r % 7).astype(np.float32) - 3.0) * np.float32(0.25) + (c % 5).astype(np.float32) * np.float32(0.125)
    r, c = np.meshgrid(np.arange(k), np.arange(n), indexing="ij")
    y = ((r % 3).astype(np.float32) + 1.0) * np.float32(0.2) - (c % 11).astype(np.float32) * np.float32(0.05)
    return x.astype(np.float32), y.astype(np.float32)


# ---- oracle against the golden cases (CPU) ---------------------------------------------------
def test_fixture_file_is_what_the_generator_writes(tmp_path):
    import runpy, shutil
    gen = os.path.join(os.path.dirname(__file__), "golden", "make_fixtures.py")
    work = tmp_path / "golden"
    work.mkdir()
    shutil.copy(gen, work / "make_fixtures.py")
    runpy.run_path(str(work / "make_fixtures.py"), run_name="__main__")
    assert json.load(open(work / "reference_cases.json")) == CASES


def test_oracle_saxpy_golden():
    c = CASES["saxpy_example"]
    got = oracle.saxpy_f32(c["a"], np.array(c["x"], np.float32), np.array(c["y"], np.float32))
    assert got.tolist() == c["expected"]
    n = CASES["async_saxpy"]["n"]
    i = np.arange(n, dtype=np.float32)
    assert np.array_equal(oracle.saxpy_f32(2.0, i, i), 2.0 * i + i)


def test_oracle_add_golden():
    c = CASES["add_ones"]
    got = oracle.add_f32(np.full(c["n"], c["x_fill"], np.float32), np.full(c["n"], c["y_fill"], np.float32))
    assert np.all(np.abs(got - c["expected_fill"]) < c["abs_tol"])


def test_oracle_gemm_golden():
    c = CASES["gemm_ones_non_divisible"]
    z = oracle.cpu_gemm_f32(np.ones((c["m"], c["k"]), np.float32), np.ones((c["k"], c["n"]), np.float32))
    assert z.shape == (c["m"], c["n"]) and np.all(np.abs(z - c["expected_fill"]) < c["abs_tol"])
    p = CASES["persistent_gemm_patterned"]
    x, y = _patterned(p)
    z = oracle.cpu_gemm_f32(x, y)
    for s in p["samples"]:                       # exact rationals evaluated independently of any float loop
        assert abs(z[s["row"], s["col"]] - s["num"] / s["den"]) < p["abs_tol"]
    assert abs(float(z.astype(np.float64).sum()) - p["sum_of_outputs"]["value"]) < 1e-2
    # a transposed operand or a swapped index changes the samples: (1,1) and (6,10) differ from their mirrors
    assert abs(z[6, 10] - z[10, 6]) > 1e-2


def test_oracle_softmax_and_mx_golden():
    x = oracle.normal_f32((8, 96), 77)
    rows = oracle.softmax_f32(x, 1, 96).sum(axis=1)
    assert np.all(np.abs(rows - 1.0) < CASES["softmax_rows_sum_to_one"]["abs_tol"])
    c = CASES["mxfp8_all_ones"]
    q = np.full((c["m"], c["k"]), c["e4m3_code"], np.uint8)
    s = np.full((c["m"], c["k"] // 32), c["e8m0_code"], np.uint8)
    z = oracle.mx_gemm_f32(q, q[: c["n"]], s, s[: c["n"]], c["alpha"])
    assert np.all(np.abs(z - c["expected_fill"]) < c["abs_tol"])


# ---- HIP kernels against the golden cases (GPU, through the C ABI) ----------------------------
@pytest.mark.gpu
def test_gpu_saxpy_and_add_golden(ct, dev):
    c = CASES["saxpy_example"]
    x = torch.tensor(c["x"], device=dev).reshape(c["shape"])
    y = torch.tensor(c["y"], device=dev).reshape(c["shape"])
    ct.saxpy(ct.partition(y, c["partition"]), c["a"], x)
    torch.cuda.synchronize()
    assert y.flatten().tolist() == c["expected"]
    a = CASES["add_ones"]
    z = torch.zeros(a["n"], device=dev)
    ct.add(ct.partition(z, a["partition"]), torch.full((a["n"],), a["x_fill"], device=dev),
           torch.full((a["n"],), a["y_fill"], device=dev), grid=tuple(a["grid"]))
    torch.cuda.synchronize()
    assert torch.all((z - a["expected_fill"]).abs() < a["abs_tol"])


@pytest.mark.gpu
def test_gpu_gemm_golden(ct, dev):
    c = CASES["gemm_ones_non_divisible"]
    # as the reference runs it: f32, tiles 16x16x8, M = N = 100 (any-layout kernel) ...
    z = torch.zeros(c["m"], c["n"], device=dev)
    ct.gemm(ct.partition(z, c["reference_tile"][:2]), torch.ones(c["m"], c["k"], device=dev),
            torch.ones(c["k"], c["n"], device=dev), c["k"], accumulate=False, generics=["f32"] + c["reference_tile"])
    torch.cuda.synchronize()
    assert torch.all((z - c["expected_fill"]).abs() < c["abs_tol"])
    # ... and on the matrix cores (ones are exact in bf16; N padded to a multiple of 8 for 16-byte rows)
    z = torch.zeros(c["m"], 104, device=dev)
    ct.gemm(ct.partition(z, [128, 128]), torch.ones(c["m"], c["k"], dtype=torch.bfloat16, device=dev),
            torch.ones(c["k"], 104, dtype=torch.bfloat16, device=dev), c["k"], accumulate=False)
    torch.cuda.synchronize()
    assert torch.all((z - c["expected_fill"]).abs() < c["abs_tol"])
    p = CASES["persistent_gemm_patterned"]
    x, y = _patterned(p)
    z = torch.zeros(p["m"], p["n"], device=dev)
    ct.gemm(ct.partition(z, p["tile"][:2]), torch.from_numpy(x).to(dev), torch.from_numpy(y).to(dev), p["k"],
            accumulate=False, generics=["f32"] + p["tile"])
    torch.cuda.synchronize()
    got = z.cpu().numpy()
    for s in p["samples"]:
        assert abs(got[s["row"], s["col"]] - s["num"] / s["den"]) < p["abs_tol"]
    assert abs(float(got.astype(np.float64).sum()) - p["sum_of_outputs"]["value"]) < 1e-2
    # the same problem on the matrix cores: inputs rounded to bf16 first (y's 0.2 and 0.05 steps are not exact)
    xb, yb = oracle.f32_to_bf16_bits(x), oracle.f32_to_bf16_bits(y)
    z = torch.zeros(p["m"], p["n"], device=dev)
    ct.gemm(ct.partition(z, [128, 128]), to_dev_bf16(xb, dev), to_dev_bf16(yb, dev), p["k"], accumulate=False,
            generics=["bf16", 128, 128, 32])
    torch.cuda.synchronize()
    ref = oracle.bf16_bits_to_f32(xb).astype(np.float64) @ oracle.bf16_bits_to_f32(yb).astype(np.float64)
    assert np.max(np.abs(z.cpu().numpy() - ref)) < p["abs_tol"]


@pytest.mark.gpu
def test_gpu_mxfp8_and_softmax_golden(ct, dev):
    c = CASES["mxfp8_all_ones"]
    x = torch.full((c["m"], c["k"]), c["e4m3_code"], dtype=torch.uint8, device=dev)
    xs = torch.full((c["m"], c["k"] // 32), c["e8m0_code"], dtype=torch.uint8, device=dev)
    z = torch.zeros(c["m"], c["n"], device=dev)
    ct.linear_tile_mxfp8(ct.partition(z, c["reference_tile"][:2]), x, x.clone(), xs, xs.clone(), c["alpha"],
                         generics=c["reference_tile"] + [c["reference_tile"][2] // 32])
    torch.cuda.synchronize()
    assert torch.all((z - c["expected_fill"]).abs() < c["abs_tol"])
    xr = torch.randn(64, 1024, device=dev)
    y = torch.empty_like(xr)
    ct.softmax(xr, ct.partition(y, [1, 1024]))
    torch.cuda.synchronize()
    assert torch.all((y.sum(dim=1) - 1.0).abs() < CASES["softmax_rows_sum_to_one"]["abs_tol"])


@pytest.mark.gpu
def test_gpu_fmha_golden_shape_and_tolerance(ct, dev):
    c = CASES["fmha_example"]
    b, h, hk, s, d = c["batch"], c["heads"], c["heads_kv"], c["seq_len"], c["head_dim"]
    cast = lambda t: oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(t))
    q, k, v = (cast(oracle.normal_f32((b, hh, s, d), 7 + i)) for i, hh in enumerate((h, hk, hk)))
    out = torch.zeros(b * h, s, d, dtype=torch.bfloat16, device=dev)
    td = lambda t: torch.from_numpy(t).to(dev).to(torch.bfloat16)
    ct.fmha(ct.partition(out, [1, c["tile"][0], d]), td(q), td(k), td(v), d ** -0.5, 0, h // hk, causal=True)
    torch.cuda.synchronize()
    ref = oracle.fmha_ref_cpu(q, k, v, d ** -0.5, 0, h // hk, True).reshape(b * h, s, d)
    got = out.float().cpu().numpy()
    # the reference compares f32 against f32 with atol = rtol = 2e-3; a bf16 output adds half a bf16 ulp (2^-9 relative)
    assert np.all(np.abs(got - ref) <= c["atol"] + (c["rtol"] + 2.0 ** -8) * np.abs(ref))
