"""The bench run's final stdout line: one JSON object of at most 4 KiB that carries the headline record with its
roofline and CPU baseline, every benchmark configuration in short form and the same run's copy ceiling.  Built
here from stub records (no GPU): the size limit and the keys a reader of the line relies on."""
import json
import os
import sys

import pytest

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import bench  # noqa: E402


def _stub(name, bound="mfma", unit="TFLOP/s", peak=2500.0, verbose=False):
    rf = {"bound": bound, "achieved": 1409.123456789, "peak": peak, "unit": "GB/s" if bound == "hbm" else "TFLOP/s",
          "frac": 0.5636493827, "traffic": 1905000000.0, "traffic_source": "x" * 80, "kernel_ms": 0.78031234567,
          "kernel_ms_min": 0.77, "kernel_ms_mean": 0.79, "kernel_ms_back_to_back": 0.85712345, "frac_back_to_back": 0.513123456,
          "frac_wall": 0.5129876543, "sustained_launch_ms": {"first": 0.8, "median": 0.85, "last": 0.86, "max": 0.9},
          "reps": 20, "protocol": "p" * 90, "algorithmic_work": 1099511627776.0}
    rec = {"workload": name, "value": 1282.7654321, "unit": unit, "ms_per_step": 0.857123456, "dtype": "bf16 in / f32 accumulate / bf16 out",
           "config": {"workload": "GEMM bf16 C[8192,8192] += A[8192,8192] . B[8192,8192], row-major, entries N(0,1)/sqrt(K)", "tile": "256x256x64"},
           "roofline": rf,
           "kernel": {"variant": "gemm_entry__bf16_256x256x64_q2x4", "chosen_by": "tuning record", "shape_class": "tiles>256"},
           "cpu_baseline": {"value": 0.0123456789, "unit": "TFLOP/s", "cores": 16, "kind": "port",
                            "sample": "64 of 8192 output rows, naive f32 triple loop (cpu_gemm), OpenMP over rows"},
           "parity": {"rel_l2_sampled_rows": 0.0012345678, "tolerance": 0.01, "ok": True}}
    if verbose:
        rec["config"]["note"] = "n" * 300
    return rec


def _records():
    recs = [_stub(n) for n in bench.BASELINE_CONFIGS]
    for r in recs:
        if r["workload"].startswith(("rms_norm", "softmax", "saxpy")):
            r["roofline"].update(bound="hbm", peak=8000.0, unit="GB/s", achieved=5808.4)
    recs += [_stub(f"other_{i}", verbose=True) for i in range(25)]      # the rest of a default run: never in the line
    return recs


def test_line_is_small_and_round_trips():
    text = bench.compact_line(_records(), 20, 5, "gfx950:sramecc+:xnack-", {"hbm_copy_GB/s": 6265.0, "hbm_copy_frac_of_8000": 0.7831,
                                                                             "hbm_copy_what": "library convert kernel"})
    assert "\n" not in text
    assert len(text.encode()) <= 4096
    line = json.loads(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
                "dtype", "data", "config", "roofline", "cpu_baseline", "parity", "kernel", "device", "baseline_configs", "ceilings_summary"):
        assert key in line, key
    assert line["n_gpus"] == 1 and line["steps"] == 20 and line["warmup"] == 5 and line["vs_baseline"] is None
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel_ms", "kernel_ms_back_to_back", "frac_back_to_back", "frac_wall"):
        assert key in line["roofline"], key
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in line["cpu_baseline"], key
    assert set(line["baseline_configs"]) == set(bench.BASELINE_CONFIGS)
    assert "also" not in line and "tuning_records" not in line and "launch_modes" not in line
    # bandwidth-bound configurations carry their distance to the same run's copy ceiling
    rms = line["baseline_configs"]["rms_norm_f16_16384x8192"]
    assert rms["frac_of_copy_ceiling"] == pytest.approx(5808.4 / 6265.0, abs=1e-4)
    assert "frac_of_copy_ceiling" not in line["baseline_configs"]["gemm_bf16_8192"]
    for e in line["baseline_configs"].values():
        assert {"achieved", "frac", "kernel_ms", "kernel_ms_b2b", "frac_b2b", "ms_per_step", "frac_wall", "parity_ok"} <= set(e)


def test_line_with_probe_summary_still_fits():
    summary = {"hbm_copy_GB/s": 6265.0, "hbm_copy_frac_of_8000": 0.7831, "hbm_copy_what": "library convert kernel f32->f32, 2^26 elements",
               "probe_TFLOP/s": {"mfma_loop_ones": 2391.1, "mfma_loop_random": 1987.2, "mfma_16x16x32_random_lds_operands": 1931.0,
                                 "vendor_library_gemm_8192": 1286.3,
                                 "own_kernels_zero_operands_flushed|b2b": {n: [1800.1, 1790.2] for n in
                                                                          ("gemm_bf16_8192", "gemm_bf16_4096", "mxfp8_gemm_8192", "fmha_bf16", "fmha_bf16_causal")}},
               "probe_GB/s": {"read": 6962.0, "write": 5845.0, "copy": 6265.0}}
    text = bench.compact_line(_records(), 50, 20, "gfx950:sramecc+:xnack-", summary)
    assert len(text.encode()) <= 4096
    assert json.loads(text)["ceilings_summary"]["probe_GB/s"]["copy"] == 6265.0


def test_oversized_line_is_an_error_not_a_long_line():
    recs = _records()
    recs[0]["config"]["workload"] = "w" * 5000
    with pytest.raises(RuntimeError, match="over the 4096-byte limit"):
        bench.compact_line(recs, 20, 5, "gfx950")


def test_default_run_leaves_out_the_example_programs():
    names = {w.name for w in bench.make_workloads()}
    assert set(bench.BASELINE_CONFIGS) <= names
    extra = {w.name for w in bench.make_extra_workloads()}
    assert extra and not (extra & names)
