#!/usr/bin/env python3
"""Throughput of the tile-kernel path on one MI355X, against the kernel's roofline.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--only] [--variant V] [--ceilings]

A step is one launch of the hot-path kernel over one batch of synthetic input that is
already resident in HBM.  The headline workload is the bf16 GEMM at M = N = K = 8192
(the configuration the target fractions are quoted on); every other benchmark
configuration is measured the same way.  The run ends with ONE JSON line of at most 4 KB
(headline record + every benchmark configuration in short form + the copy ceiling of the
same run); the full records of all workloads go to gpurun_out/bench_full.json.

Timing: W untimed launches, then exactly K launches between two device synchronisations
(wall clock -> ms_per_step / value).  roofline.achieved follows the reference's do_bench
protocol (cutile/src/bench.rs:124-211): per-launch HIP events on the launch stream, a
512 MiB cache flush before every repetition, median reported (minimum, mean and the
back-to-back average beside it; frac_back_to_back and frac_wall are the same work over
the sustained figures).  --ceilings adds the bare-resource probes, the vendor library's
GEMM, the kernels on zero operands and the launch-mode latencies.

cpu_baseline: the CPU oracle (a port of the reference's naive CPU references), timed on
this host's cores on a bounded sample of the same workload.  The sampled output is also
compared against the GPU result ("parity").
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK = {"hbm": (8000.0, "GB/s"), "mfma_bf16": (2500.0, "TFLOP/s"), "mfma_fp8": (5000.0, "TFLOP/s")}
METRIC = "GEMM/FMHA TFLOP/s + % MFMA peak; RMSNorm GB/s + % HBM peak (1 MI355X)"


def _traffic(workload):
    """HBM bytes per launch measured with rocprofv3 --pmc (profiles/traffic.json), or None."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(path):
        with open(path) as f:
            return json.load(f).get(workload)
    return None


class Workload:
    name = ""
    unit = ""
    dtype = ""
    bound = "hbm"
    peak_key = "hbm"
    work = 0.0          # algorithmic bytes or flops per launch
    config = {}

    def setup(self, ct, torch, oracle, dev):
        raise NotImplementedError

    def launch(self):
        raise NotImplementedError

    def cpu_baseline(self, oracle, np, torch):
        return None


def _td_bf16(torch, np, bits, dev):
    return torch.from_numpy(bits.view(np.int16)).to(dev).view(torch.bfloat16)


class Saxpy(Workload):
    name, unit, dtype = "saxpy_f32_16777216", "GB/s", "f32"
    n = 1 << 24
    work = 12.0 * n
    config = {"workload": "saxpy fp32 z = a*x + y, n = 16777216, a = 2.0, tiles of 1024"}

    def setup(self, ct, torch, oracle, dev):
        self.ct = ct
        self.xh, self.yh = oracle.uniform_f32(self.n, 1), oracle.uniform_f32(self.n, 2)
        self.x, self.y = torch.from_numpy(self.xh).to(dev), torch.from_numpy(self.yh).to(dev)
        self.z = torch.empty_like(self.x)
        self.zp = ct.partition(self.z, [1024])

    def launch(self):
        self.ct.axpy(self.zp, 2.0, self.x, self.y)

    def cpu_baseline(self, oracle, np, torch):
        t0 = time.perf_counter()
        reps = 20
        for _ in range(reps):
            ref = oracle.saxpy_f32(2.0, self.xh, self.yh)
        dt = (time.perf_counter() - t0) / reps
        exact = bool(np.array_equal(self.z.cpu().numpy(), ref))
        return {"value": self.work / dt / 1e9, "unit": "GB/s", "cores": oracle.num_threads(), "kind": "port",
                "sample": f"full size, {reps} passes"}, {"bit_exact": exact}


class Copy(Workload):
    """A plain copy of known size; used to calibrate the HBM traffic counters."""
    name, unit, dtype = "copy_f32_67108864", "GB/s", "f32"
    n = 1 << 26
    work = 8.0 * n
    config = {"workload": "plain copy of 2^26 f32 (convert f32 -> f32), calibration for FETCH_SIZE / WRITE_SIZE"}

    def setup(self, ct, torch, oracle, dev):
        self.ct = ct
        self.x = torch.arange(self.n, dtype=torch.float32, device=dev)
        self.z = torch.empty_like(self.x)
        self.zp = ct.partition(self.z, [128])

    def launch(self):
        self.ct.convert(self.x, self.zp)


class RmsNorm(Workload):
    name, unit, dtype = "rms_norm_f16_16384x8192", "GB/s", "f16 io / f32 math"
    m, n = 16384, 8192
    work = float(2 * m * n * 2 + n * 2)
    config = {"workload": "RMSNorm fp16 rows [16384, 8192], weight [8192], eps 1e-6"}

    def setup(self, ct, torch, oracle, dev):
        import numpy as np

        self.ct = ct
        self.xb = oracle.f32_to_f16_bits(oracle.normal_f32((self.m, self.n), 3))
        self.wb = oracle.f32_to_f16_bits(oracle.uniform_f32(self.n, 4, 0.5, 1.5))
        self.x = torch.from_numpy(self.xb.view(np.float16)).to(dev)
        self.w = torch.from_numpy(self.wb.view(np.float16)).to(dev)
        self.o = torch.empty_like(self.x)
        self.op = ct.partition(self.o, [1, self.n])

    def launch(self):
        self.ct.rms_norm_f16(self.x, self.w, self.op, 1e-6)

    def cpu_baseline(self, oracle, np, torch):
        rows = 2048
        t0 = time.perf_counter()
        ref = oracle.rms_norm_f16(self.xb[:rows], self.wb, 1e-6)
        dt = time.perf_counter() - t0
        got = self.o[:rows].cpu().numpy().view(np.uint16)
        d = np.abs(oracle.f16_bits_to_f32(got) - oracle.f16_bits_to_f32(ref))
        ok = bool(np.all(d <= np.abs(oracle.f16_bits_to_f32(ref)) * 2 ** -10 + 1e-7))
        return {"value": (2 * rows * self.n * 2) / dt / 1e9, "unit": "GB/s", "cores": oracle.num_threads(),
                "kind": "port", "sample": f"first {rows} of {self.m} rows"}, {"within_1_f16_ulp": ok}


class Softmax(RmsNorm):
    name = "softmax_f16_16384x8192"
    work = float(2 * RmsNorm.m * RmsNorm.n * 2)
    config = {"workload": "row softmax fp16 [16384, 8192], tiles [1, 8192]"}

    def launch(self):
        self.ct.softmax(self.x, self.op)

    def cpu_baseline(self, oracle, np, torch):
        rows = 2048
        t0 = time.perf_counter()
        ref = oracle.softmax_f16(self.xb[:rows], 1, self.n)
        dt = time.perf_counter() - t0
        got = self.o[:rows].cpu().numpy().view(np.uint16)
        d = np.abs(oracle.f16_bits_to_f32(got) - oracle.f16_bits_to_f32(ref))
        ok = bool(np.all(d <= np.abs(oracle.f16_bits_to_f32(ref)) * 2 ** -10 + 1e-7))
        return {"value": (2 * rows * self.n * 2) / dt / 1e9, "unit": "GB/s", "cores": oracle.num_threads(),
                "kind": "port", "sample": f"first {rows} of {self.m} rows"}, {"within_1_f16_ulp": ok}


class RmsNormAllF16(RmsNorm):
    """The benchmark program's own arithmetic (cutile-benchmarks/benches/rmsnorm.rs:20-66): every operation in f16,
    BLOCK_SIZE = 512 as the benchmark sets it; the result must equal the oracle's bit for bit."""
    name, dtype = "rms_norm_all_f16_16384x8192", "f16 throughout"
    config = {"workload": "RMSNorm fp16 rows [16384, 8192], weight [8192], eps 1e-5, all-f16 arithmetic, BLOCK_SIZE 512"}

    def launch(self):
        self.ct.rms_norm_all_f16(self.x, self.w, self.op, 1e-5, generics=[self.n, 512])

    def cpu_baseline(self, oracle, np, torch):
        rows = 1024
        t0 = time.perf_counter()
        ref = oracle.rms_norm_all_f16(self.xb[:rows], self.wb, 1e-5, 512)
        dt = time.perf_counter() - t0
        got = self.o[:rows].cpu().numpy().view(np.uint16)
        return {"value": (2 * rows * self.n * 2) / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"first {rows} of {self.m} rows (numpy, one f16 rounding per operation)"}, {"bit_exact": bool(np.array_equal(got, ref))}


class SoftmaxAllF16(Softmax):
    """cutile-benchmarks/benches/softmax.rs:19-35 with its own arithmetic: every operation in f16."""
    name, dtype = "softmax_all_f16_16384x8192", "f16 throughout"
    config = {"workload": "row softmax fp16 [16384, 8192], tiles [1, 8192], all-f16 arithmetic"}

    def launch(self):
        self.ct.softmax_all_f16(self.x, self.op)

    def cpu_baseline(self, oracle, np, torch):
        rows = 1024
        t0 = time.perf_counter()
        ref = oracle.softmax_all_f16(self.xb[:rows], 1, self.n)
        dt = time.perf_counter() - t0
        got = self.o[:rows].cpu().numpy().view(np.uint16)
        def ordered(u):
            u = u.astype(np.int32)
            return np.where(u & 0x8000, -(u & 0x7FFF), u)
        d = np.abs(ordered(got) - ordered(ref))
        return {"value": (2 * rows * self.n * 2) / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"first {rows} of {self.m} rows (numpy, one f16 rounding per operation)"}, {"within_2_f16_steps": bool(d.max() <= 2)}


def tuned_tile(kernel, problem, default):
    """The tile shape the tuner's (tile, variant) sweep chose for this problem (cutile-rs_amd/tune/tune_baseline.cpp files
    it in the kernel's tuning record under the bucket "problem|<problem>"), or `default` where no record says."""
    path = os.path.join(ROOT, "cutile-rs_amd", "tuned", kernel + ".json")
    try:
        with open(path) as f:
            for e in json.load(f).get("entries", []):
                if e.get("bucket") == "problem|" + problem:
                    p = e["config"]["params"]
                    return (int(p["bm"]), int(p["bn"])), "tuning record"
    except (OSError, ValueError, KeyError):
        pass
    return default, "default"


class Gemm(Workload):
    unit, dtype, bound, peak_key = "TFLOP/s", "bf16 in / f32 acc / bf16 out", "mfma", "mfma_bf16"

    function = "gemm"          # the launcher --variant pins

    def __init__(self, s, k=None, accumulate=True):
        self.s, self.k, self.accumulate = s, k or s, accumulate
        self.name = f"gemm_bf16_{s}" + (f"_k{k}" if k else "") + ("" if accumulate else "_new")
        self.work = 2.0 * s * s * self.k
        # the tile is the caller's choice (the partition of z): taken from the tuner's sweep over tile shapes
        self.tile, chosen_by = tuned_tile("gemm", f"bf16|{s}x{s}x{self.k}", (256, 256))
        self.config = {"workload": f"GEMM bf16 M=N={s}, K={self.k}, z {'+=' if accumulate else '='} A·B, row-major A,B ~ N(0,1)/sqrt(K), f32 accumulate, bf16 z",
                       "tile": f"{self.tile[0]}x{self.tile[1]}x64", "tile_chosen_by": chosen_by}

    def setup(self, ct, torch, oracle, dev):
        import numpy as np

        s, k = self.s, self.k
        self.ct = ct
        self.ab = oracle.f32_to_bf16_bits(oracle.normal_f32((s, k), 5, 0, k ** -0.5))
        self.bb = oracle.f32_to_bf16_bits(oracle.normal_f32((k, s), 6, 0, k ** -0.5))
        self.a, self.b = _td_bf16(torch, np, self.ab, dev), _td_bf16(torch, np, self.bb, dev)
        self.z = torch.zeros(s, s, dtype=torch.bfloat16, device=dev)
        self.zp = ct.partition(self.z, list(self.tile))

    def launch(self):
        # z is read as the initial accumulator and written back, like the reference's
        # benchmark kernel (cutile-benchmarks/benches/gemm.rs:34-40: z.load(); mma...; z.store()).
        self.ct.gemm(self.zp, self.a, self.b, self.k, accumulate=self.accumulate)

    def cpu_baseline(self, oracle, np, torch):
        rng = np.random.default_rng(7)
        rows = np.sort(rng.choice(self.s, size=1024 if self.s >= 8192 else 512, replace=False)).astype(np.int64)
        self.z.zero_()          # the timed launches accumulated into z: one launch from zero for the comparison
        self.launch()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ref = oracle.gemm_bf16(self.ab, self.bb, rows=rows, f32out=True)
        dt = time.perf_counter() - t0
        got = self.z[torch.from_numpy(rows).to(self.z.device)].float().cpu().numpy()
        rel = float(np.linalg.norm(got - ref) / np.linalg.norm(ref))
        flops = 2.0 * len(rows) * self.s * self.k
        return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": oracle.num_threads(), "kind": "port",
                "sample": f"{len(rows)} of {self.s} output rows of the same problem (naive f32 loop)"}, \
               {"rel_l2_sampled_rows": rel, "tolerance": 1e-2, "ok": rel <= 1e-2}


class GemmPersistent(Gemm):
    """The reference's persistent form (cutile-examples/examples/persistent_gemm.rs): one tile block per CU walks
    the tiles of a mapped output partition in grouped order; zero initial accumulator (z is not read)."""

    function = "gemm_persistent"

    def __init__(self, s, tile_blocks=256, group_m=8):
        super().__init__(s)
        self.name = f"gemm_bf16_{s}_persistent"
        self.tile_blocks, self.group_m = tile_blocks, group_m
        self.config = {"workload": f"persistent GEMM bf16 M=N=K={s}, z = A·B over a mapped partition: map [{group_m}, 1], "
                                   f"{tile_blocks} tile blocks, f32 accumulate, bf16 z", "tile": "256x256x64"}

    def setup(self, ct, torch, oracle, dev):
        super().setup(ct, torch, oracle, dev)
        self.zm = ct.mapped(self.zp, [self.group_m, 1], self.tile_blocks)

    def launch(self):
        self.ct.gemm_persistent(self.zm, self.a, self.b)


class Fmha(Workload):
    unit, dtype, bound, peak_key = "TFLOP/s", "bf16 io / f32 softmax+acc", "mfma", "mfma_bf16"
    b, h, s, d = 4, 32, 4096, 128
    bm = 256
    function = "fmha"

    def __init__(self, causal):
        self.causal = causal
        self.name = "fmha_bf16_causal" if causal else "fmha_bf16"
        self.work = (2.0 if causal else 4.0) * self.s * self.s * self.d * self.h * self.b
        self.config = {"workload": f"FMHA fwd bf16 b=4 h=32 s=4096 d=128 {'causal' if causal else 'non-causal'}, "
                                   "scale 1/sqrt(128)", "tile": f"BM={self.bm}"}

    def setup(self, ct, torch, oracle, dev):
        import numpy as np

        self.ct = ct
        shape = (self.b, self.h, self.s, self.d)
        self.qb, self.kb, self.vb = (oracle.f32_to_bf16_bits(oracle.normal_f32(shape, 8 + i)) for i in range(3))
        self.q, self.k, self.v = (_td_bf16(torch, np, t, dev) for t in (self.qb, self.kb, self.vb))
        self.o = torch.zeros(self.b * self.h, self.s, self.d, dtype=torch.bfloat16, device=dev)
        self.op = ct.partition(self.o, [1, self.bm, self.d])

    def launch(self):
        self.ct.fmha(self.op, self.q, self.k, self.v, self.d ** -0.5, 0, 1, causal=self.causal)

    def cpu_baseline(self, oracle, np, torch):
        rng = np.random.default_rng(9)
        total = self.b * self.h * self.s
        rows = np.sort(rng.choice(total, size=65536, replace=False)).astype(np.int64)
        q, k, v = (oracle.bf16_bits_to_f32(t) for t in (self.qb, self.kb, self.vb))
        t0 = time.perf_counter()
        ref = oracle.fmha_ref_cpu(q, k, v, self.d ** -0.5, 0, 1, self.causal, rows=rows)
        dt = time.perf_counter() - t0
        got = self.o.reshape(total, self.d)[torch.from_numpy(rows).to(self.o.device)].float().cpu().numpy()
        err = float(np.max(np.abs(got - ref)))
        flops = len(rows) * 4.0 * self.s * self.d        # the reference evaluates every key, masked or not
        return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": oracle.num_threads(), "kind": "port",
                "sample": f"{len(rows)} of {total} query rows of the same problem"}, \
               {"max_abs_sampled_rows": err, "tolerance": 2e-2, "ok": err <= 2e-2}


class MxGemm(Workload):
    name, unit, bound, peak_key = "mxfp8_gemm_8192", "TFLOP/s", "mfma", "mfma_fp8"
    dtype = "fp8 e4m3 x e8m0 block scale / f32 acc / bf16 out"
    function = "linear_tile"
    s = 8192
    work = 2.0 * s ** 3
    tile = 256
    config = {"workload": "MX block-scaled fp8 GEMM A[8192,8192] B[8192,8192], e4m3 + e8m0 per 32 K, bf16 out",
              "tile": "256x256x128"}

    def setup(self, ct, torch, oracle, dev):
        s = self.s
        self.ct = ct
        self.xq, self.xs = oracle.mx_quantize_e4m3(oracle.normal_f32((s, s), 12))
        self.yq, self.ys = oracle.mx_quantize_e4m3(oracle.normal_f32((s, s), 13))
        td = lambda t: torch.from_numpy(t).to(dev)
        self.x, self.y, self.xsd, self.ysd = td(self.xq), td(self.yq), td(self.xs), td(self.ys)
        self.z = torch.zeros(s, s, dtype=torch.bfloat16, device=dev)
        self.zp = ct.partition(self.z, [self.tile, self.tile])

    def launch(self):
        self.ct.linear_tile_mxfp8(self.zp, self.x, self.y, self.xsd, self.ysd, 1.0)

    def cpu_baseline(self, oracle, np, torch):
        rng = np.random.default_rng(11)
        rows = np.sort(rng.choice(self.s, size=128, replace=False)).astype(np.int64)
        t0 = time.perf_counter()
        ref = oracle.mx_gemm_f32(self.xq, self.yq, self.xs, self.ys, 1.0, rows=rows)
        dt = time.perf_counter() - t0
        got = self.z[torch.from_numpy(rows).to(self.z.device)].float().cpu().numpy()
        rel = float(np.linalg.norm(got - ref) / np.linalg.norm(ref))
        flops = 2.0 * len(rows) * self.s * self.s
        return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": oracle.num_threads(), "kind": "port",
                "sample": f"{len(rows)} of {self.s} output rows, f32 dequantised reference"}, \
               {"rel_l2_sampled_rows": rel, "tolerance": 3e-2, "ok": rel <= 3e-2}


class Nvfp4Gemm(Workload):
    name, unit, bound, peak_key = "nvfp4_gemm_8192", "TFLOP/s", "mfma", "mfma_bf16"
    dtype = "fp4 e2m1 x e4m3 scale per 16 K, expanded exactly to f16 / f32 acc / f32 out"
    s = 8192
    work = 2.0 * s ** 3
    tile = 256
    # Two roofs.  roofline.frac is against the f16 pipe this kernel computes on; frac_of_fp4_peak is the same rate
    # against the fp4 pipe's 10.1 PFLOP/s.  The exact path needs f16: an e4m3 scale per 16 elements has a mantissa,
    # the hardware block scale is a power of two per 32, and e2m1 x (1 + m/8) does not fit an fp8 operand.
    other_roofs = {"mfma_fp4": 10100.0}
    config = {"workload": "NVFP4 block-scaled GEMM A[8192,8192] B[8192,8192] packed e2m1 + e4m3fn scale per 16 K, f32 out; "
                          "matrix work runs on the f16 pipe (peak 2.5 PFLOP/s; the fp4 pipe's 10.1 PFLOP/s is quoted beside it): "
                          "CDNA4's fp4 pipe cannot take e4m3 scales per 16",
              "tile": "256x256x64"}

    def setup(self, ct, torch, oracle, dev):
        s = self.s
        self.ct = ct
        self.xq, self.xs = oracle.nvfp4_quantize(oracle.normal_f32((s, s), 14))
        self.yq, self.ys = oracle.nvfp4_quantize(oracle.normal_f32((s, s), 15))
        td = lambda t: torch.from_numpy(t).to(dev)
        self.x, self.y, self.xsd, self.ysd = td(self.xq), td(self.yq), td(self.xs), td(self.ys)
        self.z = torch.zeros(s, s, dtype=torch.float32, device=dev)
        self.zp = ct.partition(self.z, [self.tile, self.tile])

    def launch(self):
        self.ct.linear_tile_nvfp4(self.zp, self.x, self.y, self.xsd, self.ysd, 1.0)

    def cpu_baseline(self, oracle, np, torch):
        rng = np.random.default_rng(16)
        rows = np.sort(rng.choice(self.s, size=128, replace=False)).astype(np.int64)
        t0 = time.perf_counter()
        ref = oracle.nvfp4_gemm_f32(self.xq, self.yq, self.xs, self.ys, 1.0, rows=rows)
        dt = time.perf_counter() - t0
        got = self.z[torch.from_numpy(rows).to(self.z.device)].cpu().numpy()
        rel = float(np.linalg.norm(got - ref) / np.linalg.norm(ref))
        flops = 2.0 * len(rows) * self.s * self.s
        return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": oracle.num_threads(), "kind": "port",
                "sample": f"{len(rows)} of {self.s} output rows, f32 dequantised reference (includes dequantising B once)"}, \
               {"rel_l2_sampled_rows": rel, "tolerance": 1e-5, "ok": rel <= 1e-5}


def _td_f16(torch, np, bits, dev):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.float16)).to(dev)


def _f16_close(oracle, np, got_bits, ref_bits):
    """every element within one f16 ulp of the oracle (relative 2^-10, absolute 1e-7 near zero)"""
    g, r = oracle.f16_bits_to_f32(got_bits), oracle.f16_bits_to_f32(ref_bits)
    return bool(np.all(np.abs(g - r) <= np.abs(r) * 2 ** -10 + 1e-7))


class AddRmsNorm(Workload):
    name, unit, dtype = "add_rms_norm_f16_16384x8192", "GB/s", "f16 io / f32 math"
    m, n = 16384, 8192
    work = float(4 * m * n * 2 + n * 2)
    config = {"workload": "add_rms_norm fp16: residual + x [16384, 8192] -> normalised rows and the new residual, eps 1e-6"}

    def setup(self, ct, torch, oracle, dev):
        import numpy as np

        self.ct = ct
        self.rb = oracle.f32_to_f16_bits(oracle.normal_f32((self.m, self.n), 21))
        self.xb = oracle.f32_to_f16_bits(oracle.normal_f32((self.m, self.n), 22))
        self.wb = oracle.f32_to_f16_bits(oracle.uniform_f32(self.n, 23, 0.5, 1.5))
        self.r, self.x, self.w = (_td_f16(torch, np, t, dev) for t in (self.rb, self.xb, self.wb))
        self.o, self.ro = torch.empty_like(self.x), torch.empty_like(self.x)
        self.op, self.rop = ct.partition(self.o, [1, self.n]), ct.partition(self.ro, [1, self.n])

    def launch(self):
        self.ct.add_rms_norm_f16(self.r, self.x, self.w, self.op, self.rop, 1e-6)

    def cpu_baseline(self, oracle, np, torch):
        rows = 1024
        t0 = time.perf_counter()
        ref, res = oracle.add_rms_norm_f16(self.rb[:rows], self.xb[:rows], self.wb, 1e-6)
        dt = time.perf_counter() - t0
        ok = _f16_close(oracle, np, self.o[:rows].cpu().numpy().view(np.uint16), ref)
        exact = bool(np.array_equal(self.ro[:rows].cpu().numpy().view(np.uint16), res))
        return {"value": (4 * rows * self.n * 2) / dt / 1e9, "unit": "GB/s", "cores": oracle.num_threads(), "kind": "port",
                "sample": f"first {rows} of {self.m} rows"}, {"within_1_f16_ulp": ok, "residual_bit_exact": exact}


class SiluMul(Workload):
    name, unit, dtype = "silu_mul_f16_16384x8192", "GB/s", "f16 io / f32 math"
    m, n = 16384, 8192
    work = float(3 * m * n * 2)
    config = {"workload": "silu_mul_2d fp16: silu(gate) * up, [16384, 8192], tiles [1, 1024]"}

    def setup(self, ct, torch, oracle, dev):
        import numpy as np

        self.ct = ct
        self.gb = oracle.f32_to_f16_bits(oracle.normal_f32((self.m, self.n), 24))
        self.ub = oracle.f32_to_f16_bits(oracle.normal_f32((self.m, self.n), 25))
        self.g, self.u = _td_f16(torch, np, self.gb, dev), _td_f16(torch, np, self.ub, dev)
        self.o = torch.empty_like(self.g)
        self.op = ct.partition(self.o, [1, 1024])

    def launch(self):
        self.ct.silu_mul_2d_f16(self.op, self.g, self.u)

    def cpu_baseline(self, oracle, np, torch):
        rows = 2048
        t0 = time.perf_counter()
        ref = oracle.silu_mul_f16(self.gb[:rows], self.ub[:rows])
        dt = time.perf_counter() - t0
        ok = _f16_close(oracle, np, self.o[:rows].cpu().numpy().view(np.uint16), ref)
        return {"value": (3 * rows * self.n * 2) / dt / 1e9, "unit": "GB/s", "cores": oracle.num_threads(), "kind": "port",
                "sample": f"first {rows} of {self.m} rows"}, {"within_1_f16_ulp": ok}


class QkNorm(Workload):
    name, unit, dtype = "qk_norm_f16_655360x128", "GB/s", "f16 io / f32 math"
    tokens, qh, kh, d = 16384, 32, 8, 128
    work = float(2 * tokens * (qh + kh) * d * 2)
    config = {"workload": "qk_norm fp16: 16384 tokens x (32 q + 8 k) heads of 128, per-head RMSNorm with q/k weights, eps 1e-6"}

    def setup(self, ct, torch, oracle, dev):
        import numpy as np

        self.ct = ct
        self.qb = oracle.f32_to_f16_bits(oracle.normal_f32((self.tokens * self.qh, self.d), 26))
        self.kb = oracle.f32_to_f16_bits(oracle.normal_f32((self.tokens * self.kh, self.d), 27))
        self.qwb = oracle.f32_to_f16_bits(oracle.uniform_f32(self.d, 28, 0.5, 1.5))
        self.kwb = oracle.f32_to_f16_bits(oracle.uniform_f32(self.d, 29, 0.5, 1.5))
        self.q, self.k, self.qw, self.kw = (_td_f16(torch, np, t, dev) for t in (self.qb, self.kb, self.qwb, self.kwb))
        self.o = torch.empty(self.tokens * (self.qh + self.kh), self.d, dtype=torch.float16, device=dev)
        self.op = ct.partition(self.o, [1, self.d])

    def launch(self):
        self.ct.qk_norm_f16(self.q, self.k, self.qw, self.kw, self.op, 1e-6, self.tokens * self.qh)

    def cpu_baseline(self, oracle, np, torch):
        t0 = time.perf_counter()
        ref = oracle.qk_norm_f16(self.qb, self.kb, self.qwb, self.kwb, 1e-6)
        dt = time.perf_counter() - t0
        ok = _f16_close(oracle, np, self.o.cpu().numpy().view(np.uint16), ref)
        return {"value": self.work / dt / 1e9, "unit": "GB/s", "cores": oracle.num_threads(), "kind": "port",
                "sample": "full size"}, {"within_1_f16_ulp": ok}


class Rope(Workload):
    name, unit, dtype = "rope_f16_32768x32x128", "GB/s", "f16 io / f32 math"
    seq, heads, d = 32768, 32, 128
    work = float(2 * seq * heads * d * 2)
    config = {"workload": "rope_seq fp16: x [32768, 32, 128], inv_freq [64] (base 10000), start position 7"}

    def setup(self, ct, torch, oracle, dev):
        import numpy as np

        self.ct = ct
        self.xb = oracle.f32_to_f16_bits(oracle.normal_f32((self.seq, self.heads, self.d), 30))
        self.inv = (1.0 / 10000.0 ** (np.arange(self.d // 2) / (self.d // 2))).astype(np.float32)
        self.x, self.fr = _td_f16(torch, np, self.xb, dev), torch.from_numpy(self.inv).to(dev)
        self.o = torch.empty_like(self.x)
        self.op = ct.partition(self.o, [1, 1, self.d // 2])

    def launch(self):
        self.ct.rope_f16(self.op, self.x, self.fr, 7)

    def cpu_baseline(self, oracle, np, torch):
        rows = 1024
        t0 = time.perf_counter()
        ref = oracle.rope_seq_f16(self.xb[:rows], self.inv, 7)
        dt = time.perf_counter() - t0
        ok = _f16_close(oracle, np, self.o[:rows].cpu().numpy().view(np.uint16), ref)
        return {"value": (2 * rows * self.heads * self.d * 2) / dt / 1e9, "unit": "GB/s", "cores": oracle.num_threads(),
                "kind": "port", "sample": f"first {rows} of {self.seq} positions"}, {"within_1_f16_ulp": ok}


class KvCacheUpdate(Workload):
    name, unit, dtype = "kv_cache_update_f16_32768x8x128", "GB/s", "f16 (copy)"
    seq, heads, d, max_seq = 32768, 8, 128, 32768
    work = float(4 * seq * heads * d * 2)
    config = {"workload": "kv_cache_update_seq fp16 (prefill form): new K,V [32768, 8, 128] into caches [8, 32768, 128] at row 0"}

    def setup(self, ct, torch, oracle, dev):
        import numpy as np

        self.ct = ct
        self.nkb = oracle.f32_to_f16_bits(oracle.normal_f32((self.seq, self.heads, self.d), 31))
        self.nvb = oracle.f32_to_f16_bits(oracle.normal_f32((self.seq, self.heads, self.d), 32))
        self.nk, self.nv = _td_f16(torch, np, self.nkb, dev), _td_f16(torch, np, self.nvb, dev)
        self.kc = torch.zeros(self.heads, self.max_seq, self.d, dtype=torch.float16, device=dev)
        self.vc = torch.zeros_like(self.kc)
        self.kp, self.vp = ct.partition(self.kc, [1, 16, self.d]), ct.partition(self.vc, [1, 16, self.d])

    def launch(self):
        self.ct.kv_cache_update_f16(self.nk, self.nv, self.kp, self.vp, 0, self.seq)

    def cpu_baseline(self, oracle, np, torch):
        zero = np.zeros((self.heads, self.max_seq, self.d), np.uint16)
        t0 = time.perf_counter()
        k_ref, v_ref = oracle.kv_cache_update_f16(self.nkb, self.nvb, zero, zero, 0, self.seq)
        dt = time.perf_counter() - t0
        exact = bool(np.array_equal(self.kc.cpu().numpy().view(np.uint16), k_ref) and
                     np.array_equal(self.vc.cpu().numpy().view(np.uint16), v_ref))
        return {"value": self.work / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port", "sample": "full size"}, \
               {"bit_exact": exact}


class DecodeAttention(Workload):
    name, unit, dtype = "decode_gqa_f16_h8g4d128_s131072", "GB/s", "f16 io / f32 softmax+acc"
    heads, group, d, s, splits, bn = 8, 4, 128, 131072, 32, 64
    work = float(2 * heads * s * d * 2)          # every K and V byte once; q, partials and out are < 0.2 %
    config = {"workload": "decode attention fp16: fmha_decode_gqa_split + splitk_reduce_merge, 8 KV heads x GROUP 4, D 128, "
                          "131072 cached keys, 32 KV splits (one workgroup per CU), BN 64 (two launches per step)"}

    def setup(self, ct, torch, oracle, dev):
        import numpy as np

        self.ct = ct
        self.qb = oracle.f32_to_f16_bits(oracle.normal_f32((self.heads, self.group, self.d), 33))
        self.kb = oracle.f32_to_f16_bits(oracle.normal_f32((self.heads, self.s, self.d), 34))
        self.vb = oracle.f32_to_f16_bits(oracle.normal_f32((self.heads, self.s, self.d), 35))
        self.q, self.k, self.v = (_td_f16(torch, np, t, dev) for t in (self.qb, self.kb, self.vb))
        self.att = torch.empty(self.heads, self.splits * self.group, self.d, dtype=torch.float16, device=dev)
        self.lse = torch.empty(self.heads, self.splits * self.group, dtype=torch.float32, device=dev)
        self.o = torch.empty(self.heads, self.group, self.d, dtype=torch.float16, device=dev)
        self.pos = torch.tensor([self.s - 1], dtype=torch.int32, device=dev)
        self.ap, self.lp = ct.partition(self.att, [1, self.group, self.d]), ct.partition(self.lse, [1, self.group])
        self.op = ct.partition(self.o, [1, self.group, self.d])
        self.scale = float(np.float16(self.d ** -0.5))

    def launch_dominant(self):
        self.ct.fmha_decode_gqa_split(self.q, self.k, self.v, self.ap, self.lp, self.scale, self.pos,
                                      generics=[self.group, self.bn, self.d, self.splits])

    def launch(self):
        self.launch_dominant()
        self.ct.splitk_reduce_merge(self.att, self.lse, self.op)

    def cpu_baseline(self, oracle, np, torch):
        t0 = time.perf_counter()
        att, lse = oracle.fmha_decode_gqa_split(self.qb, self.kb, self.vb, self.scale, self.s - 1, self.bn, self.splits)
        ref = oracle.splitk_reduce_merge(att, lse, self.group)
        dt = time.perf_counter() - t0
        got = oracle.f16_bits_to_f32(self.o.cpu().numpy().view(np.uint16))
        err = float(np.max(np.abs(got - oracle.f16_bits_to_f32(ref))))
        return {"value": self.work / dt / 1e9, "unit": "GB/s", "cores": oracle.num_threads(), "kind": "port",
                "sample": "full size"}, {"max_abs": err, "tolerance": 2e-2, "ok": err <= 2e-2}


class DecodeAttentionWide(DecodeAttention):
    """GROUP 8: the split kernel runs on the matrix cores (heads are the N dimension of a 16x16x32 MFMA)."""
    name = "decode_gqa_f16_h8g8d128_s131072"
    group, splits = 8, 32
    config = {"workload": "decode attention fp16: fmha_decode_gqa_split + splitk_reduce_merge, 8 KV heads x GROUP 8, D 128, "
                          "131072 cached keys, 32 KV splits (one workgroup per CU), BN 64 (two launches per step)"}


class DecodeAttentionGrouped(Workload):
    """attention_decode_kernel_grouped (cutile-kernels/src/experimental/attention.rs:385-846): the split-KV decode partial
    over a batch of sequences; every cached K and V byte is read once."""
    name, unit, dtype = "decode_grouped_f16_b8h8g4d128_s16384", "GB/s", "f16 io / f32 softmax+acc"
    batch, heads, group, d, s, splits, tile_n = 8, 8, 4, 128, 16384, 4, 64
    work = float(2 * batch * heads * s * d * 2)
    config = {"workload": "attention_decode_kernel_grouped fp16: batch 8 x 8 KV heads x GROUP 4, D 128, 16384 cached keys each, "
                          "4 KV splits of 4096 keys (one workgroup per CU), TILE_N 64"}

    def setup(self, ct, torch, oracle, dev):
        import numpy as np

        self.ct = ct
        bits = lambda shape, seed: oracle.f32_to_f16_bits(oracle.normal_f32(shape, seed))
        self.qb = bits((self.batch, self.heads, self.group, self.d), 91)
        self.kb, self.vb = bits((self.batch, self.heads, self.s, self.d), 92), bits((self.batch, self.heads, self.s, self.d), 93)
        self.q, self.k, self.v = (_td_f16(torch, np, t, dev) for t in (self.qb, self.kb, self.vb))
        self.att = torch.empty(self.batch, self.heads, self.group, self.splits, self.d, dtype=torch.float16, device=dev)
        self.lse = torch.empty(self.batch, self.heads, self.group, self.splits, dtype=torch.float32, device=dev)
        self.count = torch.tensor([self.s], dtype=torch.int32, device=dev)
        self.scale = float(np.float16(self.d ** -0.5))

    def launch(self):
        self.ct.attention_decode_kernel_grouped_f16(self.q, self.k, self.v, self.att, self.lse, self.scale, self.count,
                                                    tile_n=self.tile_n, kv_len_per_split=self.s // self.splits,
                                                    query_group_tile_size=16)

    def cpu_baseline(self, oracle, np, torch):
        nb = 2                                   # the first two sequences of the batch: independent sub-problems
        t0 = time.perf_counter()
        att, lse = oracle.attention_decode_grouped_f16(self.qb[:nb], self.kb[:nb], self.vb[:nb], self.scale, self.s, self.tile_n,
                                                       self.s // self.splits, self.splits)
        dt = time.perf_counter() - t0
        got = oracle.f16_bits_to_f32(self.att[:nb].cpu().numpy().view(np.uint16))
        err = float(np.max(np.abs(got - oracle.f16_bits_to_f32(att))))
        err_lse = float(np.max(np.abs(self.lse[:nb].cpu().numpy() - lse)))
        return {"value": self.work * nb / self.batch / dt / 1e9, "unit": "GB/s", "cores": oracle.num_threads(), "kind": "port",
                "sample": f"the first {nb} of {self.batch} sequences"}, \
               {"max_abs": err, "max_abs_lse": err_lse, "tolerance": 2e-2, "ok": err <= 2e-2 and err_lse <= 2e-3}


class KvbmCopy(Workload):
    """copy_stacked_to_contiguous_f16 (cutile-kernels/src/experimental/kvbm.rs:112-187): per-layer NHD chunks gathered into
    universal blocks [nh, nl, no, nt, hd] through pointer tables; every element is read once and written once."""
    name, unit, dtype = "kvbm_stacked_nhd_to_universal_f16_256x4MiB", "GB/s", "f16 (layout conversion)"
    blocks, nh, nl, no, nt, hd = 256, 8, 32, 2, 32, 128
    work = 2.0 * blocks * nh * nl * no * nt * hd * 2
    config = {"workload": "copy_stacked_to_contiguous fp16: 256 blocks x (8 heads, 32 layers, K and V, 32 tokens, 128), 16384 stacked "
                          "NHD chunks of 64 KiB -> 256 universal blocks of 4 MiB"}

    def setup(self, ct, torch, oracle, dev):
        import numpy as np

        self.ct, self.np = ct, np
        per_chunk = self.nt * self.nh * self.hd
        n_chunks = self.blocks * self.nl * self.no
        rng = np.random.default_rng(97)
        self.host = rng.integers(0, 65536, (n_chunks, per_chunk), dtype=np.uint16)
        self.stacked = torch.from_numpy(self.host.view(np.int16)).to(dev).view(torch.float16)
        self.out = torch.zeros(self.blocks, self.nh * self.nl * self.no * self.nt * self.hd, dtype=torch.float16, device=dev)
        base, step = self.stacked.data_ptr(), per_chunk * 2
        self.s_table = torch.tensor([base + c * step for c in range(n_chunks)], dtype=torch.int64, device=dev)
        self.c_table = torch.tensor([self.out[b].data_ptr() for b in range(self.blocks)], dtype=torch.int64, device=dev)

    def launch(self):
        self.ct.kvbm_copy_f16(False, self.ct.KVBM_STACKED_NHD, self.ct.KVBM_UNIVERSAL, self.blocks, self.s_table, self.c_table,
                              self.nh, self.nl, self.no, self.nt, self.hd)

    def cpu_baseline(self, oracle, np, torch):
        nb = 32
        st = self.host[: nb * self.nl * self.no].reshape(nb, self.nl, self.no, self.nt, self.nh, self.hd)
        t0 = time.perf_counter()
        ref = oracle.kvbm_stacked_to_contiguous(st, "nhd", "universal")
        dt = time.perf_counter() - t0
        got = self.out[:nb].cpu().numpy().view(np.uint16).reshape(ref.shape)
        same = bool(np.array_equal(got, ref))
        return {"value": self.work * nb / self.blocks / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"the first {nb} of {self.blocks} blocks (numpy transpose)"}, {"bit_exact": same, "ok": same}


class PrefillAttention(Workload):
    """fmha_prefill_causal (cutile-kernels/src/attention.rs:242-391): f16, [seq, heads, D] queries against a
    [kv_heads, seq, D] cache, grouped heads; flops counted like the causal FMHA bench (half of 4 s^2 d per head)."""
    name, unit, bound, peak_key = "prefill_attention_f16_s8192_h32g4_d128", "TFLOP/s", "mfma", "mfma_bf16"
    dtype = "f16 io / f32 softmax+acc"
    s, heads, group, d = 8192, 32, 4, 128
    work = 2.0 * s * s * d * heads
    config = {"workload": "fmha_prefill_causal fp16: q [8192, 32, 128], k/v [8, 8192, 128] (GROUP 4), causal, query_start 0, "
                          "scale 1/sqrt(128)", "tile": "BM=256"}

    def setup(self, ct, torch, oracle, dev):
        import numpy as np

        self.ct = ct
        kvh = self.heads // self.group
        f16 = lambda a: a.astype(np.float16)
        self.qh = f16(oracle.normal_f32((self.s, self.heads, self.d), 41))
        self.kh, self.vh = f16(oracle.normal_f32((kvh, self.s, self.d), 42)), f16(oracle.normal_f32((kvh, self.s, self.d), 43))
        self.q, self.k, self.v = (torch.from_numpy(t).to(dev) for t in (self.qh, self.kh, self.vh))
        self.o = torch.zeros(self.s, self.heads, self.d, dtype=torch.float16, device=dev)
        self.op = ct.partition(self.o, [128, 1, self.d])

    def launch(self):
        self.ct.fmha_seq_f16(self.q, self.k, self.v, self.op, self.d ** -0.5, self.group, kv_len=self.s, query_start=0, causal=True)

    def cpu_baseline(self, oracle, np, torch):
        # the first 1024 queries of the same problem see the first 1024 keys only: a self-contained sub-problem
        n = 1024
        q, k, v = self.qh[:n].astype(np.float32), self.kh[:, :n].astype(np.float32), self.vh[:, :n].astype(np.float32)
        t0 = time.perf_counter()
        ref = oracle.attention_seq_ref(q, k, v, self.d ** -0.5, self.group, n, 0, True)
        dt = time.perf_counter() - t0
        err = float(np.max(np.abs(self.o[:n].float().cpu().numpy() - ref)))
        flops = 2.0 * n * n * self.d * self.heads
        return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": oracle.num_threads(), "kind": "port",
                "sample": f"the first {n} of {self.s} queries (they see the first {n} keys only)"}, \
               {"max_abs": err, "tolerance": 2e-2, "ok": err <= 2e-2}


class FusedQkNormRopeKv(Workload):
    """qk_norm_rope_kv_prefill_raw_f16 (cutile-kernels/src/experimental/fused_transformer.rs:22-345): Q/K norm, rotary
    embedding and KV-cache update in one pass; every q, k, v element is read once and written once."""
    name, unit, dtype = "qk_norm_rope_kv_f16_32768x48x128", "GB/s", "f16 io / f32 math"
    seq, nq, nkv, d = 32768, 32, 8, 128
    work = 4.0 * seq * (nq + 2 * nkv) * d
    config = {"workload": "qk_norm_rope_kv_prefill_raw fp16: 32768 positions x (32 q + 8 k + 8 v heads) x 128, caches [8, 32768, 128]"}

    def setup(self, ct, torch, oracle, dev):
        import numpy as np

        self.ct = ct
        f16 = lambda shape, seed: oracle.f32_to_f16_bits(oracle.normal_f32(shape, seed))
        self.qb, self.kb, self.vb = f16((self.seq, self.nq, self.d), 71), f16((self.seq, self.nkv, self.d), 72), f16((self.seq, self.nkv, self.d), 73)
        self.qwb = oracle.f32_to_f16_bits(oracle.uniform_f32(self.d, 74, 0.5, 1.5))
        self.kwb = oracle.f32_to_f16_bits(oracle.uniform_f32(self.d, 75, 0.5, 1.5))
        self.inv = (1.0 / 10000.0 ** (np.arange(self.d // 2) / (self.d // 2))).astype(np.float32)
        td = lambda bits: torch.from_numpy(bits.view(np.int16)).to(dev).view(torch.float16)
        self.q, self.k, self.v, self.qw, self.kw = td(self.qb), td(self.kb), td(self.vb), td(self.qwb), td(self.kwb)
        self.invd = torch.from_numpy(self.inv).to(dev)
        self.qo = torch.zeros_like(self.q)
        self.kc = torch.zeros(self.nkv, self.seq, self.d, dtype=torch.float16, device=dev)
        self.vc = torch.zeros_like(self.kc)

    def launch(self):
        self.ct.qk_norm_rope_kv_prefill_raw_f16(self.q, self.k, self.v, self.qw, self.kw, self.invd, self.qo, self.kc, self.vc, 1e-6, 0, self.seq)

    def cpu_baseline(self, oracle, np, torch):
        n = 2048
        kc0 = np.zeros((self.nkv, n, self.d), np.uint16)
        t0 = time.perf_counter()
        rq, rk, rv = oracle.qk_norm_rope_kv_f16(self.qb[:n], self.kb[:n], self.vb[:n], self.qwb, self.kwb, self.inv, kc0, kc0, 1e-6, 0)
        dt = time.perf_counter() - t0
        bits = lambda t: t.cpu().numpy().view(np.uint16)
        f = oracle.f16_bits_to_f32
        err = max(float(np.max(np.abs(f(bits(self.qo[:n])) - f(rq)))), float(np.max(np.abs(f(bits(self.kc[:, :n])) - f(rk)))))
        exact = bool(np.array_equal(bits(self.vc[:, :n]), rv))
        return {"value": 4.0 * n * (self.nq + 2 * self.nkv) * self.d / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"first {n} of {self.seq} positions"}, {"max_abs": err, "tolerance": 4e-3, "ok": err <= 4e-3 and exact, "v_bit_exact": exact}


class GroupGemm(Workload):
    """group_gemm_f16_nt_desc (cutile-kernels/src/experimental/moe.rs:67-128): expert batches of unequal size, one launch."""
    name, unit, bound, peak_key = "group_gemm_f16_32x4096x4096", "TFLOP/s", "mfma", "mfma_bf16"
    dtype = "f16 in / f32 acc / f16 out"
    groups, n, k = 32, 4096, 4096
    rows = [256 + 96 * ((7 * g) % 17) for g in range(32)]                 # 256 .. 1792 tokens per expert, multiples of 16
    work = 2.0 * sum(rows) * n * k
    config = {"workload": f"group_gemm_f16_nt_desc fp16: 32 groups, A_g [256..1792 rows ({sum(rows)} in all), 4096] x B_g [4096, 4096], "
                          "descriptor tables in device memory, 256 persistent tile blocks", "tile": "256x256x64"}

    def setup(self, ct, torch, oracle, dev):
        import numpy as np

        self.ct = ct
        self.ab = [oracle.f32_to_f16_bits(oracle.normal_f32((m, self.k), 60 + g, 0, self.k ** -0.5)) for g, m in enumerate(self.rows)]
        self.bb = oracle.f32_to_f16_bits(oracle.normal_f32((self.k, self.n), 59, 0, self.k ** -0.5))
        td = lambda bits: torch.from_numpy(bits.view(np.int16)).to(dev).view(torch.float16)
        self.a = [td(b) for b in self.ab]
        self.b = [td(self.bb) if g == 0 else td(self.bb).clone() for g in range(self.groups)]   # one weight matrix per expert
        self.c = [torch.zeros(m, self.n, dtype=torch.float16, device=dev) for m in self.rows]

        def tables(ts):
            ptrs = torch.tensor([t.data_ptr() for t in ts], dtype=torch.int64, device=dev)
            metas = torch.zeros(len(ts), 8, dtype=torch.int32)
            for i, t in enumerate(ts):
                metas[i, 0], metas[i, 1], metas[i, 2] = t.shape[0], t.shape[1], t.stride(0)
            return ptrs, metas.to(dev)
        self.tabs = tables(self.a) + tables(self.b) + tables(self.c)

    def launch(self):
        ap, am, bp, bm, cp, cm = self.tabs
        self.ct.group_gemm_f16_nt_desc(ap, bp, cp, am, bm, cm, self.groups, generics=[256, 256, 64, 256])

    def cpu_baseline(self, oracle, np, torch):
        g, rows = 5, 128
        x = oracle.f16_bits_to_f32(self.ab[g][:rows])
        t0 = time.perf_counter()
        ref = oracle.cpu_gemm_f32(x, oracle.f16_bits_to_f32(self.bb))
        dt = time.perf_counter() - t0
        got = self.c[g][:rows].float().cpu().numpy()
        rel = float(np.linalg.norm(got - ref) / np.linalg.norm(ref))
        return {"value": 2.0 * rows * self.n * self.k / dt / 1e12, "unit": "TFLOP/s", "cores": oracle.num_threads(), "kind": "port",
                "sample": f"the first {rows} rows of group {g} (naive f32 loop)"}, \
               {"rel_l2_sampled_rows": rel, "tolerance": 1e-2, "ok": rel <= 1e-2}


class LmHeadArgmax(Workload):
    """lm_head_argmax_blocks_f16 + argmax_reduce_blocks_to_u32 (cutile-kernels/src/argmax.rs:88-158, 173-213): the greedy
    token of one decode step; the weights stream through once, the logits are never stored."""
    name, unit, dtype = "lm_head_argmax_f16_128256x4096", "GB/s", "f16 io / f32 accumulate"
    vocab, k = 128256, 4096
    work = 2.0 * vocab * k + 2.0 * k + 8.0 * (vocab // 64)
    config = {"workload": "lm_head_argmax_blocks fp16: weights [128256, 4096], hidden [1, 4096], 2004 blocks of 64 rows, then "
                          "argmax_reduce_blocks_to_u32 (two launches per step)"}

    def setup(self, ct, torch, oracle, dev):
        import numpy as np

        self.ct = ct
        self.wb = oracle.f32_to_f16_bits(oracle.normal_f32((self.vocab, self.k), 51))
        self.hb = oracle.f32_to_f16_bits(oracle.normal_f32(self.k, 52))
        td = lambda bits: torch.from_numpy(bits.view(np.int16)).to(dev).view(torch.float16)
        self.w, self.h = td(self.wb), td(self.hb.reshape(1, self.k))
        self.nb = self.vocab // 64
        self.bm = torch.zeros(self.nb, device=dev)
        self.bi = torch.zeros(self.nb, dtype=torch.int32, device=dev)
        self.out = torch.zeros(1, dtype=torch.int32, device=dev)
        self.bmp, self.bip, self.outp = ct.partition(self.bm, [1]), ct.partition(self.bi, [1]), ct.partition(self.out, [1])

    def launch_dominant(self):
        self.ct.lm_head_argmax_blocks_f16(self.w, self.h, self.bmp, self.bip, self.vocab)

    def launch(self):
        self.launch_dominant()
        self.ct.argmax_reduce_blocks_to_u32(self.bm, self.bi, self.outp, self.nb)

    def cpu_baseline(self, oracle, np, torch):
        t0 = time.perf_counter()
        rm, ri = oracle.lm_head_argmax_blocks_f16(self.wb, self.hb, self.vocab)
        want = oracle.argmax_reduce_blocks_to_u32(rm, ri, self.nb)
        dt = time.perf_counter() - t0
        got = int(self.out.item())
        same_blocks = float(np.mean(self.bi.cpu().numpy().view(np.uint32) == ri))
        return {"value": self.work / dt / 1e9, "unit": "GB/s", "cores": oracle.num_threads(), "kind": "port", "sample": "full size"}, \
               {"token": got, "oracle_token": want, "ok": got == want, "blocks_with_the_same_index": same_blocks,
                "max_abs_block_max": float(np.max(np.abs(self.bm.cpu().numpy() - rm)))}


class EmbeddingBatch(Workload):
    """embedding_batch_f16 (cutile-kernels/src/embeddings.rs:21-41): one table row per token."""
    name, unit, dtype = "embedding_batch_f16_32768x4096", "GB/s", "f16 (gather)"
    tokens, vocab, d = 32768, 128256, 4096
    work = 4.0 * tokens * d + 4.0 * tokens
    config = {"workload": "embedding_batch fp16: 32768 token ids into a [128256, 4096] table, out [32768, 4096] tiles [1, 1024]"}

    def setup(self, ct, torch, oracle, dev):
        import numpy as np

        self.ct = ct
        self.tb = oracle.f32_to_f16_bits(oracle.normal_f32((self.vocab, self.d), 53))
        self.ids = (np.random.default_rng(54).integers(0, self.vocab, self.tokens)).astype(np.uint32)
        self.table = torch.from_numpy(self.tb.view(np.int16)).to(dev).view(torch.float16)
        self.idd = torch.from_numpy(self.ids.view(np.int32)).to(dev)
        self.out = torch.zeros(self.tokens, self.d, dtype=torch.float16, device=dev)
        self.op = ct.partition(self.out, [1, 1024])

    def launch(self):
        self.ct.embedding_batch_f16(self.idd, self.table, self.op)

    def cpu_baseline(self, oracle, np, torch):
        t0 = time.perf_counter()
        ref = oracle.embedding_batch_f16(self.ids, self.tb)
        dt = time.perf_counter() - t0
        exact = bool(np.array_equal(self.out.cpu().numpy().view(np.uint16), ref))
        return {"value": self.work / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port", "sample": "full size"}, {"bit_exact": exact}


class BatchMatmul(Workload):
    """batch_matmul (cutile-examples/examples/batch_matmul.rs:16-44) at a size that fills the chip: 16 batches of 2048^3."""
    name, unit, dtype, bound, peak_key = "batch_matmul_bf16_16x2048x2048x2048", "TFLOP/s", "bf16 in / f32 acc / bf16 out", "mfma", "mfma_bf16"
    batch, s = 16, 2048
    work = 2.0 * batch * s ** 3
    config = {"workload": "batch_matmul bf16: 16 batches of M=N=K=2048, c[p] = a[p]·b[p], entries ~ N(0,1)/sqrt(K), tiles [1, 256, 256]",
              "tile": "256x256x64"}

    def setup(self, ct, torch, oracle, dev):
        import numpy as np

        self.ct = ct
        b, s = self.batch, self.s
        self.ab = oracle.f32_to_bf16_bits(oracle.normal_f32((b, s, s), 61, 0, s ** -0.5))
        self.bb = oracle.f32_to_bf16_bits(oracle.normal_f32((b, s, s), 62, 0, s ** -0.5))
        self.a, self.b = _td_bf16(torch, np, self.ab, dev), _td_bf16(torch, np, self.bb, dev)
        self.c = torch.zeros(b, s, s, dtype=torch.bfloat16, device=dev)
        self.cp = ct.partition(self.c, [1, 256, 256])

    def launch(self):
        self.ct.batch_matmul(self.cp, self.a, self.b, self.s)

    def cpu_baseline(self, oracle, np, torch):
        rows = np.arange(0, self.s, 16, dtype=np.int64)          # 128 rows of every batch
        t0 = time.perf_counter()
        ref = np.stack([oracle.gemm_bf16(self.ab[i], self.bb[i], rows=rows, f32out=True) for i in range(self.batch)])
        dt = time.perf_counter() - t0
        got = self.c[:, ::16].float().cpu().numpy()
        rel = float(np.linalg.norm(got - ref) / np.linalg.norm(ref))
        flops = 2.0 * self.batch * len(rows) * self.s * self.s
        return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": oracle.num_threads(), "kind": "port",
                "sample": f"{len(rows)} of {self.s} output rows of every batch (naive f32 loop)"}, \
               {"rel_l2_sampled_rows": rel, "tolerance": 1e-2, "ok": rel <= 1e-2}


class Matvec(Workload):
    """matvec (cutile-examples/examples/async_mlp.rs:38-54): the matrix is the stream."""
    name, unit, dtype = "matvec_f32_16384x16384", "GB/s", "f32"
    m = k = 16384
    work = 4.0 * m * k + 4.0 * k + 8.0 * m
    config = {"workload": "matvec fp32: z[16384] += x[16384, 16384] · y[16384], tiles of 64 rows"}

    def setup(self, ct, torch, oracle, dev):
        self.ct = ct
        self.xh, self.yh = oracle.normal_f32((self.m, self.k), 63), oracle.normal_f32(self.k, 64, 0, self.k ** -0.5)
        self.x, self.y = torch.from_numpy(self.xh).to(dev), torch.from_numpy(self.yh).to(dev)
        self.z = torch.zeros(self.m, device=dev)
        self.zp = ct.partition(self.z, [64])

    def launch(self):
        self.ct.matvec(self.zp, self.x, self.y, self.k)

    def cpu_baseline(self, oracle, np, torch):
        self.z.zero_()          # the timed launches accumulated into z: one launch from zero for the comparison
        self.launch()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ref = oracle.matvec_f32(np.zeros(self.m, np.float32), self.xh, self.yh)
        dt = time.perf_counter() - t0
        mag = np.abs(self.xh).astype(np.float64) @ np.abs(self.yh).astype(np.float64)
        err = np.abs(self.z.cpu().numpy().astype(np.float64) - ref)
        return {"value": self.work / dt / 1e9, "unit": "GB/s", "cores": oracle.num_threads(), "kind": "port", "sample": "full size"}, \
               {"max_err_over_sum_of_magnitudes": float((err / mag).max()), "tolerance": 1e-5, "ok": bool((err <= 1e-5 * mag).all())}


class ExampleStream(Workload):
    """relu / dropout / scale_ptr of the example programs on 2^26 f32: one read and one write per element."""
    unit, dtype = "GB/s", "f32"
    n = 1 << 26
    work = 8.0 * n

    def __init__(self, kind):
        self.kind = kind
        self.name = f"{kind}_f32_{self.n}"
        what = {"relu": "relu in place (async_mlp.rs:56-61), tiles of 1024", "dropout": "dropout p = 0.4 (dropout.rs:17-32), tiles of 1024",
                "scale_ptr": "scale_ptr on raw pointers, scale 3 (scale_ptr.rs:26-80), grid (1024, 1, 1)"}[kind]
        self.config = {"workload": f"{what}, n = 2^26 f32"}

    def setup(self, ct, torch, oracle, dev):
        self.ct = ct
        self.xh = oracle.uniform_f32(self.n, 65, 0.0, 1.0) if self.kind == "dropout" else oracle.normal_f32(self.n, 65)
        self.x = torch.from_numpy(self.xh).to(dev)
        self.out = self.x.clone() if self.kind == "relu" else torch.empty_like(self.x)
        self.op = ct.partition(self.out, [1024])

    def launch(self):
        if self.kind == "relu":
            self.ct.relu(self.op)
        elif self.kind == "dropout":
            self.ct.dropout(0.4, self.x, self.x, self.op)
        else:
            self.ct.scale_ptr(self.out.data_ptr(), self.x.data_ptr(), 3.0, self.n, grid=(1024, 1, 1))

    def cpu_baseline(self, oracle, np, torch):
        t0 = time.perf_counter()
        ref = {"relu": lambda: oracle.relu_f32(self.xh), "dropout": lambda: oracle.dropout_f32(0.4, self.xh),
               "scale_ptr": lambda: oracle.scale_f32(self.xh, 3.0)}[self.kind]()
        dt = time.perf_counter() - t0
        exact = bool(np.array_equal(self.out.cpu().numpy(), ref))
        return {"value": self.work / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port", "sample": "full size (numpy)"}, {"bit_exact": exact}


def make_workloads():
    """The default run: the benchmark configurations first, then the other kernels of the path."""
    return [Gemm(8192), Gemm(4096), GemmPersistent(8192), Fmha(False), Fmha(True), RmsNorm(), Softmax(), Saxpy(), MxGemm(), Nvfp4Gemm(),
            Copy(), RmsNormAllF16(), SoftmaxAllF16(), AddRmsNorm(), SiluMul(), QkNorm(), Rope(), KvCacheUpdate(), DecodeAttention(), DecodeAttentionWide(), DecodeAttentionGrouped(), KvbmCopy(), PrefillAttention(), LmHeadArgmax(), EmbeddingBatch(), GroupGemm(), FusedQkNormRopeKv()]


# the reference's small example programs: only by name (--workload), never in the default run
def make_extra_workloads():
    # the example programs, and the GEMM at M = N = 8192 over a range of K with and without the accumulator read: the
    # slope over K is the cost of a K tile, the intercept what a launch costs whatever its K
    scan = [Gemm(8192, k, acc) for k in (1024, 2048, 4096) for acc in (True, False)] + [Gemm(8192, None, False)]
    return [BatchMatmul(), Matvec(), ExampleStream("relu"), ExampleStream("dropout"), ExampleStream("scale_ptr")] + scan


WARMUP_BUDGET_S = 0.05       # untimed launches continue until this much time has passed (the reference's budget is 25 ms)
FLUSH_BYTES = 512 << 20      # larger than the 256 MB memory-side cache and every L2


def _quantile(sorted_vals, q):
    """linear interpolation between closest ranks, as cutile::bench::quantile (cutile/src/bench.rs:266-291)"""
    if not sorted_vals:
        return float("nan")
    pos = q * (len(sorted_vals) - 1)
    lo = int(pos)
    hi = min(lo + 1, len(sorted_vals) - 1)
    return sorted_vals[lo] + (sorted_vals[hi] - sorted_vals[lo]) * (pos - lo)


def measure(w, ct, torch, steps, warmup, with_cpu, oracle, np, flush):
    """Two protocols on the same launches.

    ms_per_step / value: W untimed launches, then exactly K launches back to back between two device
    synchronisations (wall clock; launch overhead included).

    roofline: the reference's do_bench protocol (cutile/src/bench.rs:124-211) on the dominant kernel: before every
    repetition the caches are flushed by zero-filling a 512 MiB buffer, the launch is bracketed by its own pair of
    HIP events on the launch stream, and the median of the repetitions gives roofline.achieved (minimum, mean and the
    back-to-back average of K launches between one event pair are reported beside it)."""
    for _ in range(warmup):
        w.launch()
    torch.cuda.synchronize()
    # Warm-up by time budget on top of the W steps, as do_bench has it ("absorbs JIT and clock ramp",
    # cutile/src/bench.rs:33-35,188-192): after tens of milliseconds without work this device needs about 30 ms of
    # launches before they run at their steady rate (a launch of the 8192^3 GEMM takes 0.9-1.07 ms there, 0.77 ms after),
    # and W = 5 launches of a 0.8 ms kernel end well inside that ramp.
    t_w = time.perf_counter()
    while time.perf_counter() - t_w < WARMUP_BUDGET_S:
        for _ in range(4):
            w.launch()
        torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        w.launch()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    # roofline: the dominant kernel alone where a step is more than one launch
    dominant = getattr(w, "launch_dominant", w.launch)
    timer = ct.EventTimer()
    timer.start()
    for _ in range(steps):
        dominant()
    back_to_back_ms = timer.stop() / steps
    # the same sustained run once more with an event between every two launches: shows whether the launches of a
    # back-to-back run slow down as the run goes on (clock management) or the first ones are slow (ramp from idle)
    series = ct.EventSeries(steps)
    series.mark()
    for _ in range(steps):
        dominant()
        series.mark()
    gaps = series.gaps_ms()
    series.close()
    reps = max(10, min(steps, 40))
    times = []
    for _ in range(reps):
        flush.zero_()
        timer.start()
        dominant()
        times.append(timer.stop())
    timer.close()
    times.sort()
    kernel_ms = _quantile(times, 0.5)
    scale = 1e9 if w.unit == "GB/s" else 1e12
    peak, punit = PEAK[w.peak_key]
    achieved = w.work / (kernel_ms * 1e-3) / scale
    rec = {
        "workload": w.name, "value": w.work / (wall_ms * 1e-3) / scale, "unit": w.unit, "ms_per_step": wall_ms,
        "dtype": w.dtype, "config": w.config,
        "roofline": {"bound": w.bound, "achieved": achieved, "peak": peak, "unit": punit, "frac": achieved / peak,
                     "traffic": _traffic(w.name), "traffic_source": "profiles/traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE)",
                     "kernel_ms": kernel_ms, "kernel_ms_min": times[0], "kernel_ms_mean": sum(times) / len(times),
                     "kernel_ms_back_to_back": back_to_back_ms, "frac_back_to_back": w.work / (back_to_back_ms * 1e-3) / scale / peak,
                     "frac_wall": w.work / (wall_ms * 1e-3) / scale / peak,
                     "sustained_launch_ms": {"first": gaps[0], "median": _quantile(sorted(gaps), 0.5), "last": gaps[-1], "max": max(gaps)},
                     "reps": reps,
                     "protocol": "median of per-launch HIP-event times, 512 MiB cache flush before each",
                     "algorithmic_work": w.work},
    }
    for key, other_peak in getattr(w, "other_roofs", {}).items():      # the same rate against a second published peak
        rec["roofline"]["frac_of_" + key.replace("mfma_", "") + "_peak"] = achieved / other_peak
        rec["roofline"]["peak_" + key.replace("mfma_", "")] = other_peak
    try:      # which precompiled variant ran, and whether a tuning record, a pin or the table's order chose it
        got = ct.last_resolved()
        rec["kernel"] = {"variant": got["variant"], "chosen_by": got["source"], "shape_class": got["bucket"]}
    except ct.CutileError:
        pass
    if with_cpu:
        res = w.cpu_baseline(oracle, np, torch)
        if res:
            rec["cpu_baseline"], rec["parity"] = res
    return rec


def library_same_box(torch, flush, reps=20):
    """Informational only (never on the product path): the vendor library's bf16 GEMM at 8192^3 through torch.matmul
    (no read of z), timed with the same flush + event protocol; the figure the power-cap argument is made against."""
    s = 8192
    a = torch.randn(s, s, device="cuda", dtype=torch.float32).mul_(s ** -0.5).to(torch.bfloat16)
    b = torch.randn(s, s, device="cuda", dtype=torch.float32).mul_(s ** -0.5).to(torch.bfloat16)
    for _ in range(5):
        torch.matmul(a, b)
    torch.cuda.synchronize()
    times = []
    for _ in range(reps):
        flush.zero_()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        torch.matmul(a, b)
        e1.record()
        e1.synchronize()
        times.append(e0.elapsed_time(e1))
    times.sort()
    med = _quantile(times, 0.5)
    return {"what": "torch.matmul bf16 8192^3 (hipBLASLt), z = A·B", "kernel_ms": med, "kernel_ms_min": times[0],
            "tflops": 2.0 * s ** 3 / (med * 1e-3) / 1e12, "frac_of_2500": 2.0 * s ** 3 / (med * 1e-3) / 1e12 / 2500.0}


def _timed(ct, torch, flush, launch, reps=15, warm=3):
    for _ in range(warm):
        launch()
    torch.cuda.synchronize()
    timer = ct.EventTimer()
    times = []
    for _ in range(reps):
        flush.zero_()
        timer.start()
        launch()
        times.append(timer.stop())
    timer.close()
    times.sort()
    return _quantile(times, 0.5), times[0]


def probe_ceilings(ct, torch, flush):
    """What this box sustains on the bare resources (cutile-rs_amd/bench/ceilings.hip, a code object of its own
    launched through the C ABI's module calls), under the same flush + event protocol as the workloads:
    nothing but bf16 MFMAs on register operands (ones: few bits toggle; random: the bit activity of real data), the
    same loop with the GEMM kernel's LDS operand traffic, and nontemporal read / write / copy streams of 1 GiB."""
    import ctypes as C

    path = os.path.join(ROOT, "cutile-rs_amd", "lib", "probes.hsaco")
    if not os.path.exists(path):
        return {"error": "lib/probes.hsaco is not built"}
    with open(path, "rb") as f:
        mod = ct.Module(f.read())
    out = {}
    cus = 256
    sink = torch.empty(2 * cus * 512, dtype=torch.float32, device="cuda")
    iters = 20000
    flops = 2.0 * cus * 8 * iters * 2 * 8 * (2 * 32 * 32 * 16)
    for name, fn in (("mfma_bf16_registers", "probe_mfma_bf16"), ("mfma_bf16_lds_operands", "probe_mfma_bf16_lds"),
                     ("mfma_16x16x32_bf16_registers", "probe_mfma16_bf16"), ("mfma_16x16x32_bf16_lds_operands", "probe_mfma16_bf16_lds")):
        f = mod.function(fn)
        for mode, label in ((0, "ones"), (1, "random")):
            med, mn = _timed(ct, torch, flush, lambda: ct.Module.launch(
                f, (2 * cus, 1, 1), (512, 1, 1), [C.c_void_p(sink.data_ptr()), C.c_int32(iters), C.c_int32(mode)]), reps=7, warm=1)
            fl = flops * (2.0 if "16x16x32" in name else 1.0)     # 64 MFMAs of 16 x 16 x 32 per iteration: twice the flops of 16 of 32 x 32 x 16
            out[f"{name}_{label}"] = {"TFLOP/s": round(fl / (med * 1e-3) / 1e12, 1), "frac_of_2500": round(fl / (med * 1e-3) / 1e12 / 2500, 4),
                                      "kernel_ms": round(med, 3)}
    # v_exp_f32 against a software exp2's multiply-adds (16 chains per lane and iteration, 2 wavefronts per SIMD,
    # one workgroup per CU): nanoseconds per wavefront and chain
    f = mod.function("probe_valu_exp2")
    v_iters = 20000
    valu = {}
    for mode, label in ((0, "exp2_and_add"), (1, "seven_fma"), (2, "both_interleaved")):
        med, mn = _timed(ct, torch, flush, lambda: ct.Module.launch(
            f, (cus, 1, 1), (512, 1, 1), [C.c_void_p(sink.data_ptr()), C.c_int32(v_iters), C.c_int32(mode)]), reps=5, warm=1)
        valu[label + "_ns"] = round(med * 1e6 / (2.0 * v_iters * 16), 2)
    out["valu_exp2_vs_fma"] = valu
    n_bytes = 1 << 30
    n_vec = n_bytes // 16
    src = torch.empty(n_bytes // 4, dtype=torch.int32, device="cuda").fill_(0x3c003c00)
    dst = torch.empty(n_bytes // 4, dtype=torch.int32, device="cuda")
    small = torch.empty(4096, dtype=torch.int32, device="cuda")
    streams = [("hbm_read", "probe_stream_read", n_bytes, (512, 1024, 2048))]
    streams += [(f"hbm_write_{pol}", f"probe_stream_write_{pol}", n_bytes, (512, 8192, 32768)) for pol in ("plain", "nt", "sc1", "sc0sc1")]
    streams += [(f"hbm_copy_{pol}", f"probe_stream_copy_{pol}", 2 * n_bytes, (2048, 8192, 32768)) for pol in ("plain_v8", "nt_v8", "nt_v4", "sc0sc1_v8")]
    for name, fn, moved, grids in streams:
        f = mod.function(fn)
        best = None
        for g in grids:
            if fn == "probe_stream_read":
                params = [C.c_void_p(src.data_ptr()), C.c_void_p(small.data_ptr()), C.c_uint64(n_vec)]
            elif "write" in fn:
                params = [C.c_void_p(dst.data_ptr()), C.c_uint64(n_vec)]
            else:
                params = [C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr()), C.c_uint64(n_vec)]
            med, mn = _timed(ct, torch, flush, lambda: ct.Module.launch(f, (g, 1, 1), (256, 1, 1), params), reps=9, warm=2)
            rate = moved / (med * 1e-3) / 1e9
            if best is None or rate > best["GB/s"]:
                best = {"GB/s": round(rate, 1), "frac_of_8000": round(rate / 8000, 4), "workgroups": g, "kernel_ms": round(med, 4)}
        out[name] = best
    # the best of each kind: what a kernel that only reads / only writes / reads and writes once can reach here
    for kind in ("write", "copy"):
        k = max((n for n in out if n.startswith(f"hbm_{kind}_")), key=lambda n: out[n]["GB/s"])
        out[f"hbm_{kind}"] = dict(out[k], policy=k[len(f"hbm_{kind}_"):])
    mod.close()
    return out


def same_kernel_zero_operands(ct, torch, flush):
    """The library's own GEMM 8192^3 and FMHA kernels, launched exactly as the workloads launch them, on operands that are
    all zero: the same instruction stream, memory traffic and schedule, but no bits toggle in the matrix pipes, so the
    clock the power limit allows is higher.  What these reach is what the kernels' structure sustains; the distance from
    there to the figures on random data is the device's power management, not the schedule.  Both protocols: the
    flushed median of the workloads, and ten launches back to back (warm caches, steady clocks)."""
    def both(launch, flops):
        med, _ = _timed(ct, torch, flush, launch, reps=9, warm=3)
        timer = ct.EventTimer()
        runs = []
        for _ in range(5):
            timer.start()
            for _ in range(10):
                launch()
            runs.append(timer.stop() / 10)
        timer.close()
        runs.sort()
        tf = lambda ms: round(flops / (ms * 1e-3) / 1e12, 1)
        return {"TFLOP/s": tf(med), "frac_of_2500": round(tf(med) / 2500, 4), "back_to_back_TFLOP/s": tf(runs[len(runs) // 2]),
                "back_to_back_frac_of_2500": round(tf(runs[len(runs) // 2]) / 2500, 4)}

    out = {}
    for s in (8192, 4096):
        a = torch.zeros(s, s, dtype=torch.bfloat16, device="cuda")
        b = torch.zeros(s, s, dtype=torch.bfloat16, device="cuda")
        z = torch.zeros(s, s, dtype=torch.bfloat16, device="cuda")
        zp = ct.partition(z, [256, 256])
        out[f"gemm_bf16_{s}"] = both(lambda: ct.gemm(zp, a, b, s, accumulate=True), 2.0 * s ** 3)
        del a, b, z, zp
    s = 8192                        # MXFP8: e4m3 zeros with unit scales (e8m0 127), priced at the fp8 peak
    x = torch.zeros(s, s, dtype=torch.uint8, device="cuda")
    sc = torch.full((s, s // 32), 127, dtype=torch.uint8, device="cuda")
    z = torch.zeros(s, s, dtype=torch.bfloat16, device="cuda")
    zp = ct.partition(z, [256, 256])
    r = both(lambda: ct.linear_tile_mxfp8(zp, x, x, sc, sc, 1.0), 2.0 * s ** 3)
    out["mxfp8_gemm_8192"] = {"TFLOP/s": r["TFLOP/s"], "frac_of_5000": round(r["TFLOP/s"] / 5000, 4), "back_to_back_TFLOP/s": r["back_to_back_TFLOP/s"],
                              "back_to_back_frac_of_5000": round(r["back_to_back_TFLOP/s"] / 5000, 4)}
    del x, sc, z, zp
    bb, h, sq, d = Fmha.b, Fmha.h, Fmha.s, Fmha.d
    q, k, v = (torch.zeros(bb, h, sq, d, dtype=torch.bfloat16, device="cuda") for _ in range(3))
    o = torch.zeros(bb * h, sq, d, dtype=torch.bfloat16, device="cuda")
    op = ct.partition(o, [1, Fmha.bm, d])
    for causal in (False, True):
        out["fmha_bf16_causal" if causal else "fmha_bf16"] = both(
            lambda: ct.fmha(op, q, k, v, d ** -0.5, 0, 1, causal=causal), (2.0 if causal else 4.0) * sq * sq * d * h * bb)
    return out


def launch_modes():
    """Host-visible latency of the execution modes of the C++ host surface (sync / chained / future / graph replay), one
    small kernel and a 1000-kernel chain: cutile-rs_amd/bench/launch_overhead.cpp, the measurement of the reference's
    cutile-benchmarks/paper/sec5_exp2_execution_mode_overhead.  A child process (it owns its own streams); microseconds
    only, no roofline.  The reference's published medians (another vendor's desktop GPU, RTX 5090) are beside it."""
    import subprocess

    exe = os.path.join(ROOT, "cutile-rs_amd", "bin", "launch_overhead")
    if not os.path.exists(exe):
        return {"error": "cutile-rs_amd/bin/launch_overhead is not built"}
    try:
        res = subprocess.run([exe, "--samples", "30"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=180)
        out = json.loads([l for l in res.stdout.splitlines() if l.startswith("{")][-1])
    except Exception as e:      # the measurement is informational: never fail the bench line over it
        return {"error": f"{type(e).__name__}: {e}"}
    ref = {"sync-individual/n=1": 7.282, "async/n=1": 22.024, "graph/n=1": 5.551, "sync-individual/n=1000": 7441.384,
           "sync-chained/n=1000": 3364.874, "async/n=1000": 3398.144, "graph/n=1000": 810.009}
    return {"kernel": out["kernel"], "unit": "us per pipeline, median",
            "median_us": {k: round(v["median_us"], 2) for k, v in out["modes"].items()},
            "reference_rtx5090_median_us": ref,
            "reference_source": "cutile-benchmarks/paper/sec5_exp2_execution_mode_overhead/launch_overhead_rust/results_part_a.csv"}


BASELINE_CONFIGS = ["gemm_bf16_8192", "gemm_bf16_4096", "fmha_bf16", "fmha_bf16_causal", "rms_norm_f16_16384x8192",
                    "softmax_f16_16384x8192", "saxpy_f32_16777216", "mxfp8_gemm_8192"]
LINE_LIMIT = 4096            # bytes of the final stdout line; everything else goes to FULL_RECORD
FULL_RECORD = os.path.join("gpurun_out", "bench_full.json")


def _r(x, n=4):
    return None if x is None else round(x, n)


def compact_line(records, steps, warmup, device, ceilings=None):
    """The one JSON line a run ends with: the headline workload's record (records[0]) with its roofline and CPU baseline,
    every benchmark configuration in short form, and the ceilings this run measured.  At most LINE_LIMIT bytes: the
    full records are written to a file, never into this line."""
    h = records[0]
    rf = h["roofline"]
    line = {
        "metric": METRIC, "value": _r(h["value"], 2), "unit": h["unit"], "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": _r(h["ms_per_step"], 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "warmup_ms_budget": WARMUP_BUDGET_S * 1e3, "dtype": h["dtype"], "data": "synthetic (seeded host PRNG, same bytes fed to the CPU oracle)", "config": h["config"],
        "roofline": {"bound": rf["bound"], "achieved": _r(rf["achieved"], 2), "peak": rf["peak"], "unit": rf["unit"],
                     "frac": _r(rf["frac"]), "traffic": rf.get("traffic"), "kernel_ms": _r(rf["kernel_ms"], 5),
                     "kernel_ms_back_to_back": _r(rf.get("kernel_ms_back_to_back"), 5),
                     "frac_back_to_back": _r(rf.get("frac_back_to_back")), "frac_wall": _r(rf.get("frac_wall")),
                     "protocol": "frac: median of per-launch HIP-event times, 512 MiB cache flush before each; "
                                 "frac_back_to_back / frac_wall: K launches in a row (events / host clock)"},
    }
    for k in ("cpu_baseline", "parity", "kernel"):
        if k in h:
            line[k] = h[k]
    line["device"] = device
    by_name = {r["workload"]: r for r in records}
    ceilings = ceilings or {}
    copy_rate = ceilings.get("hbm_copy_GB/s")
    short = {}
    for n in BASELINE_CONFIGS:
        if n not in by_name:
            continue
        r = by_name[n]["roofline"]
        e = {"achieved": _r(r["achieved"], 1), "frac": _r(r["frac"]), "kernel_ms": _r(r["kernel_ms"]),
             "kernel_ms_b2b": _r(r.get("kernel_ms_back_to_back")), "frac_b2b": _r(r.get("frac_back_to_back")),
             "ms_per_step": _r(by_name[n]["ms_per_step"]), "frac_wall": _r(r.get("frac_wall")),
             "parity_ok": all(v for k, v in by_name[n].get("parity", {}).items() if isinstance(v, bool))}
        if r["bound"] == "hbm" and copy_rate:
            e["frac_of_copy_ceiling"] = _r(r["achieved"] / copy_rate)
        short[n] = e
    line["baseline_configs"] = short
    if ceilings:
        line["ceilings_summary"] = ceilings
    line["full_record"] = FULL_RECORD
    text = json.dumps(line, separators=(",", ":"))
    for drop in ("full_record", "kernel", "parity", "ceilings_summary"):      # never reached with real records; a guard, not a plan
        if len(text) <= LINE_LIMIT:
            break
        line.pop(drop, None)
        text = json.dumps(line, separators=(",", ":"))
    if len(text) > LINE_LIMIT:
        raise RuntimeError(f"bench line is {len(text)} bytes, over the {LINE_LIMIT}-byte limit")
    return text


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="gemm_bf16_8192")
    ap.add_argument("--only", action="store_true", help="measure only --workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline / sampled parity leg")
    ap.add_argument("--variant", default=None, help="pin this kernel variant for --workload's launcher (otherwise: tuning record, then table order)")
    ap.add_argument("--ceilings", action="store_true", help="also run the ceiling probes (cutile-rs_amd/bench/ceilings.hip), the vendor-library GEMM, "
                                                            "the kernels on zero operands and the launch-mode latencies")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (every kernel here is a one-GPU tile kernel; "
                 "nothing uses a second device) — run with --gpus 1")

    import numpy as np
    import torch

    import __graft_entry__ as entry
    import oracle

    ct = entry.load_package()
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    workloads = make_workloads()
    head = next((w for w in workloads if w.name == args.workload), None)
    if head is None:
        head = next((w for w in make_extra_workloads() if w.name == args.workload), None)
        args.only = args.only or head is not None
    if head is None:
        sys.exit(f"unknown workload {args.workload}; choose from {[w.name for w in workloads + make_extra_workloads()]}")
    order = [head] + ([] if args.only else [w for w in workloads if w is not head])
    if args.variant:
        if not getattr(head, "function", None):
            sys.exit(f"--variant: workload {head.name} does not name the launcher it pins")
        ct.set_preferred_variant(head.function, args.variant)
    flush = torch.empty(FLUSH_BYTES // 4, dtype=torch.int32, device=dev)
    records = []
    for w in order:
        w.setup(ct, torch, oracle, dev)
        with_cpu = not args.no_cpu
        records.append(measure(w, ct, torch, args.steps, args.warmup, with_cpu, oracle, np, flush))
        # free device memory before the next workload
        for k in list(w.__dict__):
            if hasattr(w.__dict__[k], "is_cuda"):
                del w.__dict__[k]
        torch.cuda.empty_cache()
    by_name = {r["workload"]: r for r in records}
    full = {"records": records, "tuning_records": ct.tuning_report().strip().splitlines()}
    summary = {}
    if "copy_f32_67108864" in by_name:      # the library's own convert kernel as a plain copy: what one read + one write reaches here
        c = by_name["copy_f32_67108864"]["roofline"]
        summary["hbm_copy_GB/s"] = round(c["achieved"], 1)
        summary["hbm_copy_frac_of_8000"] = round(c["frac"], 4)
        summary["hbm_copy_what"] = "library convert kernel f32->f32, 2^26 elements, same flush + event protocol"
    if args.ceilings:
        full["library_same_box"] = library_same_box(torch, flush)
        pr = full["probes"] = probe_ceilings(ct, torch, flush)
        full["same_kernel_zero_operands"] = same_kernel_zero_operands(ct, torch, flush)
        full["launch_modes"] = launch_modes()
        if "mfma_bf16_registers_random" in pr:
            summary["probe_TFLOP/s"] = {
                "mfma_loop_ones": pr["mfma_bf16_registers_ones"]["TFLOP/s"], "mfma_loop_random": pr["mfma_bf16_registers_random"]["TFLOP/s"],
                "mfma_16x16x32_random_lds_operands": pr.get("mfma_16x16x32_bf16_lds_operands_random", {}).get("TFLOP/s"),
                "vendor_library_gemm_8192": round(full["library_same_box"]["tflops"], 1),
                "own_kernels_zero_operands_flushed|b2b": {n: [v["TFLOP/s"], v["back_to_back_TFLOP/s"]] for n, v in full["same_kernel_zero_operands"].items()}}
            summary["probe_GB/s"] = {"read": pr["hbm_read"]["GB/s"], "write": pr["hbm_write"]["GB/s"], "copy": pr["hbm_copy"]["GB/s"]}
    text = compact_line(records, args.steps, args.warmup, ct.device_arch(0), summary)
    full["line"] = json.loads(text)
    try:
        os.makedirs(os.path.dirname(FULL_RECORD), exist_ok=True)
        with open(FULL_RECORD, "w") as f:
            json.dump(full, f, indent=1)
    except OSError as e:
        sys.stderr.write(f"bench.py: could not write {FULL_RECORD}: {e}\n")
    print(text, flush=True)


if __name__ == "__main__":
    main()
