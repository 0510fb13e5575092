"""Builds the gfx950 code objects and the C-ABI host library, in tree.

    python cutile-rs_amd/build.py [--force]

Outputs (git-ignored, carried to the GPU box with the tree):
    cutile-rs_amd/lib/*.hsaco          one ELF code object per kernel source
    cutile-rs_amd/lib/libcutile_hip.so host library with the code objects embedded

The device side is compiled by hipcc for gfx950 only; the host side is plain
C++17 compiled by g++ and binds the HIP runtime with dlopen, so no GPU (and no
HIP runtime) is needed to build or to load the library.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

ROOT = os.path.dirname(os.path.abspath(__file__))
KERNEL_DIR = os.path.join(ROOT, "csrc", "kernels")
HOST_DIR = os.path.join(ROOT, "csrc", "host")
LIB_DIR = os.path.join(ROOT, "lib")
BUILD_DIR = os.path.join(ROOT, "build")
LIB_PATH = os.path.join(LIB_DIR, "libcutile_hip.so")
SCRATCH_LIB_PATH = os.path.join(LIB_DIR, "libcutile_hip_scratch.so")

# image symbol -> kernel source
IMAGES = {
    "elementwise": "elementwise.hip",
    "rowwise": "rowwise.hip",
    "gemm": "gemm_bf16.hip",
    "fmha": "fmha.hip",
    "mxgemm": "mxfp8_gemm.hip",
    "nvfp4": "nvfp4_gemm.hip",
    "rng": "rng.hip",
}
HOST_SOURCES = ["hip_api.cpp", "driver.cpp", "kernel_table.cpp", "launch.cpp", "runtime.cpp", "tuning.cpp"]
# The recording stand-in for the HIP runtime (include/cutile_hip_testing.h) is not part of the product library: the CPU
# tests load a second library, the same objects plus this source.
TESTING_SOURCES = ["fake_hip.cpp"]
TESTING_LIB_PATH = os.path.join(LIB_DIR, "libcutile_hip_testing.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
CXX = os.environ.get("CXX", "g++")
DEVICE_FLAGS = [
    "--offload-arch=gfx950", "--cuda-device-only", "--no-gpu-bundle-output", "-c", "-O3", "-std=c++17",
    # packed FP32 instructions are kept off on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
# extra device-compiler flags for one-off builds (e.g. -DNAME=1), space separated
DEVICE_FLAGS += os.environ.get("CUTILE_EXTRA_DEVICE_FLAGS", "").split()
HOST_FLAGS = ["-std=c++17", "-O2", "-g0", "-fPIC", "-Wall", "-Wextra", "-Wno-unused-parameter",
              "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", "-pthread"]


def _newer(target: str, sources: list[str]) -> bool:
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(s) <= t for s in sources)


def _run(cmd: list[str]) -> None:
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + res.stdout)
        raise RuntimeError(f"build step failed: {cmd[0]} ... {cmd[-1]}")


def build_code_objects(force: bool = False) -> dict[str, str]:
    os.makedirs(LIB_DIR, exist_ok=True)
    headers = [os.path.join(KERNEL_DIR, f) for f in os.listdir(KERNEL_DIR) if f.endswith(".h")]
    jobs = []
    out = {}
    for name, src in IMAGES.items():
        src_path = os.path.join(KERNEL_DIR, src)
        dst = os.path.join(LIB_DIR, name + ".hsaco")
        out[name] = dst
        if force or not _newer(dst, [src_path] + headers):
            jobs.append([HIPCC] + DEVICE_FLAGS + ["-o", dst, src_path])
    with ThreadPoolExecutor(max_workers=4) as ex:
        list(ex.map(_run, jobs))
    return out


def build_host_library(images: dict[str, str], force: bool = False) -> str:
    os.makedirs(BUILD_DIR, exist_ok=True)
    embed = os.path.join(BUILD_DIR, "embed.S")
    lines = ['.section .rodata', '']
    for name, path in images.items():
        lines += [f".global cutile_img_{name}_start", f".global cutile_img_{name}_end", ".balign 4096",
                  f"cutile_img_{name}_start:", f'.incbin "{path}"', f"cutile_img_{name}_end:", ""]
    lines += ['.section .note.GNU-stack,"",@progbits', ""]
    text = "\n".join(lines)
    if not os.path.exists(embed) or open(embed).read() != text:
        with open(embed, "w") as f:
            f.write(text)
    # the device compiler's identity, for the provenance of tuning records
    ver = subprocess.run([HIPCC, "--version"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True).stdout
    keep = [l.strip() for l in ver.splitlines() if l.startswith(("HIP version", "AMD clang version", "clang version"))]
    fingerprint = "; ".join(keep)[:200].replace("\\", "/").replace('"', "'") or "unknown"
    toolchain = os.path.join(BUILD_DIR, "toolchain.h")
    text_h = f'#define CUTILE_TOOLCHAIN_FINGERPRINT "{fingerprint}"\n'
    if not os.path.exists(toolchain) or open(toolchain).read() != text_h:
        with open(toolchain, "w") as f:
            f.write(text_h)
    sources = [os.path.join(HOST_DIR, s) for s in HOST_SOURCES]
    testing = [os.path.join(HOST_DIR, s) for s in TESTING_SOURCES]
    include = os.path.join(ROOT, "..", "include")
    deps = sources + testing + [embed, toolchain] + list(images.values()) + [
        os.path.join(HOST_DIR, f) for f in os.listdir(HOST_DIR) if f.endswith(".h")
    ] + [os.path.join(include, "cutile_hip.h"), os.path.join(include, "cutile_hip_testing.h")] + [
        os.path.join(include, "cutile", f) for f in ("tune.hpp", "json.hpp", "bench.hpp", "runtime.hpp", "error.hpp", "device_op.hpp")]
    if force or not _newer(LIB_PATH, deps) or not _newer(TESTING_LIB_PATH, deps):
        objs = {}
        jobs = []
        for s in sources + testing + [embed]:
            o = os.path.join(BUILD_DIR, os.path.basename(s) + ".o")
            objs[s] = o
            if force or not _newer(o, deps):
                jobs.append([CXX] + HOST_FLAGS + ["-I", BUILD_DIR, "-c", s, "-o", o])
        with ThreadPoolExecutor(max_workers=6) as ex:
            list(ex.map(_run, jobs))
        product = [objs[s] for s in sources + [embed]]
        _run([CXX, "-shared", "-o", LIB_PATH] + product + ["-ldl", "-pthread", "-Wl,--no-undefined"])
        _run([CXX, "-shared", "-o", TESTING_LIB_PATH] + product + [objs[s] for s in testing] + ["-ldl", "-pthread", "-Wl,--no-undefined"])
    return LIB_PATH


PROBES_PATH = os.path.join(LIB_DIR, "probes.hsaco")


def build_probes(force: bool = False) -> str:
    """Ceiling probes for `bench.py --ceilings` (bare MFMA loop, streaming reads / writes / copies): a code object of their own,
    not embedded in the host library."""
    src = os.path.join(ROOT, "bench", "ceilings.hip")
    if force or not _newer(PROBES_PATH, [src]):
        _run([HIPCC] + DEVICE_FLAGS + ["-o", PROBES_PATH, src])
    return PROBES_PATH


def build_scratch_library(force: bool = False) -> str:
    """The side library that holds the device-resident scratch array: the one file hipcc compiles for host and
    device.  It links the HIP runtime by soname; libcutile_hip.so opens it only after it has bound a runtime."""
    src = os.path.join(HOST_DIR, "scratch.hip")
    deps = [src, os.path.join(HOST_DIR, "scratch.h")]
    if force or not _newer(SCRATCH_LIB_PATH, deps):
        _run([HIPCC, "--offload-arch=gfx950", "-O2", "-std=c++17", "-fPIC", "-shared",
              "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
              "-o", SCRATCH_LIB_PATH, src])
    return SCRATCH_LIB_PATH


CPP_TEST_DIR = os.path.join(ROOT, "..", "tests", "cpp")
CPP_TESTS = {
    # binary -> (source, library it links: True = the product library, "testing" = the one with the recording runtime, extra flags)
    "test_host_surface": ("test_host_surface.cpp", "testing", []),
    "test_gpu_surface": ("test_gpu_surface.cpp", True, []),
    "write_record": ("write_record.cpp", True, []),
    "test_slot_table": ("test_slot_table.cpp", False, []),
    "test_slot_table_tsan": ("test_slot_table.cpp", False, ["-fsanitize=thread"]),
}


def build_cpp_tests(force: bool = False) -> str:
    """Compiles the C++ host-surface test programs (run by tests/test_cpp_surface.py)."""
    out_dir = os.path.join(CPP_TEST_DIR, "bin")
    os.makedirs(out_dir, exist_ok=True)
    include = os.path.join(ROOT, "..", "include")
    headers = [os.path.join(include, "cutile", f) for f in os.listdir(os.path.join(include, "cutile"))]
    headers += [os.path.join(include, f) for f in os.listdir(include) if f.endswith(".h")]
    headers += [os.path.join(CPP_TEST_DIR, "check.hpp"), os.path.join(HOST_DIR, "slot_table.h")]
    jobs = []
    for name, (src, needs_lib, extra) in CPP_TESTS.items():
        dst = os.path.join(out_dir, name)
        src_path = os.path.join(CPP_TEST_DIR, src)
        deps = [src_path] + headers + ([TESTING_LIB_PATH if needs_lib == "testing" else LIB_PATH] if needs_lib else [])
        if force or not _newer(dst, deps):
            cmd = [CXX, "-std=c++17", "-O1", "-g0", "-I" + include, "-Wall", "-Wextra", "-Wno-unused-parameter"] + extra
            cmd += [src_path, "-o", dst, "-pthread"]
            if needs_lib:
                cmd += ["-L" + LIB_DIR, "-lcutile_hip_testing" if needs_lib == "testing" else "-lcutile_hip",
                        "-Wl,-rpath,$ORIGIN/../../../cutile-rs_amd/lib"]
            jobs.append(cmd)
    with ThreadPoolExecutor(max_workers=4) as ex:
        list(ex.map(_run, jobs))
    return out_dir


PROGRAMS = {
    # cutile-rs_amd/bin/<name>: programs on the C++ host surface
    "tune_baseline": os.path.join("tune", "tune_baseline.cpp"),        # writes the tuning records
    "launch_overhead": os.path.join("bench", "launch_overhead.cpp"),   # execution-mode latency, run by bench.py
}


def build_tuner(force: bool = False) -> str:
    """The programs of the package that sit on the C++ host surface (cutile-rs_amd/bin/)."""
    out_dir = os.path.join(ROOT, "bin")
    os.makedirs(out_dir, exist_ok=True)
    include = os.path.join(ROOT, "..", "include")
    headers = [os.path.join(include, "cutile", f) for f in os.listdir(os.path.join(include, "cutile"))]
    jobs = []
    for name, rel in PROGRAMS.items():
        src, dst = os.path.join(ROOT, rel), os.path.join(out_dir, name)
        if force or not _newer(dst, [src, LIB_PATH] + headers):
            jobs.append([CXX, "-std=c++17", "-O2", "-g0", "-I" + include, "-Wall", "-Wextra", "-Wno-unused-parameter", src, "-o", dst, "-pthread",
                         "-L" + LIB_DIR, "-lcutile_hip", "-Wl,-rpath,$ORIGIN/../lib"])
    with ThreadPoolExecutor(max_workers=2) as ex:
        list(ex.map(_run, jobs))
    return out_dir


def build(force: bool = False) -> str:
    lib = build_host_library(build_code_objects(force), force)
    build_tuner(force)
    build_scratch_library(force)
    build_probes(force)
    build_cpp_tests(force)
    return lib


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
