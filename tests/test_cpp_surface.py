"""Runs the C++ test programs of the host surface (tests/cpp/*.cpp, built in tree by
cutile-rs_amd/build.py).  The CPU programs use the recording stand-in for the HIP runtime
or no runtime at all; the GPU program drives the real device through the same headers."""
import os
import subprocess

import pytest

BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "bin")


def _run(name, timeout=300, records=False):
    path = os.path.join(BIN, name)
    assert os.path.exists(path), f"{path} is missing: run python cutile-rs_amd/build.py"
    env = dict(os.environ)
    if not records:
        env["CUTILE_TUNING_RECORDS"] = ""     # variant choices these programs assert are the table's own, not a tuning record's
    res = subprocess.run([path], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=timeout, env=env)
    tail = "\n".join(res.stdout.splitlines()[-25:])
    assert res.returncode == 0 and "TESTS PASSED" in res.stdout, tail
    return res.stdout


def test_host_surface_on_recording_runtime():
    out = _run("test_host_surface")
    assert out.count("PASS ") >= 15


def test_slot_table_protocol():
    _run("test_slot_table")


def test_slot_table_protocol_under_thread_sanitizer():
    out = _run("test_slot_table_tsan")
    assert "ThreadSanitizer" not in out


@pytest.mark.gpu
def test_host_surface_on_gpu():
    out = _run("test_gpu_surface")
    assert out.count("PASS ") >= 12
    print(out)
