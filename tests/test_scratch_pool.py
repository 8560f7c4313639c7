"""Bookkeeping of the K-slice scratch (per device and stream, retire-behind-event, no free
inside a launch), exercised on the host with a fake device runtime."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_scratch_pool_bookkeeping(tmp_path):
    exe = tmp_path / "scratch_pool_check"
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
                           "-pthread", "-I", os.path.join(ROOT, "tensor-core-fp8_amd", "csrc"),
                           os.path.join(ROOT, "tests", "host", "scratch_pool_check.cpp"), "-o", str(exe)])
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "all checks passed" in r.stdout
