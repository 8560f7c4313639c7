"""The harness's generators of the reference's sparse operand formats (blocked-ELL column lists,
CSR with row padding) and its row orders, checked on the host under the sanitizers."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "tensor-core-fp8_amd")


def test_sparse_generators_and_row_orders(tmp_path):
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    exe = tmp_path / "sparse_formats_check"
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-g", "-fopenmp", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
                           "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(rocm, "include"), "-I", os.path.join(PKG, "GEMM", "include"),
                           "-I", os.path.join(ROOT, "include"), os.path.join(ROOT, "tests", "host", "sparse_formats_check.cpp"),
                           os.path.join(PKG, "csrc", "host_util.cpp"), "-o", str(exe)])
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120,
                       env=dict(os.environ, ASAN_OPTIONS="detect_leaks=0"))
    assert r.returncode == 0, r.stdout + r.stderr
    assert "all checks passed" in r.stdout
