"""The C++ harness (counterpart of the reference's GEMM/gemm_main.cpp): command line and
the CPU reference path, which run without a GPU."""
import os
import subprocess

import pytest


@pytest.fixture(scope="module")
def gemm_bin(pkg):
    path = os.path.join(pkg.HARNESS_DIR, "out", "gemm")
    if not os.path.exists(path):
        pkg.build()
    return path


def run(gemm_bin, *args):
    return subprocess.run([gemm_bin] + [str(a) for a in args], capture_output=True, text=True,
                          cwd=os.path.dirname(os.path.dirname(gemm_bin)), timeout=300)


def test_usage_on_wrong_argument_count(gemm_bin):
    r = run(gemm_bin, 128, 128, 128)
    assert r.returncode == 1 and "Input Format" in r.stdout and "[dimM] [dimK] [dimN] [kernel]" in r.stdout
    assert run(gemm_bin, "--help", 0, 0, 0, 0, 0, 0).returncode == 1


def test_cpu_reference_path_runs_and_is_thread_invariant(gemm_bin):
    r = run(gemm_bin, 192, 256, 160, 0, 0, 0, 0, "normal", 5)
    assert r.returncode == 0, r.stderr
    assert "CPU reference GEMM e4m3 x e4m3: M = 192, K = 256, N = 160" in r.stdout
    assert "bit-identical to 1 thread: yes" in r.stdout
    again = run(gemm_bin, 192, 256, 160, 0, 0, 0, 0, "normal", 5)
    assert [l for l in r.stdout.splitlines() if "checksum" in l] == [l for l in again.stdout.splitlines() if "checksum" in l]
    other = run(gemm_bin, 192, 256, 160, 0, 0, 0, 0, "normal", 6)
    assert [l for l in r.stdout.splitlines() if "checksum" in l] != [l for l in other.stdout.splitlines() if "checksum" in l]


def test_harness_cpu_path_agrees_with_the_oracle(gemm_bin, pkg, oracle):
    """Same seeded operands through the harness's own loop and through the oracle: the
    checksum printed by the harness is the float64 sum of the fp32 outputs."""
    M, K, N, seed = 64, 384, 48, 9
    r = run(gemm_bin, M, K, N, 0, 0, 0, 0, "normal4", seed)
    assert r.returncode == 0, r.stderr
    line = [l for l in r.stdout.splitlines() if "checksum" in l][0]
    got = float(line.split()[-1])
    A = pkg.fill((M, K), 0, seed=0xA11CE + seed, dist="normal", sigma=4.0)
    B = pkg.fill((N, K), 0, seed=0xB0B + seed, dist="normal", sigma=4.0)
    want = float(oracle.gemm(A, 0, B, 0).astype("float64").sum())
    assert abs(got - want) <= 1e-6 * max(1.0, abs(want))


def test_unsupported_kernel_id(gemm_bin):
    r = run(gemm_bin, 128, 128, 128, 42, 0, 0, 0)
    assert r.returncode == 0 and "unsupported kernel" in r.stdout


def test_sweep_table_and_plots_from_records(pkg, tmp_path):
    """plot_sweep.py on records in the harness's CSV format (M,K,N,GFLOPS per row) and a
    comparator log: table with roofline fractions, two PNG files."""
    import sys
    data = tmp_path / "data"
    data.mkdir()
    (data / "fp8_gemm_v1.csv").write_text("4096,4096,4096,2000000.0\n8192,8192,8192,2500000.0\n16,8192,28672,170000.0\n")
    (data / "fp8_gemm_v3.csv").write_text("4096,4096,4096,1900000.0\n")
    vendor = tmp_path / "vendor.log"
    vendor.write_text("Average hipblasLtMatmul execution time 0.48 (ms)\n"
                      "GEMM-hipblaslt-fp8: M[8192] x N[8192] x K[8192], performance = 2250000.0GFLOPS.\n")
    script = os.path.join(pkg.HARNESS_DIR, "plot_sweep.py")
    r = subprocess.run([sys.executable, script, "--data", str(data), "--vendor", str(vendor), "--plot"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    row = [l for l in r.stdout.splitlines() if l.split()[:3] == ["8192", "8192", "8192"]][0].split()
    assert row[3] == "2500.0" and row[-1] == "2250.0"
    assert abs(float(row[4]) - 2 * 8192 ** 3 / (6.0 * 8192 ** 2)) < 0.1          # flop per byte
    assert abs(float(row[6].rstrip("%")) - 100 * 2500.0 / 5000.0) < 0.1           # MFMA-bound
    skinny = [l for l in r.stdout.splitlines() if l.split()[:3] == ["16", "8192", "28672"]][0].split()
    bytes_ = 16 * 8192 + 28672 * 8192 + 4 * 16 * 28672
    assert abs(float(skinny[5]) - 2 * 16 * 8192 * 28672 / bytes_ * 8.0) < 0.2     # HBM-bound: intensity x 8 TB/s
    assert (data / "fp8_gemm_sweep.png").stat().st_size > 1000 and (data / "fp8_gemm_roofline.png").stat().st_size > 1000
    assert subprocess.run([sys.executable, script, "--data", str(tmp_path / "none")], capture_output=True).returncode == 1
