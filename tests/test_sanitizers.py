"""Host code under AddressSanitizer + UndefinedBehaviorSanitizer (no GPU involved): the
product codec and generators, the CPU oracle, and the harness's CPU reference path
(kernel id 0).  Device code cannot be sanitized here; these builds cover what runs on the host."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "tensor-core-fp8_amd")
SAN = ["-g", "-O1", "-fno-omit-frame-pointer", "-fsanitize=address,undefined", "-fno-sanitize-recover=all"]
ENV = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1", OMP_NUM_THREADS="4")


def test_codec_generators_and_oracle_under_sanitizers(tmp_path):
    inc = ["-I", os.path.join(ROOT, "include"), "-I", os.path.join(PKG, "GEMM", "include")]
    obj = tmp_path / "oracle.o"
    subprocess.check_call(["gcc", "-std=gnu11", "-fopenmp", "-ffp-contract=off"] + SAN +
                          ["-c", os.path.join(ROOT, "oracle", "fp8_oracle.c"), "-o", str(obj)])
    exe = tmp_path / "sanitize_check"
    subprocess.check_call(["g++", "-std=c++17", "-fopenmp"] + SAN + inc +
                          [os.path.join(ROOT, "tests", "host", "sanitize_check.cpp"), os.path.join(PKG, "csrc", "host_util.cpp"),
                           str(obj), "-o", str(exe), "-lm"])
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=600, env=ENV)
    assert r.returncode == 0, (r.stdout + r.stderr)[-3000:]
    assert "all checks passed" in r.stdout


def test_harness_cpu_path_under_sanitizers(tmp_path, pkg):
    """GEMM/gemm_main.cpp built with the sanitizers and run with kernel id 0 (CPU reference
    GEMM only: the HIP runtime is linked but never called)."""
    lib_dir = os.path.join(PKG, "lib")
    if not os.path.exists(os.path.join(lib_dir, "libfp8gemm.so")):
        pkg.build()
    exe = tmp_path / "gemm_san"
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    subprocess.check_call(["g++", "-std=c++17", "-fopenmp", "-D__HIP_PLATFORM_AMD__"] + SAN +
                          ["-I", os.path.join(rocm, "include"), "-I", os.path.join(PKG, "GEMM", "include"),
                           "-I", os.path.join(ROOT, "include"), os.path.join(PKG, "GEMM", "gemm_main.cpp"), "-o", str(exe),
                           "-L", lib_dir, "-lfp8gemm", "-L", os.path.join(rocm, "lib"), "-lamdhip64",
                           "-Wl,-rpath," + lib_dir, "-Wl,-rpath," + os.path.join(rocm, "lib")])
    for args in (["96", "208", "80", "0", "0", "0", "0", "normal", "3"], ["33", "48", "17", "0", "0", "0", "0", "loguniform", "9"],
                 ["5", "16", "300", "0", "0", "0", "0"]):
        r = subprocess.run([str(exe)] + args, capture_output=True, text=True, timeout=600, env=ENV, cwd=str(tmp_path))
        assert r.returncode == 0, (r.stdout + r.stderr)[-3000:]
        assert "bit-identical to 1 thread: yes" in r.stdout
        assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr
