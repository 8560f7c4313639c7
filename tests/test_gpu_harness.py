"""The re-created C++ harness on the GPU: kernel ids 1..8 through the C++ overloads
gemm::GEMM / gemm::GEMM4 (GEMM/include/gemm.h), the timing loop, verification against the
harness's own CPU loop and the CSV records -- the flow of the reference's
GEMM/gemm_main.cpp:66-184, 223-263 and of `make gemm_test` (GEMM/makefile:48-49)."""
import os
import re
import shutil
import subprocess

import pytest

pytestmark = pytest.mark.gpu

PAIRING = {1: "e4m3 * e4m3", 2: "e4m3 * e4m3", 3: "e5m2 * e5m2", 4: "e5m2 * e5m2",
           5: "e4m3 * e5m2", 6: "e4m3 * e5m2", 7: "e5m2 * e4m3", 8: "e5m2 * e4m3"}


@pytest.fixture(scope="module")
def harness(pkg, tmp_path_factory):
    """The built harness, run from a scratch directory so that its ./data records do not
    mix with anything else."""
    exe = os.path.join(pkg.HARNESS_DIR, "out", "gemm")
    if not os.path.exists(exe):
        raise RuntimeError("the harness is not built (%s): run __graft_entry__.build()" % exe)
    cwd = tmp_path_factory.mktemp("harness")

    def run(*args, timeout=600, env=None):
        return subprocess.run([exe] + [str(a) for a in args], capture_output=True, text=True, cwd=str(cwd),
                              timeout=timeout, env=dict(os.environ, **(env or {})))
    run.cwd = cwd
    return run


def check_verified(r, kernel, M, K, N, absolute=True):
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    out = r.stdout
    assert PAIRING[kernel] + " = fp32" in out
    assert "GEMM-stage%d:  M = %d, K = %d, N = %d" % (4 if kernel % 2 == 0 else 2, M, K, N) in out
    assert "Result Verified!" in out, out[-1500:]
    assert "errors." not in out
    m = re.search(r"worst \|err\| / \(2\*K\*2\^-24\*sum\|a\*b\|\) = ([0-9.eE+-]+); outputs off by more than 0.25: (\d+)", out)
    assert m, out[-1500:]
    assert float(m.group(1)) < 1.0 or K < 1024          # below 1024 the MFMA window term is part of the bound
    if absolute:
        # the reference's own criterion (gemm_main.cpp:166-170): made for its uniform(-1, 1)
        # operands, where |C| stays below ~sqrt(K); with operands scaled up to the format's
        # largest value an fp32 rounding step alone exceeds it
        assert int(m.group(2)) == 0
    g = re.search(r"FP8-TC Avager Performance = \S*?([0-9.]+)\S* \S*GFlops", out)
    assert g and float(g.group(1)) > 0.0
    assert "end BmFN" in out


@pytest.mark.parametrize("kernel", [1, 2, 3, 4, 5, 6, 7, 8])
def test_reference_self_test_shape_every_kernel_id(harness, kernel):
    """`make gemm_test` of the reference is `out/gemm 128 128 128 2 1 0 0`; here every id runs it
    (the reference leaves 4, 6 and 8 commented out, gemm_main.cpp:236-255)."""
    check_verified(harness(128, 128, 128, kernel, 1, 0, 0), kernel, 128, 128, 128)


@pytest.mark.parametrize("kernel", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("shape,dist", [((256, 256, 256), "normal4"), ((300, 384, 200), "normal4"),
                                        ((64, 1024, 512), "weights"), ((300, 208, 200), "loguniform")])
def test_seeded_distributions_and_ragged_shapes(harness, kernel, shape, dist):
    """Shapes the reference would silently leave unfinished (not multiples of 128,
    GEMM/src/gemm.cu:45-47) and the seeded distributions of the benchmark configurations."""
    M, K, N = shape
    check_verified(harness(M, K, N, kernel, 1, 0, 0, dist, 7), kernel, M, K, N, absolute=(dist == "normal4"))


def test_records_are_appended_as_the_reference_writes_them(harness):
    """record=1: one row M,K,N,GFLOPS per run in ./data/fp8_gemm_v<kernel>.csv
    (gemm_main.cpp:87-110 of the reference), plus the extended record."""
    data = harness.cwd / "data"
    shutil.rmtree(data, ignore_errors=True)
    for kernel, (M, K, N) in [(2, (512, 512, 512)), (2, (1024, 256, 768)), (7, (512, 512, 512))]:
        r = harness(M, K, N, kernel, 0, 1, 0)
        assert r.returncode == 0, r.stderr
        assert "Result Verified!" not in r.stdout           # verify=0: no CPU pass
    rows = (data / "fp8_gemm_v2.csv").read_text().strip().splitlines()
    assert len(rows) == 2
    for row, (M, K, N) in zip(rows, [(512, 512, 512), (1024, 256, 768)]):
        f = row.split(",")
        assert [int(f[0]), int(f[1]), int(f[2])] == [M, K, N] and float(f[3]) > 0 and len(f) == 4
    ext = (data / "fp8_gemm_v2_ext.csv").read_text().strip().splitlines()
    assert len(ext) == 2 and len(ext[0].split(",")) == 9
    f = [float(x) for x in ext[0].split(",")]
    assert abs(f[4] - f[3] / 1e3) < 1e-6 * f[4] + 1e-9              # TFLOPS column
    assert abs(f[7] - f[4] / 5000.0) < 1e-6                          # fraction of the dense FP8 peak
    assert len((data / "fp8_gemm_v7.csv").read_text().strip().splitlines()) == 1


def test_sweep_mode_walks_the_reference_sizes(harness):
    """testbench=1 ignores the given dimensions and walks 256, 512, ... (gemm_main.cpp:264-313
    of the reference; all 64 sizes take minutes, GEMM_TESTBENCH_SIZES shortens the walk);
    an unsupported id ends the sweep at its first entry."""
    r = harness(1, 1, 1, 42, 0, 0, 1)
    assert r.returncode == 0 and r.stdout.count("unsupported kernel") == 1
    r = harness(1, 1, 1, 3, 0, 1, 1, env={"GEMM_TESTBENCH_SIZES": "4"})
    assert r.returncode == 0, r.stderr
    sizes = [tuple(int(x) for x in m) for m in re.findall(r"GEMM-stage2:  M = (\d+), K = (\d+), N = (\d+)", r.stdout)]
    assert sizes == [(256, 256, 256), (512, 512, 512), (768, 768, 768), (1024, 1024, 1024)]
    rows = (harness.cwd / "data" / "fp8_gemm_v3.csv").read_text().strip().splitlines()
    assert [row.split(",")[0] for row in rows[-4:]] == ["256", "512", "768", "1024"]


def test_make_gemm_test_target(pkg):
    r = subprocess.run(["make", "-C", pkg.HARNESS_DIR, "gemm_test"], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-1500:] + r.stderr[-1500:]
    assert "Result Verified!" in r.stdout


def test_vendor_comparator_runs_both_libraries_and_compares_them(pkg, tmp_path):
    """`out/hipblaslt` (the counterpart of the reference's `out/cublas`, GEMM/src/cublas.cu with
    GEMM/include/helper.h): hipBLASLt and this library on the same operands, both timed, the two
    results compared.  Sweep mode on two small sizes, the single-shape mode on a skinny shape."""
    exe = os.path.join(pkg.HARNESS_DIR, "out", "hipblaslt")
    if not os.path.exists(exe):
        raise RuntimeError("the comparator is not built (%s): run __graft_entry__.build()" % exe)

    def run(*args):
        r = subprocess.run([exe] + [str(a) for a in args], capture_output=True, text=True, cwd=str(tmp_path), timeout=300)
        assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
        return r.stdout

    def check(out, shapes):
        vendor = re.findall(r"GEMM-hipblaslt-fp8: M\[(\d+)\] x N\[(\d+)\] x K\[(\d+)\], performance = ([0-9.]+)GFLOPS", out)
        ours = re.findall(r"GEMM-fp8gemm-fp8:\s+M\[(\d+)\] x N\[(\d+)\] x K\[(\d+)\], performance = ([0-9.]+)GFLOPS", out)
        diffs = re.findall(r"max \|hipblaslt - fp8gemm\| = ([0-9.eE+-]+) \(largest \|C\| = ([0-9.eE+-]+)", out)
        assert [tuple(int(x) for x in v[:3]) for v in vendor] == shapes == [tuple(int(x) for x in v[:3]) for v in ours]
        assert all(float(v[3]) > 0 for v in vendor) and all(float(v[3]) > 0 for v in ours)
        assert len(diffs) == len(shapes)
        for (m, n, k), (diff, largest) in zip(shapes, diffs):
            # both are fp32 sums of the same exact products in different orders
            assert float(diff) <= 2.0 * k * 2.0 ** -24 * float(largest) + 1e-6

    check(run(5, 256, 512, 256), [(256, 256, 256), (512, 512, 512)])
    check(run(5, "shape", 16, 1024, 512), [(16, 512, 1024)])
    # the reference sample's scalars and pointers (alpha 2, beta 1, scales 2 / 0.5 / 1 / 1, amax): this library's
    # side is the epilogue entry point, and the two results and largest magnitudes are compared
    out = run(5, 256, 512, 256, "sample")
    check(out, [(256, 256, 256), (512, 512, 512)])
    both = re.findall(r"largest \|D\|: hipblaslt ([0-9.eE+-]+), fp8gemm ([0-9.eE+-]+)", out)
    own = re.findall(r"largest \|D\|: fp8gemm ([0-9.eE+-]+) \(hipblaslt took no amax pointer\)", out)
    assert len(both) + len(own) == 2
    for v, o in both:
        assert abs(float(v) - float(o)) <= 1e-3 * float(o)
    assert all(float(o) > 0 for o in own)
    assert subprocess.run([exe], capture_output=True, text=True).returncode == 1      # usage


@pytest.mark.parametrize("kernel,shape,env", [
    (10, (512, 1024, 300), {}),                                     # blocked-ELL SpMM, 128 x 128 blocks: the tiled kernel
    (10, (512, 1024, 300), {"GEMM_SPARSE_BLOCK": "256", "GEMM_SPARSE_KEEP": "0.5"}),
    (10, (256, 512, 40), {"GEMM_SPARSE_BLOCK": "32"}),               # small blocks: the direct kernel
    (11, (2048, 4096, 1), {"GEMM_SPARSE_BLOCK": "64"}),              # blocked-ELL SpMV
    (12, (300, 1024, 200), {}),                                      # CSR SpMM through the dense scratch
    (13, (3000, 2048, 1), {"GEMM_SPARSE_KEEP": "0.05"}),             # CSR SpMV, longest rows first
])
def test_sparse_kernel_ids(harness, kernel, shape, env):
    """Kernel ids 10..13: the sparse kernels on operands from the re-created generators of the
    reference's bm_test_utils.h (blocked-ELL column lists, CSR with row padding, sorted row
    order), timed and verified against the harness's own CPU loop over the stored entries."""
    M, K, N = shape
    r = harness(M, K, N, kernel, 1, 0, 0, env=env)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert "sparse e4m3 * e4m3 = fp32" in r.stdout
    assert "Result Verified!" in r.stdout and "errors." not in r.stdout, r.stdout[-1500:]
    m = re.search(r"worst \|err\| / tolerance = ([0-9.eE+-]+)", r.stdout)
    assert m and float(m.group(1)) < 1.0
    g = re.search(r"([0-9.]+) GFlops on the stored entries", r.stdout)
    assert g and float(g.group(1)) > 0.0
    assert "end BmSparse" in r.stdout


@pytest.mark.parametrize("shape,env", [((512, 256, 384), {}), ((96, 1040, 200), {"GEMM_SDDMM_VEC": "16", "GEMM_SPARSE_KEEP": "0.3"}),
                                       ((60, 100, 50), {"GEMM_SDDMM_VEC": "4"})])
def test_sddmm_kernel_id(harness, shape, env):
    """Kernel id 14: the sampled dense-dense product on a pattern from the re-created CSR generator,
    verified against the harness's Host_sddmm (the reference's host helper of that name,
    GEMM/include/bm_test_utils.h:172-194 there)."""
    M, K, N = shape
    r = harness(M, K, N, 14, 1, 0, 0, env=env)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert "sampled e4m3 * e4m3 = fp32" in r.stdout
    assert "Result Verified!" in r.stdout and "errors." not in r.stdout, r.stdout[-1500:]
    m = re.search(r"worst \|err\| / tolerance = ([0-9.eE+-]+)", r.stdout)
    assert m and float(m.group(1)) < 1.0
    assert "end BmSddmm" in r.stdout
