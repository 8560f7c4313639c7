#!/usr/bin/env python3
"""Benchmark of the gfx950 FP8 GEMM library on one MI355X.

One "step" is one launch of the hot path (a whole GEMM) through the C ABI on
synthetic operands that are already resident in HBM.  The headline workload is
the compute-bound square shape M=N=K=8192, e4m3 x e4m3 -> fp32; the same run
also times the HBM-bound skinny shape M=16, N=28672, K=8192 and a bounded
sample of the reference's CPU GEMM loop on the host cores.

Prints ONE JSON line (see the keys below).  `python bench.py --gpus N` with
N > 1 exits with a message: this build measures one GPU.
"""
import argparse
import importlib.util
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))

PEAK_FP8_TFLOPS = 5000.0     # MI355X dense FP8 MFMA peak, TFLOP/s
PEAK_HBM_GBS = 8000.0        # MI355X HBM3E peak, GB/s

# HBM bytes moved by one 8192^3 launch of the tiled kernel, from rocprofv3
# FETCH_SIZE / WRITE_SIZE counter runs scaled by the reading of a plain copy
# kernel of known size (summary under profiles/).
TRAFFIC_BYTES_8192 = (2 * 393411 + 262872) * 1024   # FETCH_SIZE x 2.0 (copy-kernel scale) + WRITE_SIZE x 1.0, KiB -> bytes


def load_package():
    name = "tensor_core_fp8_amd"
    if name in sys.modules:
        return sys.modules[name]
    spec = importlib.util.spec_from_file_location(name, os.path.join(ROOT, "tensor-core-fp8_amd", "__init__.py"))
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


def load_oracle():
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import oracle
    return oracle


def time_launches(torch, fn, steps, warmup):
    """Average milliseconds per launch: HIP events on the launch stream around `steps` launches."""
    for _ in range(warmup):
        fn(0)
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        fn(i)
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return e0.elapsed_time(e1) / steps, wall_ms / steps


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=300)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the host CPU leg")
    ap.add_argument("--no-vendor", action="store_true", help="skip the hipBLASLt comparison (a child process)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy, the known-size kernel that FETCH_SIZE / WRITE_SIZE "
                         "counter readings are scaled by when this script runs under rocprofv3 --pmc")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py measures one GPU: the FP8 GEMM path has no multi-GPU part in this build "
                 "(it would shard over N with no exchange); run with --gpus 1")

    import numpy as np
    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    pkg = load_package()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(3)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)          # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    # ---------------------------------------------------------------- square, compute-bound
    M = N = K = 8192
    A_h = pkg.fill((M, K), pkg.E4M3, seed=0xA11CE + 3, dist="normal")
    B_h = pkg.fill((N, K), pkg.E4M3, seed=0xB0B + 3, dist="normal")
    A = torch.from_numpy(A_h).to(dev)
    B = torch.from_numpy(B_h).to(dev)
    C = torch.empty((M, N), dtype=torch.float32, device=dev)
    L = pkg.lib()
    stream = torch.cuda.current_stream().cuda_stream      # events and launches share this stream

    def raw_launch(m, k, n, a, b, c):
        """The bare C-ABI call (a few microseconds of host time, so short kernels stay back to back)."""
        pa, pb, pc = a.data_ptr(), b.data_ptr(), c.data_ptr()
        def go(_i):
            code = L.fp8gemm_launch(m, k, n, pa, 0, pb, 0, pc, 2, stream)
            if code != 0:
                pkg.check(code)
        return go

    ms, wall_ms = time_launches(torch, raw_launch(M, K, N, A, B, C), args.steps, args.warmup)
    flops = 2.0 * M * N * K
    tflops = flops / (ms * 1e-3) / 1e12
    alg_bytes = M * K + N * K + 4 * M * N

    # parity on a sample of full rows, against the CPU oracle (checker only)
    parity = None
    try:
        oracle = load_oracle()
        rows = np.array([0, 1, 31, 32, 127, 128, 255, 256, 4095, 4096 + 129, 8191], dtype=np.int32)
        Cs = C[torch.from_numpy(rows).long().to(dev)].cpu().numpy()
        Cref, S = oracle.gemm(A_h, 0, B_h, 0, rows=rows, with_scale=True)
        err = np.abs(Cs.astype(np.float64) - Cref)
        tol = oracle.tolerance(K, S)
        parity = {"rows_checked": int(rows.size), "worst_err_over_tol": float((err / tol).max()),
                  "pass": bool((err <= tol).all())}
    except Exception as ex:  # the oracle is only the checker; say so if it is unavailable
        parity = {"error": str(ex)[:200]}

    # ---------------------------------------------------------------- skinny, HBM-bound
    m2, n2, k2 = 16, 28672, 8192
    A2 = torch.from_numpy(pkg.fill((m2, k2), pkg.E4M3, seed=0xA11CE + 4, dist="normal")).to(dev)
    W_h = pkg.fill((n2, k2), pkg.E4M3, seed=0xB0B + 4, dist="weights", sigma=0.02)
    # six distinct weight buffers (1.4 GB): a launch finds nothing of its operand left in the
    # 256 MB Infinity Cache (with three, about a tenth of B is still served from it)
    NBUF = 6
    Ws = [torch.from_numpy(W_h).to(dev)]
    for j in range(1, NBUF):
        Ws.append(Ws[0].clone())
    C2 = torch.empty((m2, n2), dtype=torch.float32, device=dev)
    gos = [raw_launch(m2, k2, n2, A2, W, C2) for W in Ws]
    ms_cold, _ = time_launches(torch, lambda i: gos[i % NBUF](i), max(args.steps, 30), args.warmup)
    ms_warm, _ = time_launches(torch, gos[0], max(args.steps, 30), args.warmup)
    bytes2 = m2 * k2 + n2 * k2 + 4 * m2 * n2
    skinny = {"workload": "M=16 N=28672 K=8192 e4m3 activations x e4m3 weights -> fp32",
              "algorithmic_bytes": bytes2,
              "us_cold": ms_cold * 1e3, "gbs_cold": bytes2 / (ms_cold * 1e-3) / 1e9,
              "us_warm": ms_warm * 1e3, "gbs_warm": bytes2 / (ms_warm * 1e-3) / 1e9,
              "frac_hbm_peak_cold": bytes2 / (ms_cold * 1e-3) / 1e9 / PEAK_HBM_GBS,
              "note": "cold = rotating over 6 weight buffers (1.4 GB, nothing left in the 256 MB Infinity Cache), "
                      "warm = same buffer every launch"}

    # ---------------------------------------------------------------- CPU baseline (host cores)
    cpu = None
    if not args.no_cpu_baseline:
        try:
            oracle = load_oracle()
            mc = nc = kc = 1024
            Ac = pkg.fill((mc, kc), pkg.E4M3, seed=0xA11CE + 1, dist="normal")
            Bc = pkg.fill((nc, kc), pkg.E4M3, seed=0xB0B + 1, dist="normal")
            rows_c = 384                      # bounded sample: 384 of the 1024 rows, ~10 s single-thread
            t0 = time.perf_counter()
            oracle.gemm_verbatim(Ac[:rows_c], 0, Bc, 0)
            t_verb = time.perf_counter() - t0
            t0 = time.perf_counter()
            oracle.gemm(Ac, 0, Bc, 0)
            t_fast = time.perf_counter() - t0
            cpu = {"value": 2.0 * rows_c * nc * kc / t_verb / 1e12, "unit": "TFLOPS", "cores": 1, "kind": "port",
                   "sample": "first %d rows of the M=N=K=1024 e4m3 CPU-path configuration, the reference's m-n-k "
                             "loop order, one thread, %.1f s" % (rows_c, t_verb),
                   "all_cores": {"value": 2.0 * mc * nc * kc / t_fast / 1e12, "unit": "TFLOPS",
                                 "cores": oracle.num_threads(),
                                 "what": "bit-identical blocked/OpenMP form of the same loop, full 1024^3"}}
        except Exception as ex:
            cpu = {"error": str(ex)[:200]}

    # ---------------------------------------------------------------- vendor library beside it
    # hipBLASLt on the same shape through the harness's comparator (a child process; per-launch
    # events, both libraries warmed up and timed in alternating blocks).  Informational only.
    vendor = None
    if not args.no_vendor:
        try:
            import re
            import subprocess
            exe = os.path.join(ROOT, "tensor-core-fp8_amd", "GEMM", "out", "hipblaslt")
            r = subprocess.run([exe, "40", "8192", "8192", "1"], capture_output=True, text=True, timeout=120)
            mv = re.search(r"GEMM-hipblaslt-fp8: .* performance = ([0-9.eE+-]+)GFLOPS", r.stdout)
            mo = re.search(r"GEMM-fp8gemm-fp8: .* performance = ([0-9.eE+-]+)GFLOPS", r.stdout)
            md = re.search(r"max \|hipblaslt - fp8gemm\| = ([0-9.eE+-]+)", r.stdout)
            if mv and mo:
                vendor = {"library": "hipBLASLt e4m3 x e4m3 -> fp32, M=N=K=8192, per-launch events",
                          "hipblaslt_tflops": float(mv.group(1)) / 1e3, "this_library_tflops": float(mo.group(1)) / 1e3,
                          "max_abs_difference": float(md.group(1)) if md else None}
            else:
                vendor = {"error": (r.stdout + r.stderr)[-200:]}
        except Exception as ex:
            vendor = {"error": str(ex)[:200]}

    out = {
        "metric": "FP8 GEMM TFLOPS at 8192^3 e4m3 (skinny M=16 HBM GB/s in `skinny`)",
        "value": tflops,
        "unit": "TFLOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms,
        "wall_ms_per_step": wall_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8 e4m3 x e4m3 -> fp32 accumulate (MFMA f8f6f4)",
        "data": "synthetic: seeded N(0,1) rounded to nearest even to OCP e4m3, resident in HBM",
        "config": {"workload": "M=N=K=8192, A row-major MxK e4m3, B stored NxK e4m3, C fp32 row-major",
                   "entry_point": "fp8gemm_launch (automatic kernel choice), stages=2"},
        "frac_of_fp8_peak": tflops / PEAK_FP8_TFLOPS,
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s",
                     "frac": tflops / PEAK_FP8_TFLOPS, "traffic": TRAFFIC_BYTES_8192,
                     "algorithmic_flops": flops, "algorithmic_bytes": alg_bytes,
                     "kernel_ms": ms},
        "skinny": skinny,
        "parity": parity,
        "cpu_baseline": cpu,
        "vendor": vendor,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
