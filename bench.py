#!/usr/bin/env python3
"""Benchmark of the gfx950 FP8 GEMM library on one MI355X.

One "step" is one launch of the hot path (a whole GEMM) through the C ABI on
synthetic operands that are already resident in HBM.  The headline workload is
the compute-bound square shape M=N=K=8192, e4m3 x e4m3 -> fp32; the same run
also times the LLM-linear skinny shapes (HBM-bound) and the reference's CPU
GEMM loop on the host cores.

The 8192^3 kernel runs at the board's power limit, and the chip's power
management takes some tens of milliseconds of continuous load to settle (the
first launches after idle run at other clocks than the hundredth).  So that the
timed steps show what a caller in a loop gets, whatever --warmup says, an
untimed settle phase comes first: launches in blocks of 20 until three
successive blocks agree within 2 % (at most 2 s).  The rate of the very first
block after idle is reported beside it (`cold_burst`).

Prints ONE JSON line.  `python bench.py --gpus N` with N > 1 exits with a
message: this build measures one GPU.
"""
import argparse
import glob
import importlib.util
import json
import os
import statistics
import sys
import threading
import time

ROOT = os.path.dirname(os.path.abspath(__file__))

PEAK_FP8_TFLOPS = 5000.0     # MI355X dense FP8 MFMA peak, TFLOP/s
PEAK_HBM_GBS = 8000.0        # MI355X HBM3E peak, GB/s

# HBM-side bytes moved by one 8192^3 launch of the tiled kernel: a constant taken from the
# rocprofv3 FETCH_SIZE / WRITE_SIZE counter runs summarised under profiles/ (each scaled by
# what the same counter reads for a plain copy kernel of known size), not a reading of this run.
TRAFFIC_8192 = {"fetch_kib": 393431, "fetch_scale": 2.0, "write_kib": 262624, "write_scale": 1.0}
TRAFFIC_BYTES_8192 = int((TRAFFIC_8192["fetch_kib"] * TRAFFIC_8192["fetch_scale"] +
                          TRAFFIC_8192["write_kib"] * TRAFFIC_8192["write_scale"]) * 1024)

SETTLE_BLOCK = 20            # launches per settle block
SETTLE_AGREE = 1.02          # three successive blocks within 2 %
SETTLE_CAP_S = 2.0


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


class BoardSampler(threading.Thread):
    """Shader clock and board power from sysfs while the timed launches run (both are
    firmware averages; absent files are skipped)."""

    def __init__(self):
        super().__init__(daemon=True)
        self.power_files = glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input") + \
            glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_average")
        self.cap_files = glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_cap")
        self.sclk_files = glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk")
        self.stop_flag = threading.Event()
        self.power_w, self.sclk_mhz = [], []

    @staticmethod
    def _read(path):
        try:
            with open(path) as f:
                return f.read()
        except OSError:
            return None

    def run(self):
        while not self.stop_flag.is_set():
            for p in self.power_files[:1]:
                v = self._read(p)
                if v and v.strip().isdigit():
                    self.power_w.append(int(v) / 1e6)
            for p in self.sclk_files[:1]:
                v = self._read(p) or ""
                for line in v.splitlines():
                    if line.rstrip().endswith("*"):
                        digits = "".join(ch for ch in line.split(":")[1] if ch.isdigit())
                        if digits:
                            self.sclk_mhz.append(int(digits))
            time.sleep(0.005)

    def summary(self):
        cap = None
        for p in self.cap_files[:1]:
            v = self._read(p)
            if v and v.strip().isdigit():
                cap = int(v) / 1e6
        if not self.power_w and not self.sclk_mhz:
            return {"available": False}
        out = {"available": True, "samples": max(len(self.power_w), len(self.sclk_mhz)), "power_cap_w": cap}
        if self.power_w:
            out.update(power_w_last=self.power_w[-1], power_w_max=max(self.power_w), power_w_median=statistics.median(self.power_w))
        if self.sclk_mhz:
            out.update(shader_clock_mhz_last=self.sclk_mhz[-1], shader_clock_mhz_median=statistics.median(self.sclk_mhz),
                       shader_clock_mhz_nominal=2400)
        return out


def time_block(torch, fn, n, offset=0):
    """Milliseconds per launch over n back-to-back launches: HIP events on the launch stream."""
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(n):
        fn(offset + i)
    e1.record()
    e1.synchronize()
    return e0.elapsed_time(e1) / n


def settle(torch, fn, block=SETTLE_BLOCK, cap_s=SETTLE_CAP_S):
    """Untimed: launches until the chip's clocks have settled under this load.  Returns the
    per-launch time of every block (the first one is the burst right after idle)."""
    blocks = [time_block(torch, fn, block)]
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < cap_s:
        blocks.append(time_block(torch, fn, block))
        last = blocks[-3:]
        if len(blocks) >= 4 and max(last) <= SETTLE_AGREE * min(last):
            break
    return blocks


def time_launches(torch, fn, steps, warmup):
    """The contract's measurement: `warmup` untimed launches, then exactly `steps` timed ones
    between synchronisations.  Returns (ms per launch by HIP events, by the host clock)."""
    for i in range(warmup):
        fn(i)
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


FMT_NAME = {0: "e4m3", 1: "e5m2"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the host CPU leg")
    ap.add_argument("--no-vendor", action="store_true", help="skip the hipBLASLt comparison (a child process)")
    ap.add_argument("--no-llm-shapes", action="store_true", help="time only M=16 N=28672 K=8192 of the skinny shapes")
    ap.add_argument("--no-sparse", action="store_true", help="skip the SpMV / SpMM shapes")
    ap.add_argument("--no-more-shapes", action="store_true",
                    help="skip 16384^3, the four pairings at 4096^3 and the K=32768 stress shapes")
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

    L = pkg.lib()
    stream = torch.cuda.current_stream().cuda_stream      # events and launches share this stream

    def raw_launch(m, k, n, a, b, c, fa=0, fb=0):
        """The bare C-ABI call (a few microseconds of host time, so short kernels stay back to back)."""
        pa, pb, pc = a.data_ptr(), b.data_ptr(), c.data_ptr()

        def go(_i):
            code = L.fp8gemm_launch(m, k, n, pa, fa, pb, fb, pc, 2, stream)
            if code != 0:
                pkg.check(code)
        return go

    def time_settled(m, k, n, fa, fb, A_host, B_host, steps, rows):
        """One more benchmark shape through fp8gemm_launch: operands to HBM, clocks settled under
        this shape's own load, `steps` timed launches, a sample of full rows against the CPU
        oracle (checker only).  Returns the record for the JSON line."""
        dA = torch.from_numpy(A_host).to(dev)
        dB = torch.from_numpy(B_host).to(dev)
        dC = torch.empty((m, n), dtype=torch.float32, device=dev)
        fn = raw_launch(m, k, n, dA, dB, dC, fa, fb)
        settle(torch, fn)
        ms_, _ = time_launches(torch, fn, steps, 5)
        tf = 2.0 * m * n * k / (ms_ * 1e-3) / 1e12
        rec = {"M": m, "N": n, "K": k, "a": FMT_NAME[fa], "b": FMT_NAME[fb], "steps": steps, "ms": ms_, "tflops": tf,
               "frac_of_fp8_peak": tf / PEAK_FP8_TFLOPS, "plan": list(pkg.plan(m, k, n))}
        try:
            oracle = load_oracle()
            ridx = np.asarray(rows, dtype=np.int32)
            got = dC[torch.from_numpy(ridx).long().to(dev)].cpu().numpy()
            ref, S = oracle.gemm(A_host, fa, B_host, fb, rows=ridx, with_scale=True)
            err = np.abs(got.astype(np.float64) - ref)
            tol = oracle.tolerance(k, S)
            rec["parity"] = {"rows_checked": int(ridx.size), "worst_err_over_tol": float((err / tol).max()),
                             "pass": bool(np.isfinite(got).all() and (err <= tol).all())}
        except Exception as ex:
            rec["parity"] = {"error": str(ex)[:200]}
        del dA, dB, dC
        torch.cuda.empty_cache()
        return rec

    # ---------------------------------------------------------------- square, compute-bound
    M = N = K = 8192
    A_h = pkg.fill((M, K), pkg.E4M3, seed=0xA11CE + 3, dist="normal")
    B_h = pkg.fill((N, K), pkg.E4M3, seed=0xB0B + 3, dist="normal")
    A = torch.from_numpy(A_h).to(dev)
    B = torch.from_numpy(B_h).to(dev)
    C = torch.empty((M, N), dtype=torch.float32, device=dev)
    torch.cuda.synchronize()
    flops = 2.0 * M * N * K
    alg_bytes = M * K + N * K + 4 * M * N

    def to_tflops(ms):
        return flops / (ms * 1e-3) / 1e12

    go = raw_launch(M, K, N, A, B, C)
    sampler = BoardSampler()
    sampler.start()
    settle_blocks = settle(torch, go)
    ms, wall_ms = time_launches(torch, go, args.steps, args.warmup)
    # the same measurement five more times, back to back: how far one block of `steps` launches scatters
    repeat_ms = [time_block(torch, go, args.steps) for _ in range(5)]
    sampler.stop_flag.set()
    sampler.join()
    # board power and shader clock over one more second of the same launches, sampled every 5 ms
    board_sampler = BoardSampler()
    board_sampler.start()
    t_board = time.perf_counter()
    while time.perf_counter() - t_board < 1.0:
        time_block(torch, go, 50)
    board_sampler.stop_flag.set()
    board_sampler.join()
    tflops = to_tflops(ms)

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

    # The same launch on all-zero operands: same instructions, same memory traffic, far less
    # switching in the matrix pipe.  What it gains over the figure above is what the board's power
    # limit takes from the kernel on real data (reported beside `value`, never as it).
    A.zero_()
    B.zero_()
    zero_sampler = BoardSampler()
    zero_sampler.start()
    settle(torch, go)
    zero_ms, _ = time_launches(torch, go, args.steps, args.warmup)
    zero_sampler.stop_flag.set()
    zero_sampler.join()
    zero_operands = {"what": "the same kernel and shape on all-zero operands (not a result: it shows how much of the "
                             "gap to the peak is the board's power limit on N(0,1) data)",
                     "tflops": to_tflops(zero_ms), "frac_of_fp8_peak": to_tflops(zero_ms) / PEAK_FP8_TFLOPS,
                     "board": zero_sampler.summary()}
    del A, B, C
    torch.cuda.empty_cache()

    # ---------------------------------------------------------------- the other compute-bound benchmark shapes
    # (each through fp8gemm_launch, clocks settled under its own load; `value` stays the 8192^3 figure)
    square_sweep = [{"M": M, "N": N, "K": K, "a": "e4m3", "b": "e4m3", "steps": args.steps, "ms": ms, "tflops": tflops,
                     "frac_of_fp8_peak": tflops / PEAK_FP8_TFLOPS, "plan": list(pkg.plan(M, K, N)), "parity": parity}]
    pairings_4096, stress_k32768 = [], []
    if not args.no_more_shapes:
        n16 = 16384
        square_sweep.append(time_settled(
            n16, n16, n16, 0, 0, pkg.fill((n16, n16), pkg.E4M3, seed=0xA11CE + 3, dist="normal"),
            pkg.fill((n16, n16), pkg.E4M3, seed=0xB0B + 3, dist="normal"), max(10, args.steps // 5), [0, 255, 256, 8191, 16383]))
        for fa, fb in [(0, 0), (1, 1), (0, 1), (1, 0)]:
            pairings_4096.append(time_settled(
                4096, 4096, 4096, fa, fb, pkg.fill((4096, 4096), fa, seed=0xA11CE + 2, dist="normal", sigma=4.0),
                pkg.fill((4096, 4096), fb, seed=0xB0B + 2, dist="normal", sigma=4.0), args.steps, [0, 129, 1000, 2047, 4095]))
        for fa, fb in [(1, 0), (0, 1)]:
            stress_k32768.append(time_settled(
                4096, 32768, 4096, fa, fb, pkg.fill((4096, 32768), fa, seed=0xA11CE + 5, dist="loguniform"),
                pkg.fill((4096, 32768), fb, seed=0xB0B + 5, dist="loguniform"), max(10, args.steps // 2), [0, 1027, 4095]))

    # ---------------------------------------------------------------- LLM-linear shapes, HBM-bound
    # Cold figures: every launch reads a weight buffer that has been pushed out of the 256 MB
    # Infinity Cache by the launches before it (rotation over buffers totalling 1.2 GB and more).
    def graph_time(m2, k2, n2, A2, Ws, C2, steps2):
        """The cold rotation again, as a serving loop would issue it: one launch per weight buffer
        captured into a HIP graph (through the entry point that allocates nothing, which is what a
        capture needs) and the graph replayed.  Milliseconds per launch, or None if the shape's
        scratch does not fit the static array."""
        if L.fp8gemm_scratch_bytes(m2, k2, n2) > pkg.NOALLOC_SCRATCH_BYTES:
            return None
        side = torch.cuda.Stream()
        pa, pc = A2.data_ptr(), C2.data_ptr()

        def enqueue():
            for W in Ws:
                code = L.fp8gemm_launch_noalloc(m2, k2, n2, pa, 0, W.data_ptr(), 0, pc, 2, side.cuda_stream)
                if code != 0:
                    pkg.check(code)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            enqueue()                       # eager once: the address of the static array is looked up here
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            enqueue()
        replays = max(3, steps2 // len(Ws))
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(replays):
            graph.replay()
        e1.record()
        e1.synchronize()
        return e0.elapsed_time(e1) / (replays * len(Ws))

    def time_llm(n2, k2, ms_list, W_h):
        res = []
        nbuf = max(3, -(-(1200 << 20) // (n2 * k2)))
        Ws = [torch.from_numpy(W_h).to(dev)]
        for _ in range(1, nbuf):
            Ws.append(Ws[0].clone())
        for m2 in ms_list:
            A2 = torch.from_numpy(pkg.fill((m2, k2), pkg.E4M3, seed=0xA11CE + 4 + m2, dist="normal")).to(dev)
            C2 = torch.empty((m2, n2), dtype=torch.float32, device=dev)
            gos = [raw_launch(m2, k2, n2, A2, W, C2) for W in Ws]
            steps2 = max(args.steps, 60)
            # (the host has just spent seconds generating data and the chip sat idle: bring the
            # clocks back under this shape's own load first, as for the square shape)
            settle(torch, lambda i: gos[i % nbuf](i), block=100, cap_s=0.5)
            ms_cold, _ = time_launches(torch, lambda i: gos[i % nbuf](i), steps2, 30)
            ms_warm, _ = time_launches(torch, gos[0], steps2, 30)
            ms_graph = graph_time(m2, k2, n2, A2, Ws, C2, steps2)
            bytes2 = m2 * k2 + n2 * k2 + 4 * m2 * n2
            flops2 = 2.0 * m2 * n2 * k2
            gbs = bytes2 / (ms_cold * 1e-3) / 1e9
            tf = flops2 / (ms_cold * 1e-3) / 1e12
            res.append({"M": m2, "N": n2, "K": k2, "algorithmic_bytes": bytes2, "plan": list(pkg.plan(m2, k2, n2)),
                        "us_cold": ms_cold * 1e3, "gbs_cold": gbs, "frac_hbm_peak_cold": gbs / PEAK_HBM_GBS,
                        "tflops_cold": tf, "frac_fp8_peak_cold": tf / PEAK_FP8_TFLOPS,
                        "us_warm": ms_warm * 1e3, "gbs_warm": bytes2 / (ms_warm * 1e-3) / 1e9,
                        "us_cold_in_graph": None if ms_graph is None else ms_graph * 1e3,
                        "frac_hbm_peak_cold_in_graph": None if ms_graph is None else bytes2 / (ms_graph * 1e-3) / 1e9 / PEAK_HBM_GBS,
                        "weight_buffers": nbuf})
        return res

    llm = []
    groups = [(28672, 8192, [16] if args.no_llm_shapes else [1, 16, 64, 256])]
    if not args.no_llm_shapes:
        groups += [(8192, 28672, [1, 16, 64, 256]), (10240, 8192, [1, 16, 64, 256])]
    for gi, (n2, k2, ms_list) in enumerate(groups):
        W_h = pkg.fill((n2, k2), pkg.E4M3, seed=0xB0B + 4 + gi, dist="weights", sigma=0.02)
        llm += time_llm(n2, k2, ms_list, W_h)
        torch.cuda.empty_cache()
    head = [r for r in llm if (r["M"], r["N"], r["K"]) == (16, 28672, 8192)][0]
    skinny = {"workload": "M=16 N=28672 K=8192 e4m3 activations x e4m3 weights -> fp32",
              "algorithmic_bytes": head["algorithmic_bytes"],
              "us_cold": head["us_cold"], "gbs_cold": head["gbs_cold"],
              "us_warm": head["us_warm"], "gbs_warm": head["gbs_warm"],
              "frac_hbm_peak_cold": head["frac_hbm_peak_cold"],
              "note": "cold = rotating over %d weight buffers (nothing of the next one left in the 256 MB Infinity "
                      "Cache), warm = same buffer every launch" % head["weight_buffers"]}

    # ---------------------------------------------------------------- sparse operands (SpMV: HBM-bound, SpMM: MFMA on stored blocks)
    sparse = []
    if not args.no_sparse:
        rng = np.random.default_rng(0x5BA)

        def raw_time(fn_of_i, steps2):
            settle(torch, fn_of_i, block=50, cap_s=0.3)
            return time_launches(torch, fn_of_i, steps2, 20)[0]

        def ck(code):
            if code != 0:
                pkg.check(code)

        # blocked-ELL: block columns as the reference's generator draws them (distinct, rising, uniform)
        def bell_operand(m2, k2, block, ell):
            cols = np.stack([np.sort(rng.permutation(k2 // block)[:ell]) for _ in range(m2 // block)]).astype(np.int32)
            vals = pkg.fill((m2, ell * block), pkg.E4M3, seed=0x5BA + m2 + block, dist="normal")
            return torch.from_numpy(vals).to(dev), torch.from_numpy(cols).to(dev)

        # matrix-vector, blocked-ELL: pruned weight matrix 28672 x 8192, a quarter of the 64 x 64 blocks kept
        m2, k2, block, ell = 28672, 8192, 64, 32
        ncopy = 6
        ops = [bell_operand(m2, k2, block, ell) for _ in range(ncopy)]
        xv = torch.from_numpy(pkg.fill((k2,), pkg.E4M3, seed=0x5BA + 1, dist="normal")).to(dev)
        yv = torch.empty(m2, dtype=torch.float32, device=dev)

        def go_bell_mv(i):
            v, c = ops[i % ncopy]
            ck(L.fp8gemm_spmv_bell(m2, k2, block, ell, v.data_ptr(), 0, c.data_ptr(), xv.data_ptr(), 0, yv.data_ptr(), stream))
        ms_c = raw_time(go_bell_mv, 120)
        ms_w = raw_time(lambda i: go_bell_mv(0), 120)
        by = m2 * ell * block + (m2 // block) * ell * 4 + k2 + 4 * m2
        sparse.append({"kernel": "fp8gemm_spmv_bell", "M": m2, "K": k2, "block": block, "stored_blocks_per_row": ell,
                       "density": ell * block / k2, "algorithmic_bytes": by, "us_cold": ms_c * 1e3, "us_warm": ms_w * 1e3,
                       "gbs_cold": by / ms_c / 1e6, "frac_hbm_peak_cold": by / ms_c / 1e6 / PEAK_HBM_GBS, "copies_rotated": ncopy})
        del ops

        # matrix-vector, CSR: the same matrix shape, one element in ten kept at uniformly drawn places
        mask = rng.random((m2, k2)) < 0.10
        offs = np.concatenate([[0], np.cumsum(mask.sum(axis=1))]).astype(np.int32)
        colh = np.nonzero(mask)[1].astype(np.int32)
        del mask
        nnz = int(offs[-1])
        ncopy = 4
        csr_ops = []
        for c in range(ncopy):
            csr_ops.append((torch.from_numpy(pkg.fill((nnz,), pkg.E4M3, seed=0x5BA + 7 + c, dist="normal")).to(dev),
                            torch.from_numpy(offs).to(dev), torch.from_numpy(colh).to(dev)))

        def go_csr_mv(i):
            v, o, c = csr_ops[i % ncopy]
            ck(L.fp8gemm_spmv_csr(m2, k2, v.data_ptr(), 0, o.data_ptr(), c.data_ptr(), None, xv.data_ptr(), 0, yv.data_ptr(), stream))
        ms_c = raw_time(go_csr_mv, 120)
        ms_w = raw_time(lambda i: go_csr_mv(0), 120)
        by = 5 * nnz + 4 * (m2 + 1) + k2 + 4 * m2
        sparse.append({"kernel": "fp8gemm_spmv_csr", "M": m2, "K": k2, "stored_entries": nnz, "density": nnz / (m2 * k2),
                       "algorithmic_bytes": by, "us_cold": ms_c * 1e3, "us_warm": ms_w * 1e3, "gbs_cold": by / ms_c / 1e6,
                       "frac_hbm_peak_cold": by / ms_c / 1e6 / PEAK_HBM_GBS, "copies_rotated": ncopy})
        del csr_ops

        # matrix-matrix, blocked-ELL, blocks of whole tiles (the LDS-tiled kernel) and small blocks (the direct kernel)
        for (m3, k3, n3, block, ell) in [(8192, 8192, 8192, 256, 8), (8192, 8192, 8192, 128, 16), (4096, 4096, 4096, 32, 32)]:
            v, c = bell_operand(m3, k3, block, ell)
            Bd = torch.from_numpy(pkg.fill((n3, k3), pkg.E4M3, seed=0x5BA + 3, dist="normal")).to(dev)
            Cd = torch.empty((m3, n3), dtype=torch.float32, device=dev)
            ms3 = raw_time(lambda i: ck(L.fp8gemm_spmm_bell(m3, k3, n3, block, ell, v.data_ptr(), 0, c.data_ptr(), Bd.data_ptr(), 0,
                                                            Cd.data_ptr(), stream)), 30)
            fl = 2.0 * m3 * ell * block * n3
            sparse.append({"kernel": "fp8gemm_spmm_bell", "M": m3, "K": k3, "N": n3, "block": block, "stored_blocks_per_row": ell,
                           "density": ell * block / k3, "us": ms3 * 1e3, "tflops_on_stored_blocks": fl / ms3 / 1e9,
                           "frac_of_fp8_peak_on_stored_blocks": fl / ms3 / 1e9 / PEAK_FP8_TFLOPS,
                           "dense_equivalent_tflops": 2.0 * m3 * k3 * n3 / ms3 / 1e9})
            del v, c, Bd, Cd
        # matrix-matrix, CSR: through the dense scratch and the dense GEMM
        m3 = k3 = n3 = 4096
        mask = rng.random((m3, k3)) < 0.10
        offs = np.concatenate([[0], np.cumsum(mask.sum(axis=1))]).astype(np.int32)
        colh = np.nonzero(mask)[1].astype(np.int32)
        nnz = int(offs[-1])
        v = torch.from_numpy(pkg.fill((nnz,), pkg.E4M3, seed=0x5BA + 9, dist="normal")).to(dev)
        o, c = torch.from_numpy(offs).to(dev), torch.from_numpy(colh).to(dev)
        Bd = torch.from_numpy(pkg.fill((n3, k3), pkg.E4M3, seed=0x5BA + 3, dist="normal")).to(dev)
        Cd = torch.empty((m3, n3), dtype=torch.float32, device=dev)
        ms3 = raw_time(lambda i: ck(L.fp8gemm_spmm_csr(m3, k3, n3, v.data_ptr(), 0, o.data_ptr(), c.data_ptr(), Bd.data_ptr(), 0,
                                                       Cd.data_ptr(), stream)), 30)
        sparse.append({"kernel": "fp8gemm_spmm_csr", "M": m3, "K": k3, "N": n3, "stored_entries": nnz, "density": nnz / (m3 * k3),
                       "us": ms3 * 1e3, "dense_equivalent_tflops": 2.0 * m3 * k3 * n3 / ms3 / 1e9,
                       "note": "S is written out as a dense fp8 matrix in scratch, then the dense GEMM runs"})
        del v, o, c, Bd, Cd, xv, yv
        # sampled dense-dense product: 8192 x 8192 outputs in column vectors of 8, one vector in ten kept, K = 512
        m_vec, vec, n4, k4 = 1024, 8, 8192, 512
        mask = rng.random((m_vec, n4)) < 0.10
        offs = np.concatenate([[0], np.cumsum(mask.sum(axis=1))]).astype(np.int32)
        colh = np.nonzero(mask)[1].astype(np.int32)
        nnz = int(offs[-1])
        o, c = torch.from_numpy(offs).to(dev), torch.from_numpy(colh).to(dev)
        Ld = torch.from_numpy(pkg.fill((m_vec * vec, k4), pkg.E4M3, seed=0x5BA + 11, dist="normal")).to(dev)
        Rd = torch.from_numpy(pkg.fill((n4, k4), pkg.E4M3, seed=0x5BA + 12, dist="normal")).to(dev)
        Od = torch.empty((nnz, vec), dtype=torch.float32, device=dev)
        ms4 = raw_time(lambda i: ck(L.fp8gemm_sddmm(m_vec, k4, vec, o.data_ptr(), c.data_ptr(), Ld.data_ptr(), 0, Rd.data_ptr(), 0,
                                                    Od.data_ptr(), stream)), 60)
        sparse.append({"kernel": "fp8gemm_sddmm", "rows": m_vec * vec, "cols": n4, "K": k4, "vec_length": vec, "stored_vectors": nnz,
                       "density": nnz / (m_vec * n4), "us": ms4 * 1e3, "tflops_on_stored_outputs": 2.0 * nnz * vec * k4 / ms4 / 1e9,
                       "gathered_rhs_gbs": nnz * k4 / ms4 / 1e6,
                       "note": "every stored vector reads one row of rhs (K bytes) out of cache; vec_length 8 fills half of the MFMA's rows"})
        del o, c, Ld, Rd, Od
        torch.cuda.empty_cache()

    # ---------------------------------------------------------------- CPU baseline (host cores)
    cpu = None
    if not args.no_cpu_baseline:
        try:
            oracle = load_oracle()
            mc = nc = kc = 1024
            Ac = pkg.fill((mc, kc), pkg.E4M3, seed=0xA11CE + 1, dist="normal")
            Bc = pkg.fill((nc, kc), pkg.E4M3, seed=0xB0B + 1, dist="normal")
            t_verb = []
            for _ in range(2):
                t0 = time.perf_counter()
                oracle.gemm_verbatim(Ac, 0, Bc, 0)
                t_verb.append(time.perf_counter() - t0)
            t_fast = []
            for _ in range(3):
                t0 = time.perf_counter()
                oracle.gemm(Ac, 0, Bc, 0)
                t_fast.append(time.perf_counter() - t0)
            fl = 2.0 * mc * nc * kc
            cpu = {"value": fl / min(t_verb) / 1e12, "unit": "TFLOPS", "cores": 1, "kind": "port",
                   "sample": "the whole M=N=K=1024 e4m3 CPU-path configuration, the reference's m-n-k loop order "
                             "with one decode per operand per multiply, one thread, 2 repetitions "
                             "(best %.2f s, mean %.2f s); value = best" % (min(t_verb), sum(t_verb) / 2),
                   "seconds_best": min(t_verb), "seconds_mean": sum(t_verb) / 2, "host_cores": os.cpu_count(),
                   "all_cores": {"value": fl / min(t_fast) / 1e12, "unit": "TFLOPS", "cores": oracle.num_threads(),
                                 "seconds_best": min(t_fast), "seconds_mean": sum(t_fast) / 3,
                                 "what": "bit-identical blocked/OpenMP form of the same loop, full 1024^3, 3 repetitions"}}
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

    rep_tf = sorted(to_tflops(x) for x in repeat_ms)
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
        "settle": {"what": "untimed launches before --warmup, in blocks of %d until three successive blocks agree "
                           "within %d %% (cap %.0f s): the chip's power management needs continuous load to settle"
                           % (SETTLE_BLOCK, round((SETTLE_AGREE - 1) * 100), SETTLE_CAP_S),
                   "settle_launches": SETTLE_BLOCK * len(settle_blocks),
                   "last_block_tflops": to_tflops(settle_blocks[-1]),
                   "slowest_block_tflops": to_tflops(max(settle_blocks))},
        "cold_burst": {"what": "the first %d launches after the chip sat idle" % SETTLE_BLOCK,
                       "ms_per_step": settle_blocks[0], "tflops": to_tflops(settle_blocks[0]),
                       "frac_of_fp8_peak": to_tflops(settle_blocks[0]) / PEAK_FP8_TFLOPS},
        "repeats": {"what": "five more blocks of `steps` launches right after the timed one",
                    "tflops_median": rep_tf[2], "tflops_min": rep_tf[0], "tflops_max": rep_tf[-1]},
        "board": dict(board_sampler.summary(), what="one more second of back-to-back launches of the same shape right after "
                                                    "the timed ones, sysfs sampled every 5 ms",
                      during_timed_steps=sampler.summary()),
        "zero_operands": zero_operands,
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s",
                     "frac": tflops / PEAK_FP8_TFLOPS, "traffic": TRAFFIC_BYTES_8192,
                     "traffic_source": "constant from the rocprofv3 --pmc summary under profiles/ "
                                       "(FETCH_SIZE %d KiB x %.1f + WRITE_SIZE %d KiB x %.1f), not read in this run"
                                       % (TRAFFIC_8192["fetch_kib"], TRAFFIC_8192["fetch_scale"],
                                          TRAFFIC_8192["write_kib"], TRAFFIC_8192["write_scale"]),
                     "algorithmic_flops": flops, "algorithmic_bytes": alg_bytes,
                     "kernel_ms": ms},
        "square_sweep": square_sweep,
        "pairings_4096": pairings_4096,
        "stress_k32768": stress_k32768,
        "skinny": skinny,
        "llm_shapes": llm,
        "sparse": sparse,
        "parity": parity,
        "cpu_baseline": cpu,
        "vendor": vendor,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
