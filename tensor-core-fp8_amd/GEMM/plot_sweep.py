#!/usr/bin/env python3
"""Tables and plots from the harness's sweep records.

Input: data/fp8_gemm_v<k>.csv as written by `out/gemm ... record=1` -- the
reference's record format, one row `M,K,N,GFLOPS` per run and kernel id k
(GEMM/gemm_main.cpp:87-110 there) -- and, optionally, the output of
`out/hipblaslt` saved to a text file (the vendor line of the comparison).

Output: a table on stdout with, per row, the arithmetic intensity
(2MNK flop over MK + NK + 4MN bytes), the roofline bound
min(MFMA peak, intensity * HBM peak) and the fraction of it reached; with
--plot, two PNG files next to the records: rate over size per kernel id, and
the same points in a roofline diagram.

    python3 plot_sweep.py [--data data] [--vendor hipblaslt.log] [--plot]
"""
import argparse
import csv
import glob
import os
import re
import sys

MFMA_PEAK_TFLOPS = 5000.0     # MI355X dense FP8 MFMA peak (the figure the harness and bench.py use)
HBM_PEAK_GBS = 8000.0
KERNEL_NAMES = {1: "e4m3 x e4m3, 2 stages", 2: "e4m3 x e4m3, 4 stages", 3: "e5m2 x e5m2, 2 stages",
                4: "e5m2 x e5m2, 4 stages", 5: "e4m3 x e5m2, 2 stages", 6: "e4m3 x e5m2, 4 stages",
                7: "e5m2 x e4m3, 2 stages", 8: "e5m2 x e4m3, 4 stages"}


def intensity(m, k, n):
    return 2.0 * m * k * n / (m * k + n * k + 4.0 * m * n)


def bound_tflops(m, k, n):
    return min(MFMA_PEAK_TFLOPS, intensity(m, k, n) * HBM_PEAK_GBS / 1000.0)


def read_records(data_dir):
    """{kernel id: [(M, K, N, TFLOPS), ...]}; a shape recorded twice keeps the last row."""
    out = {}
    for path in sorted(glob.glob(os.path.join(data_dir, "fp8_gemm_v*.csv"))):
        m = re.search(r"fp8_gemm_v(\d+)\.csv$", path)
        if not m:
            continue
        rows = {}
        with open(path, newline="") as f:
            for rec in csv.reader(f):
                if len(rec) < 4:
                    continue
                try:
                    mm, kk, nn, gf = int(rec[0]), int(rec[1]), int(rec[2]), float(rec[3])
                except ValueError:
                    continue          # header or damaged line
                rows[(mm, kk, nn)] = gf / 1000.0
        out[int(m.group(1))] = [(a, b, c, t) for (a, b, c), t in sorted(rows.items())]
    return out


def read_vendor(path):
    """[(M, K, N, TFLOPS)] from the comparator's `GEMM-hipblaslt-fp8: M[..] x N[..] x K[..], performance = ..GFLOPS.` lines."""
    rows = []
    pat = re.compile(r"GEMM-hipblaslt-fp8: M\[(\d+)\] x N\[(\d+)\] x K\[(\d+)\], performance = ([0-9.eE+-]+)GFLOPS")
    with open(path) as f:
        for line in f:
            m = pat.search(line)
            if m:
                rows.append((int(m.group(1)), int(m.group(3)), int(m.group(2)), float(m.group(4)) / 1000.0))
    return rows


def print_table(records, vendor):
    vend = {(m, k, n): t for m, k, n, t in vendor}
    for kid, rows in sorted(records.items()):
        print("kernel %d (%s)" % (kid, KERNEL_NAMES.get(kid, "?")))
        print("  %6s %6s %6s %10s %9s %10s %8s %10s" % ("M", "K", "N", "TFLOPS", "flop/B", "bound TF", "of bound", "vendor TF"))
        for m, k, n, t in rows:
            b = bound_tflops(m, k, n)
            v = vend.get((m, k, n))
            print("  %6d %6d %6d %10.1f %9.1f %10.1f %7.1f%% %10s" %
                  (m, k, n, t, intensity(m, k, n), b, 100.0 * t / b, "%.1f" % v if v is not None else "-"))


def plot(records, vendor, data_dir):
    import matplotlib
    matplotlib.use("Agg")
    import matplotlib.pyplot as plt

    fig, ax = plt.subplots(figsize=(8, 5))
    for kid, rows in sorted(records.items()):
        sq = [(m, t) for m, k, n, t in rows if m == k == n]
        if sq:
            ax.plot([s for s, _ in sq], [t for _, t in sq], marker="o", ms=3, label="%d: %s" % (kid, KERNEL_NAMES.get(kid, "?")))
    vs = [(m, t) for m, k, n, t in vendor if m == k == n]
    if vs:
        ax.plot([s for s, _ in vs], [t for _, t in vs], "k--", label="hipBLASLt e4m3 x e4m3")
    ax.axhline(MFMA_PEAK_TFLOPS, color="gray", lw=0.8)
    ax.set_xlabel("M = N = K")
    ax.set_ylabel("TFLOP/s")
    ax.set_title("FP8 GEMM, square sweep (MI355X)")
    ax.legend(fontsize=7)
    ax.grid(alpha=0.3)
    sweep_png = os.path.join(data_dir, "fp8_gemm_sweep.png")
    fig.savefig(sweep_png, dpi=130, bbox_inches="tight")
    plt.close(fig)

    fig, ax = plt.subplots(figsize=(8, 5))
    xs = [2.0 ** (e / 4.0) for e in range(0, 14 * 4 + 1)]
    ax.loglog(xs, [min(MFMA_PEAK_TFLOPS, x * HBM_PEAK_GBS / 1000.0) for x in xs], "k-", lw=1.2, label="roofline: 8 TB/s, 5.0 PFLOP/s")
    for kid, rows in sorted(records.items()):
        ax.loglog([intensity(m, k, n) for m, k, n, _ in rows], [t for _, _, _, t in rows], "o", ms=3,
                  label="%d: %s" % (kid, KERNEL_NAMES.get(kid, "?")))
    ax.set_xlabel("arithmetic intensity, flop / byte")
    ax.set_ylabel("TFLOP/s")
    ax.set_title("FP8 GEMM in the roofline (MI355X)")
    ax.legend(fontsize=7)
    ax.grid(alpha=0.3, which="both")
    roof_png = os.path.join(data_dir, "fp8_gemm_roofline.png")
    fig.savefig(roof_png, dpi=130, bbox_inches="tight")
    plt.close(fig)
    return sweep_png, roof_png


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--data", default=os.path.join(os.path.dirname(os.path.abspath(__file__)), "data"))
    ap.add_argument("--vendor", default=None, help="text output of out/hipblaslt")
    ap.add_argument("--plot", action="store_true")
    args = ap.parse_args(argv)
    records = read_records(args.data)
    if not records:
        print("no fp8_gemm_v*.csv under %s; run `out/gemm ... record=1` first" % args.data)
        return 1
    vendor = read_vendor(args.vendor) if args.vendor else []
    print_table(records, vendor)
    if args.plot:
        for p in plot(records, vendor, args.data):
            print("wrote", p)
    return 0


if __name__ == "__main__":
    sys.exit(main())
