"""Host side of the C ABI: the library loads, exports every declared symbol, validates its
arguments before touching the GPU, and generates reproducible operands."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest


def declared_symbols(header):
    text = open(header).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fp8gemm_\w+)\s*\(", text)))


def test_library_exports_every_symbol_of_the_header(pkg):
    L = pkg.lib()
    names = declared_symbols(pkg.HEADER_PATH)
    assert len(names) >= 20 and all(n in names for n in pkg.ENTRY_POINTS)
    for n in names:
        assert hasattr(L, n), "missing export " + n
    nm = subprocess.run(["nm", "-D", "--defined-only", pkg.LIB_PATH], capture_output=True, text=True).stdout
    for n in names:
        assert re.search(r"\bT %s\b" % n, nm), "not a defined text symbol: " + n


def test_argument_validation_needs_no_gpu(pkg):
    L = pkg.lib()
    INVALID = 1      # hipErrorInvalidValue
    ok_ptr = ctypes.c_void_p(0x1000)
    assert L.fp8gemm_launch(0, 128, 128, ok_ptr, 0, ok_ptr, 0, ok_ptr, 2, None) == INVALID
    assert L.fp8gemm_launch(128, -1, 128, ok_ptr, 0, ok_ptr, 0, ok_ptr, 2, None) == INVALID
    assert L.fp8gemm_launch(128, 128, 128, None, 0, ok_ptr, 0, ok_ptr, 2, None) == INVALID
    assert L.fp8gemm_launch(128, 128, 128, ok_ptr, 0, None, 0, ok_ptr, 2, None) == INVALID
    assert L.fp8gemm_launch(128, 128, 128, ok_ptr, 0, ok_ptr, 0, None, 2, None) == INVALID
    assert L.fp8gemm_launch(128, 128, 128, ok_ptr, 2, ok_ptr, 0, ok_ptr, 2, None) == INVALID
    assert L.fp8gemm_launch(128, 128, 128, ok_ptr, 0, ok_ptr, -1, ok_ptr, 2, None) == INVALID
    assert L.fp8gemm_launch(128, 128, 128, ok_ptr, 0, ok_ptr, 0, ok_ptr, 3, None) == INVALID
    assert L.fp8gemm_launch_algo(128, 128, 128, ok_ptr, 0, ok_ptr, 0, ok_ptr, 2, 9, None) == INVALID
    for name in pkg.ENTRY_POINTS:
        assert getattr(L, name)(128, 128, 128, None, None, None) == INVALID
        assert getattr(L, name)(128, 0, 128, ok_ptr, ok_ptr, ok_ptr) == INVALID
    # extended epilogue: output type code and alpha are checked as well
    assert L.fp8gemm_launch_ex(128, 128, 128, ok_ptr, 0, ok_ptr, 0, ok_ptr, 3, 1.0, None, None, None) == INVALID
    assert L.fp8gemm_launch_ex(128, 128, 128, ok_ptr, 0, ok_ptr, 0, ok_ptr, 1, float("nan"), None, None, None) == INVALID
    assert L.fp8gemm_launch_ex(128, 128, 128, ok_ptr, 0, ok_ptr, 0, None, 1, 1.0, None, None, None) == INVALID
    assert L.fp8gemm_launch_ex(0, 128, 128, ok_ptr, 0, ok_ptr, 0, ok_ptr, 0, 1.0, None, None, None) == INVALID
    assert b"invalid" in L.fp8gemm_error_string(INVALID).lower()
    assert L.fp8gemm_version() >= 100


def test_kernel_selection_is_pure_host_logic(pkg):
    L = pkg.lib()
    assert L.fp8gemm_select_algo(8192, 8192, 8192) == pkg.ALGO_TILE
    assert L.fp8gemm_select_algo(16, 8192, 28672) == pkg.ALGO_SKINNY
    assert L.fp8gemm_select_algo(1, 28672, 8192) == pkg.ALGO_SKINNY
    assert L.fp8gemm_select_algo(17, 8192, 10240) == pkg.ALGO_TILE       # from 17 rows on: the 64 x 128 streaming tile
    assert L.fp8gemm_select_algo(64, 8192, 10240) == pkg.ALGO_TILE
    assert L.fp8gemm_select_algo(256, 8192, 28672) == pkg.ALGO_TILE
    assert L.fp8gemm_select_algo(100, 100, 100) == pkg.ALGO_DIRECT       # k not a multiple of 16
    assert L.fp8gemm_select_algo(100, 112, 100) == pkg.ALGO_TILE         # k a multiple of 16: the last K tile overhangs
    assert L.fp8gemm_select_algo(512, 192, 512) == pkg.ALGO_TILE         # odd count of 64-byte K tiles
    assert L.fp8gemm_select_algo(16, 100, 64) == pkg.ALGO_DIRECT
    assert L.fp8gemm_select_algo(0, 1, 1) == -1
    assert L.fp8gemm_num_variants(pkg.ALGO_TILE) >= 2 and L.fp8gemm_num_variants(pkg.ALGO_SKINNY) >= 1
    assert L.fp8gemm_scratch_bytes(8192, 8192, 8192) == 0
    COUNTERS = 16 * 1024                   # arrival counters ahead of the partial sums
    s = L.fp8gemm_scratch_bytes(16, 28672, 8192)
    assert s == 0 or (s - COUNTERS) % (16 * 8192 * 4) == 0        # whole partial-sum planes, or none
    # the plan behind the automatic selection: family, variant, K slices, columns | rotation
    assert pkg.plan(8192, 8192, 8192) == (pkg.ALGO_TILE, 13, 1, 2)         # 256x256 persistent tiles on the 16x16x128 MFMA, no slices
    assert pkg.plan(8192, 8256, 8192) == (pkg.ALGO_TILE, 13, 1, 2)         # K not a multiple of 128: the same kernel, the last K tile overhangs
    assert pkg.plan(8192, 8192, 8192, stages=4)[:3] == (pkg.ALGO_TILE, 13, 1)        # shared with the 2-stage entry points
    assert pkg.plan(8192, 8256, 8192, stages=4)[:3] == (pkg.ALGO_TILE, 13, 1)        # ... for both entry points
    fam, var, slices, cols = pkg.plan(16, 8192, 28672)
    assert (fam, slices, cols) == (pkg.ALGO_SKINNY, 1, 64)
    fam, var, slices, _ = pkg.plan(256, 28672, 8192)
    assert fam == pkg.ALGO_TILE and slices > 1
    assert pkg.plan(100, 100, 100)[0] == pkg.ALGO_DIRECT
    for shape in [(256, 28672, 8192), (64, 28672, 8192), (300, 4096, 500), (8192, 8192, 8192), (7168, 7168, 7168)]:
        slices = pkg.plan(*shape)[2]
        assert (L.fp8gemm_scratch_bytes(*shape) > 0) == (slices > 1)
    # 64 rows: the 64 x 128 weight-streaming tile with a deep ring, K cut where the columns give too few tiles
    assert pkg.plan(64, 8192, 28672)[:3] == (pkg.ALGO_TILE, 15, 1)
    assert pkg.plan(64, 8192, 28672, stages=4)[:3] == (pkg.ALGO_TILE, 15, 1)         # its ring is 5 deep: both entry points
    fam, var, slices, _ = pkg.plan(64, 28672, 8192)
    assert (fam, var) == (pkg.ALGO_TILE, 15) and slices > 1
    assert L.fp8gemm_scratch_bytes(64, 28672, 8192) == COUNTERS + slices * (8192 // 128) * 64 * 128 * 4
    assert pkg.plan(128, 8192, 28672)[:3] == (pkg.ALGO_TILE, 16, 1)
    assert pkg.plan(16, 28672, 8192)[0] == pkg.ALGO_SKINNY
    # 28 x 28 tiles of 256 x 256: three rounds of whole tiles, the 16 left over cut into K slices
    fam, var, slices, mode = pkg.plan(7168, 7168, 7168)
    assert fam == pkg.ALGO_TILE and slices > 1 and mode >= 16
    assert L.fp8gemm_scratch_bytes(7168, 7168, 7168) == COUNTERS + slices * 16 * 256 * 256 * 4
    out = (ctypes.c_int * 4)()
    assert L.fp8gemm_plan(0, 1, 1, 2, out) == 1 and L.fp8gemm_plan(1, 1, 1, 3, out) == 1
    # few tiles and a long K: the tiled kernels cut K into slices, whole planes of partial sums
    s = L.fp8gemm_scratch_bytes(256, 28672, 8192)
    assert s >= 2 * 256 * 8192 * 4 and (s - COUNTERS) % (128 * 128 * 4) == 0


def test_generators_are_reproducible_and_counter_based(pkg):
    for dist in ("uniform", "normal", "weights", "loguniform"):
        for fmt in (0, 1):
            a = pkg.fill((300, 70), fmt, seed=42, dist=dist)
            b = pkg.fill((300, 70), fmt, seed=42, dist=dist)
            c = pkg.fill((300, 70), fmt, seed=43, dist=dist)
            assert np.array_equal(a, b) and not np.array_equal(a, c)
            if dist != "weights":     # element i depends on (seed, i) only: a prefix is a prefix
                assert np.array_equal(pkg.fill((100, 70), fmt, seed=42, dist=dist).ravel(), a.ravel()[:7000])


def test_generator_distributions(pkg, oracle):
    n = 400_000
    for fmt, top, lo in ((0, 448.0, 2.0 ** -9), (1, 57344.0, 2.0 ** -16)):
        x = oracle.decode(pkg.fill((n,), fmt, seed=7, dist="normal"), fmt)
        assert abs(x.mean()) < 0.01 and abs(x.std() - 1.0) < 0.03
        u = oracle.decode(pkg.fill((n,), fmt, seed=7, dist="uniform"), fmt)
        assert u.min() >= -1.0 and u.max() <= 1.0 and abs(u.mean()) < 0.01 and abs(u.std() - 3 ** -0.5) < 0.02
        w = oracle.decode(pkg.fill((n,), fmt, seed=7, dist="weights", sigma=0.02), fmt)
        assert np.abs(w).max() == top and abs(w.mean()) < top * 0.01
        g_codes = pkg.fill((n,), fmt, seed=7, dist="loguniform")
        g = oracle.decode(g_codes, fmt)
        assert np.isfinite(g).all() and np.abs(g).max() <= top
        nz = np.abs(g[g != 0])
        assert nz.min() == lo and nz.max() >= top / 2          # whole exponent range, subnormals included
        assert 0.45 < (g < 0).mean() < 0.55
        e = np.floor(np.log2(nz))
        counts = np.bincount((e - e.min()).astype(int))
        assert counts.min() > 0.5 * counts.mean()               # roughly flat over binades


def test_python_entry_points_refuse_host_tensors(pkg):
    import torch
    a = torch.zeros((16, 128), dtype=torch.uint8)
    with pytest.raises(pkg.Fp8GemmError):
        pkg.gemm(a, a, a_fmt=0, b_fmt=0)


def test_tile_order_is_a_bijection_with_compact_windows(pkg):
    """The persistent kernel's tile numbering (host copy of the device function): every tile
    exactly once, for plain strips and for the numbering in blocks of 16 tile columns; 32
    consecutive numbers (one XCD) touch at most two strips of 4 tile rows."""
    import ctypes
    L = pkg.lib()
    L.fp8gemm_tile_order.restype = ctypes.c_int
    L.fp8gemm_tile_order.argtypes = [ctypes.c_int] * 6 + [ctypes.POINTER(ctypes.c_int)] * 2
    tr, tc = ctypes.c_int(), ctypes.c_int()
    cases = [((1000, 512, 900), 256, 256), ((4352, 4352, 4352), 256, 256), ((300, 1024, 5000), 128, 128),
             ((4352, 12288, 16384), 256, 256),      # B of 192 MiB beside a smaller A: blocks of 16 tile columns
             ((1100, 16384, 20000), 192, 256), ((256, 1024, 256), 256, 256)]
    for (m, k, n), bm, bn in cases:
        tm, tn = -(-m // bm), -(-n // bn)
        seen = set()
        order = []
        for g in range(tm * tn):
            assert L.fp8gemm_tile_order(m, k, n, bm, bn, g, ctypes.byref(tr), ctypes.byref(tc)) == 0
            assert 0 <= tr.value < tm and 0 <= tc.value < tn
            seen.add((tr.value, tc.value))
            order.append((tr.value, tc.value))
        assert len(seen) == tm * tn, (m, k, n)
        for g0 in range(0, tm * tn - 31, 32):
            rows = {r for r, _ in order[g0:g0 + 32]}
            assert len(rows) <= 8, (m, k, n, g0)                  # at most two strips of 4 rows
    assert L.fp8gemm_tile_order(256, 256, 256, 256, 256, 1, ctypes.byref(tr), ctypes.byref(tc)) != 0
    # blocked numbering: the first 256 tiles of the 17 x 64 grid form a 16 x 16 window
    first = [None] * 256
    for g in range(256):
        L.fp8gemm_tile_order(4352, 12288, 16384, 256, 256, g, ctypes.byref(tr), ctypes.byref(tc))
        first[g] = (tr.value, tc.value)
    assert {r for r, _ in first} == set(range(16)) and {c for _, c in first} == set(range(16))


def test_plans_are_consistent_over_random_shapes(pkg):
    """Host-only sweep of the planner: whatever it picks can run the shape.  Streams: m <= 16,
    a column count per wave of 16, 32 or 64 that divides n, K slices that are whole 128-byte K
    steps.  Tiles: a compiled variant, slices only where K has K tiles to spare, scratch within
    the cap.  The scratch query agrees with the plan (arrival counters + whole fp32 planes / slots)."""
    L = pkg.lib()
    rng = np.random.default_rng(20240611)
    COUNTERS = 16 * 1024
    n_tile_variants = L.fp8gemm_num_variants(pkg.ALGO_TILE)
    n_stream_variants = L.fp8gemm_num_variants(pkg.ALGO_SKINNY)
    shapes = [(1, 8192, 10240), (16, 28672, 1024), (4, 16384, 2048), (16, 14336, 512), (17, 128, 16), (16, 128, 16)]
    for _ in range(3000):
        m = int(rng.choice([1, 2, 7, 16, 17, 33, 64, 100, 128, 256, 300, 1000, 4096, 5000]))
        k = int(rng.integers(1, 260)) * int(rng.choice([16, 64, 128]))
        n = int(rng.integers(1, 1800)) * int(rng.choice([1, 16, 16, 128]))
        shapes.append((m, k, n))
    compiled_tiles = {0, 5, 6, 8, 9, 13, 14, 15, 16}
    compiled_streams = {0, 1, 4, 5}
    for (m, k, n) in shapes:
        # the 2- and 4-stage entry points run the same plan (so one scratch figure serves both)
        assert pkg.plan(m, k, n, 4) == pkg.plan(m, k, n, 2)
        for stages in (2, 4):
            fam, var, slices, extra = pkg.plan(m, k, n, stages)
            assert fam == L.fp8gemm_select_algo(m, k, n)
            assert slices >= 1
            if fam == pkg.ALGO_SKINNY:
                assert m <= 16 and k % 128 == 0 and n % 16 == 0
                assert extra in (16, 32, 64) and n % extra == 0
                assert 0 <= var < n_stream_variants and var in compiled_streams
                assert k % (128 * slices) == 0
                if stages == 2:
                    want = COUNTERS + slices * m * n * 4 if slices > 1 else 0
                    assert L.fp8gemm_scratch_bytes(m, k, n) == want
            elif fam == pkg.ALGO_TILE:
                assert k % 16 == 0 and 0 <= var < n_tile_variants and var in compiled_tiles
                assert slices == 1 or (k + 127) // 128 >= 2 * slices
                if stages == 2:
                    need = L.fp8gemm_scratch_bytes(m, k, n)
                    assert (need > 0) == (slices > 1) and need <= (1 << 30) + COUNTERS
                    assert need == 0 or (need - COUNTERS) % 4096 == 0
            else:
                assert fam == pkg.ALGO_DIRECT and slices == 1 and L.fp8gemm_scratch_bytes(m, k, n) == 0
