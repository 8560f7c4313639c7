"""GPU parity: the HIP kernels, called through the C ABI, against the CPU oracle.

Bar (the reference's own CPU fp32 loop, GEMM/gemm_main.cpp:39-53, is the truth):
  |C_gpu - C_ref| <= 2*K*2^-24 * sum_k |a_ik * b_kj|   per element,
and bit-exact wherever no rounding can occur.
"""
import zlib

import numpy as np
import pytest

from conftest import finite_codes, random_codes

pytestmark = pytest.mark.gpu

PAIRS = [(0, 0), (1, 1), (0, 1), (1, 0)]
ALGOS = {"auto": 0, "direct": 1, "tile": 2, "skinny": 3}


def run_gpu(pkg, A, fa, B, fb, **kw):
    import torch
    dA = torch.from_numpy(A).cuda()
    dB = torch.from_numpy(B).cuda()
    out = torch.full((A.shape[0], B.shape[0]), float("nan"), dtype=torch.float32, device="cuda")
    pkg.gemm(dA, dB, out=out, a_fmt=fa, b_fmt=fb, **kw)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def mfma_window_term(oracle, A, fa, B, fb, block=8):
    """Extra error the f8f6f4 MFMA can add on top of reordered fp32 summation.

    Measured on MI355X and pinned by tests/test_gpu_mfma_numerics.py: the products of 8
    consecutive K bytes are added as a group, aligned to the group's largest product, keeping
    13 binary places below its leading bit (2^16 + 2^3 survives, 2^16 + 2^2 does not); groups,
    MFMAs and K tiles are added in plain fp32.  So each group can lose up to 2^-13 of its
    largest product per product.  Returned: 2^-13 * sum over groups of (8 * an upper bound of
    the group's largest |a*b|).
    """
    a = np.abs(oracle.decode(A, fa).astype(np.float64))
    b = np.abs(oracle.decode(B, fb).astype(np.float64))
    M, K = a.shape
    pad = (-K) % block
    if pad:
        a = np.pad(a, ((0, 0), (0, pad)))
        b = np.pad(b, ((0, 0), (0, pad)))
    # largest |a*b| of a group <= (largest |a| of the group) * (largest |b| of the group):
    # a matrix product of the group maxima instead of a pass over every product
    amax = a.reshape(M, -1, block).max(axis=2)
    bmax = b.reshape(b.shape[0], -1, block).max(axis=2)
    return (amax @ bmax.T) * block * 2.0 ** -13


def assert_within_bound(oracle, C, A, fa, B, fb, rows=None, hw_term=False, block=8):
    K = A.shape[1]
    Cref, S = oracle.gemm(A, fa, B, fb, rows=rows, with_scale=True)
    got = C if rows is None else C[rows]
    assert np.isfinite(got).all()
    err = np.abs(got.astype(np.float64) - Cref.astype(np.float64))
    tol = oracle.tolerance(K, S)
    if hw_term:
        term = mfma_window_term(oracle, A, fa, B, fb, block=block)
        tol = tol + (term if rows is None else term[rows])
    worst = float((err / np.maximum(tol, 1e-300)).max())
    assert (err <= tol).all(), "worst err/tol = %g" % worst
    return worst


SHAPES = [
    ("direct", (128, 128, 128)), ("direct", (37, 100, 53)), ("direct", (1, 1, 1)), ("direct", (65, 17, 33)),
    ("direct", (40, 1030, 70)),
    ("tile", (128, 128, 128)), ("tile", (256, 384, 512)), ("tile", (300, 256, 200)), ("tile", (512, 1024, 768)),
    ("tile", (1, 128, 1)),
    ("skinny", (16, 256, 64)), ("skinny", (1, 512, 128)), ("skinny", (13, 1024, 256)), ("skinny", (16, 512, 192)),
    ("skinny", (5, 2048, 80)),
]


@pytest.mark.parametrize("fa,fb", PAIRS)
@pytest.mark.parametrize("algo,shape", SHAPES)
def test_all_finite_codes(pkg, oracle, fa, fb, algo, shape):
    """Operands drawn uniformly from every finite code (subnormals, extremes, -0): the
    widest dynamic range the formats allow.  Bound = the fp32 reordering bound plus
    the MFMA alignment-window term measured for the hardware."""
    M, K, N = shape
    rng = np.random.default_rng(zlib.crc32(repr((fa, fb, algo, shape)).encode()))
    A = random_codes(rng, (M, K), fa)
    B = random_codes(rng, (N, K), fb)
    # keep e5m2 magnitudes below 2^10 so that fp32 sums cannot overflow
    if fa == 1:
        A = np.where(((A >> 2) & 0x1F) > 24, A & 0x83 | 0x3C, A).astype(np.uint8)
    if fb == 1:
        B = np.where(((B >> 2) & 0x1F) > 24, B & 0x83 | 0x3C, B).astype(np.uint8)
    C = run_gpu(pkg, A, fa, B, fb, algo=ALGOS[algo])
    assert_within_bound(oracle, C, A, fa, B, fb, hw_term=True)


@pytest.mark.parametrize("fa,fb", PAIRS)
@pytest.mark.parametrize("algo,shape", [
    ("direct", (64, 2048, 96)), ("tile", (256, 2048, 256)), ("tile", (384, 4096, 640)),
    ("skinny", (16, 4096, 512)), ("skinny", (9, 2048, 256)), ("skinny", (1, 8192, 256)),
    ("auto", (64, 4096, 1536)), ("auto", (33, 8192, 640)), ("auto", (17, 2048, 2048)), ("auto", (100, 4096, 1920)),
])
def test_normal_inputs_within_fp32_reordering_bound(pkg, oracle, fa, fb, algo, shape):
    """4*N(0,1) inputs (the four-pairings workload) against the plain bound
    |C_gpu - C_ref| <= 2*K*2^-24 * sum_k |a*b|."""
    M, K, N = shape
    A = pkg.fill((M, K), fa, seed=0xA11CE + K, dist="normal", sigma=4.0)
    B = pkg.fill((N, K), fb, seed=0xB0B + K, dist="normal", sigma=4.0)
    C = run_gpu(pkg, A, fa, B, fb, algo=ALGOS[algo])
    worst = assert_within_bound(oracle, C, A, fa, B, fb)
    assert worst < 0.25


@pytest.mark.parametrize("fa,fb", PAIRS)
@pytest.mark.parametrize("variant", [0, 5, 6, 8, 9, 15, 16])
@pytest.mark.parametrize("shape", [(256, 256, 256), (300, 512, 200), (1000, 1024, 900), (513, 384, 257), (64, 128, 2048),
                                   (40, 640, 1000)])
def test_every_tile_variant(pkg, oracle, variant, shape, fa, fb):
    """Each compiled shape of the tiled kernel on the 32x32x64 MFMA, on shapes that overhang
    the tile in m and n, for all four pairings."""
    M, K, N = shape
    rng = np.random.default_rng(zlib.crc32(repr((variant, shape, fa, fb)).encode()))
    A = random_codes(rng, (M, K), fa)
    B = random_codes(rng, (N, K), fb)
    if fa == 1:
        A = np.where(((A >> 2) & 0x1F) > 24, A & 0x83 | 0x3C, A).astype(np.uint8)
    if fb == 1:
        B = np.where(((B >> 2) & 0x1F) > 24, B & 0x83 | 0x3C, B).astype(np.uint8)
    C = run_gpu(pkg, A, fa, B, fb, algo=ALGOS["tile"], variant=variant)
    assert_within_bound(oracle, C, A, fa, B, fb, hw_term=True)


@pytest.mark.parametrize("shape", [(256, 256, 256), (300, 512, 200), (1000, 1024, 900), (513, 768, 257), (64, 256, 2048),
                                   (768, 2048, 1280), (300, 384, 300), (512, 1152, 256), (256, 640, 512)])
@pytest.mark.parametrize("fa,fb", PAIRS)
@pytest.mark.parametrize("variant", [13, 14])
def test_tile_variant_on_16x16x128_mfma(pkg, oracle, variant, fa, fb, shape):
    """The 256 x 256 and 192 x 256 persistent tiles computed with v_mfma_f32_16x16x128_f8f6f4
    (variants 13, 14; K a multiple of 128, odd and even counts of K tiles), all four pairings,
    on shapes that overhang the tile in m and n."""
    M, K, N = shape
    rng = np.random.default_rng(zlib.crc32(repr((variant, fa, fb, shape)).encode()))
    A = random_codes(rng, (M, K), fa)
    B = random_codes(rng, (N, K), fb)
    if fa == 1:
        A = np.where(((A >> 2) & 0x1F) > 24, A & 0x83 | 0x3C, A).astype(np.uint8)
    if fb == 1:
        B = np.where(((B >> 2) & 0x1F) > 24, B & 0x83 | 0x3C, B).astype(np.uint8)
    C = run_gpu(pkg, A, fa, B, fb, algo=ALGOS["tile"], variant=variant)
    assert_within_bound(oracle, C, A, fa, B, fb, hw_term=True)


@pytest.mark.parametrize("fa,fb", PAIRS)
@pytest.mark.parametrize("variant", [13, 14])
@pytest.mark.parametrize("shape", [(300, 144, 200), (512, 2000, 520), (1100, 4112, 700), (256, 8256, 512), (700, 1216, 300)])
def test_16x16x128_variants_with_an_overhanging_last_k_tile(pkg, oracle, variant, fa, fb, shape):
    """K a multiple of 16 but not of 128 (even and odd counts of K tiles, K a multiple of 64 or
    not): the bytes of the last K tile past the end of each row count as zeros in the
    16x16x128 kernels as well, all four pairings; K slices over such a K included."""
    M, K, N = shape
    assert K % 16 == 0 and K % 128 != 0
    A = pkg.fill((M, K), fa, seed=0xA11CE + K + variant, dist="normal", sigma=4.0)
    B = pkg.fill((N, K), fb, seed=0xB0B + K + variant, dist="normal", sigma=4.0)
    C = run_gpu(pkg, A, fa, B, fb, algo=ALGOS["tile"], variant=variant)
    worst = assert_within_bound(oracle, C, A, fa, B, fb, hw_term=K < 1024)
    assert worst < 0.5
    if (K + 127) // 128 >= 4:
        C2 = run_gpu(pkg, A, fa, B, fb, algo=ALGOS["tile"], variant=variant, split_k=2)
        assert_within_bound(oracle, C2, A, fa, B, fb, hw_term=K < 1024)


@pytest.mark.parametrize("variant", [13, 14])
def test_16x16x128_variant_refuses_a_single_k_tile(pkg, variant):
    A = np.zeros((256, 128), np.uint8)
    B = np.zeros((256, 128), np.uint8)
    with pytest.raises(RuntimeError):
        run_gpu(pkg, A, 0, B, 0, algo=ALGOS["tile"], variant=variant)


@pytest.mark.parametrize("variant,split", [(0, 2), (0, 3), (9, 5), (5, 4), (5, 7), (6, 2), (6, 16), (8, 3), (13, 2), (13, 4), (14, 3),
                                           (15, 3), (15, 4), (16, 2)])
@pytest.mark.parametrize("shape", [(256, 2048, 512), (300, 4096, 200), (1000, 2304, 900), (128, 8192, 2048)])
def test_tile_k_slices(pkg, oracle, variant, split, shape):
    """Persistent tiled kernels with the K range cut into slices whose partial sums are
    added by the reduction kernel (uneven slices included), on shapes that overhang the tile."""
    M, K, N = shape
    if variant in (13, 14) and (K // 128) // split < 2:
        pytest.skip("the 16x16x128 variant takes at least two 128-byte K tiles per slice")
    A = pkg.fill((M, K), 1, seed=0xA11CE + K + split, dist="normal", sigma=4.0)
    B = pkg.fill((N, K), 0, seed=0xB0B + K + split, dist="normal", sigma=4.0)
    C = run_gpu(pkg, A, 1, B, 0, algo=ALGOS["tile"], variant=variant, split_k=split)
    worst = assert_within_bound(oracle, C, A, 1, B, 0)
    assert worst < 0.25


@pytest.mark.parametrize("variant,split,shape", [
    (6, -3, (2200, 2048, 2300)),      # 18 x 18 tiles of 128 x 128: 256 whole items + 68 tail tiles in 3 slices
    (6, -2, (2304, 1024, 2304)),
    (5, -4, (2100, 1536, 4500)),      # 17 x 18 tiles of 128 x 256
    (0, -2, (4200, 1024, 4300)),      # 17 x 17 tiles of 256 x 256
    (8, -5, (4352, 1280, 2200)),      # 17 x 18 tiles of 256 x 128
    (9, -2, (3300, 1152, 4352)),      # 18 x 17 tiles of 192 x 256
])
def test_tile_k_slices_for_the_last_partial_round(pkg, oracle, variant, split, shape):
    """More tiles than CUs: the rounds of 256 whole tiles write C directly, the tiles left
    over are cut into K slices that go through the scratch and the reduction kernel."""
    M, K, N = shape
    A = pkg.fill((M, K), 0, seed=0xA11CE + K - split, dist="normal", sigma=4.0)
    B = pkg.fill((N, K), 1, seed=0xB0B + K - split, dist="normal", sigma=4.0)
    C = run_gpu(pkg, A, 0, B, 1, algo=ALGOS["tile"], variant=variant, split_k=split)
    rows = np.arange(0, M, 5, dtype=np.int32)
    worst = assert_within_bound(oracle, C, A, 0, B, 1, rows=rows)
    assert worst < 0.25
    # every element was written (the NaN fill is gone), the leftover tiles included
    assert np.isfinite(C).all()


@pytest.mark.parametrize("variant", [None, 0, 5, 6])
@pytest.mark.parametrize("shape", [(256, 16, 256), (300, 1000 // 16 * 16 + 16, 200), (512, 2000, 520), (1100, 4112, 700),
                                   (64, 1040, 512), (16, 8176, 1024)])
def test_k_that_is_only_a_multiple_of_16(pkg, oracle, variant, shape):
    """The last K tile overhangs K: its bytes past the end of each row must count as zeros,
    not as the next row's bytes.  Every persistent tile shape, and the automatic selection
    (which no longer needs the general kernel for these)."""
    M, K, N = shape
    assert K % 16 == 0 and K % 64 != 0
    assert pkg.lib().fp8gemm_select_algo(M, K, N) == ALGOS["tile"]
    A = pkg.fill((M, K), 1, seed=0xA11CE + K, dist="normal", sigma=4.0)
    B = pkg.fill((N, K), 0, seed=0xB0B + K, dist="normal", sigma=4.0)
    if variant is None:
        C = run_gpu(pkg, A, 1, B, 0)
    else:
        C = run_gpu(pkg, A, 1, B, 0, algo=ALGOS["tile"], variant=variant)
    worst = assert_within_bound(oracle, C, A, 1, B, 0, hw_term=K < 1024)
    assert worst < 0.5


@pytest.mark.parametrize("variant", [0, 6, None])
@pytest.mark.parametrize("shape", [(256, 64, 256), (300, 192, 200), (1100, 448, 2100), (2048, 8256, 2304)])
def test_odd_count_of_64_byte_k_tiles(pkg, oracle, variant, shape):
    """k % 64 == 0 but k % 128 != 0 (the reference's own requirement is k % 64 == 0,
    GEMM/src/gemm.cu:45-47): the last 128-byte K tile is half empty, whether the kernel is
    picked by hand or by the automatic selection."""
    M, K, N = shape
    assert pkg.lib().fp8gemm_select_algo(M, K, N) == ALGOS["tile"]
    A = pkg.fill((M, K), 0, seed=0xA11CE + K, dist="normal", sigma=4.0)
    B = pkg.fill((N, K), 1, seed=0xB0B + K, dist="normal", sigma=4.0)
    if variant is None:
        C = run_gpu(pkg, A, 0, B, 1)
    else:
        C = run_gpu(pkg, A, 0, B, 1, algo=ALGOS["tile"], variant=variant)
    rows = None if M * N * K < 2 ** 31 else np.arange(0, M, 16, dtype=np.int32)
    # one or a few MFMAs per output: their internal alignment window shows next to the
    # K-proportional bound
    worst = assert_within_bound(oracle, C, A, 0, B, 1, rows=rows, hw_term=K < 1024)
    assert worst < 0.25


@pytest.mark.parametrize("stages", [2, 4])
@pytest.mark.parametrize("fa,fb", PAIRS)
def test_entry_points_stage2_stage4(pkg, oracle, fa, fb, stages):
    """The eight per-precision entry points (GEMM / GEMM4 of the reference), default stream."""
    import torch
    M, K, N = 512, 1024, 768
    A = pkg.fill((M, K), fa, seed=3, dist="normal", sigma=4.0)
    B = pkg.fill((N, K), fb, seed=4, dist="normal", sigma=4.0)
    dt = {0: torch.float8_e4m3fn, 1: torch.float8_e5m2}
    dA = torch.from_numpy(A).cuda().view(dt[fa])
    dB = torch.from_numpy(B).cuda().view(dt[fb])
    out = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    fn = pkg.GEMM if stages == 2 else pkg.GEMM4
    assert fn(M, K, N, dA, dB, out) == 0
    torch.cuda.synchronize()
    assert_within_bound(oracle, out.cpu().numpy(), A, fa, B, fb)


@pytest.mark.parametrize("fa,fb", PAIRS)
@pytest.mark.parametrize("algo", ["direct", "tile", "skinny"])
def test_decode_through_mfma_is_bit_exact(pkg, oracle, fa, fb, algo):
    """One-hot A with value 1.0 selects single entries of B: C[i, j] == decode(B[j, k_i])
    exactly, for every finite code, and likewise with the roles swapped."""
    one = {0: 0x38, 1: 0x3C}
    K = 256
    M = 16 if algo == "skinny" else 256
    N = 256
    rng = np.random.default_rng(7)
    ks = rng.permutation(K)[:M] if M <= K else rng.integers(0, K, M)
    A = np.zeros((M, K), dtype=np.uint8)
    A[np.arange(M), ks] = one[fa]
    codes = finite_codes(fb)
    B = codes[rng.integers(0, codes.size, (N, K))]
    B[:, ks[0]] = np.resize(codes, N)            # every finite code appears at least once
    C = run_gpu(pkg, A, fa, B, fb, algo=ALGOS[algo])
    expect = oracle.decode(B, fb)[:, ks].T       # (M, N)
    assert np.array_equal(C.view(np.uint32) & 0x7FFFFFFF, expect.view(np.uint32) & 0x7FFFFFFF)
    assert np.array_equal(C, expect)
    # swapped roles: one-hot B selects entries of A (every finite code of A's format appears)
    codes_a = finite_codes(fa)
    A2 = codes_a[rng.integers(0, codes_a.size, (M, K))]
    A2[:, 0] = np.resize(codes_a, M)
    A2[0, :codes_a.size] = codes_a[:K]
    B2 = np.zeros((N, K), dtype=np.uint8)
    kn = rng.integers(0, K, N)
    kn[:K] = rng.permutation(K)[:min(K, N)]
    B2[np.arange(N), kn] = one[fb]
    C2 = run_gpu(pkg, A2, fa, B2, fb, algo=ALGOS[algo])
    assert np.array_equal(C2, oracle.decode(A2, fa)[:, kn])


@pytest.mark.parametrize("algo,variant", [("tile", 13), ("tile", 14), ("tile", 5), ("tile", 6), ("tile", 8), ("tile", 9), ("tile", 15),
                                          ("tile", 16)])
@pytest.mark.parametrize("fa,fb", PAIRS)
def test_decode_through_mfma_every_persistent_form(pkg, oracle, fa, fb, algo, variant):
    """The same bit-exact selection test for the persistent tile shapes the planner uses
    (both MFMA shapes, rings 2 to 5 slots deep): one-hot A selects codes of B and one-hot B
    selects codes of A, K = 512 so that the 16x16x128 forms see four K tiles."""
    one = {0: 0x38, 1: 0x3C}
    M, K, N = 384, 512, 512
    rng = np.random.default_rng(1000 + variant)
    codes_a, codes_b = finite_codes(fa), finite_codes(fb)
    ks = rng.integers(0, K, M)
    A = np.zeros((M, K), dtype=np.uint8)
    A[np.arange(M), ks] = one[fa]
    B = codes_b[rng.integers(0, codes_b.size, (N, K))]
    B[:, ks[0]] = np.resize(codes_b, N)
    C = run_gpu(pkg, A, fa, B, fb, algo=ALGOS[algo], variant=variant)
    assert np.array_equal(C, oracle.decode(B, fb)[:, ks].T)
    A2 = codes_a[rng.integers(0, codes_a.size, (M, K))]
    A2[:, 3] = np.resize(codes_a, M)
    kn = rng.integers(0, K, N)
    kn[0] = 3
    B2 = np.zeros((N, K), dtype=np.uint8)
    B2[np.arange(N), kn] = one[fb]
    C2 = run_gpu(pkg, A2, fa, B2, fb, algo=ALGOS[algo], variant=variant)
    assert np.array_equal(C2, oracle.decode(A2, fa)[:, kn])


def test_tall_general_kernel_shape_beyond_65535_row_tiles(pkg, oracle):
    """m = 3,000,000 rows with a K that only the general kernel takes (k % 16 != 0): the grid
    is one-dimensional, so neither tile count is capped at 65535."""
    M, K, N = 3_000_000, 8, 16
    assert pkg.lib().fp8gemm_select_algo(M, K, N) == ALGOS["direct"]
    rng = np.random.default_rng(77)
    vals = np.arange(-8, 9, dtype=np.float32)           # small integers: every sum is exact
    Af = vals[rng.integers(0, vals.size, (M, K))]
    Bf = vals[rng.integers(0, vals.size, (N, K))]
    C = run_gpu(pkg, oracle.encode(Af, 0), 0, oracle.encode(Bf, 1), 1)
    assert np.array_equal(C, Af @ Bf.T)


@pytest.mark.parametrize("algo,shape", [("direct", (96, 200, 64)), ("tile", (256, 1024, 256)), ("skinny", (12, 1024, 128))])
def test_small_integers_are_exact(pkg, oracle, algo, shape):
    """|values| <= 8 and K <= 2^10: every partial sum is an integer below 2^24, so any
    summation order gives the same bits as the oracle."""
    M, K, N = shape
    rng = np.random.default_rng(11)
    vals = np.arange(-8, 9, dtype=np.float32)
    A = oracle.encode(vals[rng.integers(0, vals.size, (M, K))], 0)
    B = oracle.encode(vals[rng.integers(0, vals.size, (N, K))], 1)
    C = run_gpu(pkg, A, 0, B, 1, algo=ALGOS[algo])
    Cref = oracle.gemm(A, 0, B, 1)
    assert np.array_equal(C, Cref)
    ints = oracle.decode(A, 0).astype(np.int64) @ oracle.decode(B, 1).astype(np.int64).T
    assert np.array_equal(C.astype(np.int64), ints)


@pytest.mark.parametrize("shape", [(256, 8192, 2048), (2200, 2048, 2300), (1000, 1040, 900), (512, 4096, 4096),
                                   (128, 8192, 4096), (3000, 512, 3000), (64, 4096, 512), (77, 200, 33)])
def test_stage4_entry_follows_the_same_plans(pkg, oracle, shape):
    """The 4-stage entry points (gemm::GEMM4) on shapes whose plans use K slices, leftover-tile
    slices, an overhanging K tile, the weight-streaming and the general kernel."""
    M, K, N = shape
    A = pkg.fill((M, K), 0, seed=0xA11CE + K + 4, dist="normal", sigma=4.0)
    B = pkg.fill((N, K), 1, seed=0xB0B + K + 4, dist="normal", sigma=4.0)
    C = run_gpu(pkg, A, 0, B, 1, stages=4)
    rows = None if M * N * K < 2 ** 33 else np.arange(0, M, 4, dtype=np.int32)
    worst = assert_within_bound(oracle, C, A, 0, B, 1, rows=rows, hw_term=K < 1024)
    assert worst < 0.5


@pytest.mark.parametrize("variant,split", [(13, -2), (0, 0), (14, 0)])
def test_column_blocked_tile_numbering(pkg, oracle, variant, split):
    """B of 192 MiB and more beside a smaller A: the tiles are numbered in blocks of 16 tile columns (whole rounds,
    leftover tiles cut into K slices and their reduction all use that numbering).  Sampled rows
    against the oracle, every tile row and every column covered."""
    M, K, N = 4352, 12288, 16384
    A = pkg.fill((M, K), 0, seed=0xC0FFEE, dist="normal", sigma=1.0)
    B = pkg.fill((N, K), 0, seed=0xBEEF, dist="normal", sigma=1.0)
    C = run_gpu(pkg, A, 0, B, 0, algo=ALGOS["tile"], variant=variant, split_k=split)
    rows = np.arange(5, M, 251, dtype=np.int32)
    worst = assert_within_bound(oracle, C, A, 0, B, 0, rows=rows)
    assert worst < 0.25
    # every row: the row sums of C against A times the column sums of B (exact in float64 up to the kernel's rounding)
    bsum = oracle.decode(B, 0).astype(np.float64).sum(axis=0)
    want = oracle.decode(A, 0).astype(np.float64) @ bsum
    got = C.astype(np.float64).sum(axis=1)
    assert np.abs(got - want).max() <= 1e-3 * np.abs(C).astype(np.float64).sum(axis=1).max()


def test_scratch_grows_and_is_reused_across_calls_and_streams(pkg, oracle):
    """Calls that need the partial-sum scratch, in growing and shrinking order, on the default
    stream and on a side stream: every result is right, before and after a stream's buffer
    has been replaced by a larger one."""
    import torch
    shapes = [(256, 8192, 1024), (256, 8192, 2048), (256, 8192, 1024), (300, 6144, 1000), (256, 8192, 2048)]
    side = torch.cuda.Stream()
    need = [pkg.lib().fp8gemm_scratch_bytes(*s) for s in shapes]
    assert need[0] > 0 and need[1] > need[0]           # the second call has to grow the buffer
    for idx, (M, K, N) in enumerate(shapes):
        A = pkg.fill((M, K), 0, seed=0xA11CE + 100 + idx, dist="normal", sigma=4.0)
        B = pkg.fill((N, K), 0, seed=0xB0B + 100 + idx, dist="normal", sigma=4.0)
        dA = torch.from_numpy(A).cuda()
        dB = torch.from_numpy(B).cuda()
        out = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()
        if idx % 2:
            with torch.cuda.stream(side):
                pkg.gemm(dA, dB, out=out, a_fmt=0, b_fmt=0, stream=side)
            side.synchronize()
        else:
            pkg.gemm(dA, dB, out=out, a_fmt=0, b_fmt=0)
            torch.cuda.synchronize()
        worst = assert_within_bound(oracle, out.cpu().numpy(), A, 0, B, 0)
        assert worst < 0.25, (idx, worst)
    assert pkg.lib().fp8gemm_scratch_held_bytes() >= max(need)
    assert pkg.lib().fp8gemm_release_scratch() == 0
    assert pkg.lib().fp8gemm_scratch_held_bytes() == 0


def test_k_sliced_launches_overlap_on_two_streams_without_caller_ordering(pkg, oracle):
    """Two streams, each queueing K-sliced GEMMs (which go through the scratch and the
    reduction kernel) back to back with no ordering between the streams and no host
    synchronisation: the launch functions are re-entrant like the reference's
    (GEMM/src/gemm.cu:263-277), so every output is right.  The grids are small enough
    (64 workgroups on 256 CUs) for kernels of the two streams to run side by side; one
    stream also grows its buffer in the middle of the sequence."""
    import torch
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    shapes = [[(256, 8192, 1024), (128, 8192, 2048), (256, 8192, 1024), (256, 8192, 2048)],
              [(128, 8192, 4096), (256, 8192, 1024), (300, 6144, 1000), (256, 8192, 1024)]]
    for sh in shapes[0] + shapes[1]:
        assert pkg.plan(*sh)[2] > 1                    # every shape here is cut into K slices
    cases = [[], []]
    for s in range(2):
        for idx in range(12):
            M, K, N = shapes[s][idx % 4]
            A = pkg.fill((M, K), 0, seed=0xA11CE + 300 + 50 * s + idx, dist="normal", sigma=2.0)
            B = pkg.fill((N, K), 1, seed=0xB0B + 300 + 50 * s + idx, dist="normal", sigma=2.0)
            cases[s].append((A, B, torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(),
                             torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")))
    torch.cuda.synchronize()
    for idx in range(12):
        for s in range(2):
            A, B, dA, dB, out = cases[s][idx]
            pkg.gemm(dA, dB, out=out, a_fmt=0, b_fmt=1, stream=streams[s])
    torch.cuda.synchronize()
    for s in range(2):
        for A, B, dA, dB, out in cases[s]:
            worst = assert_within_bound(oracle, out.cpu().numpy(), A, 0, B, 1)
            assert worst < 0.25


def test_caller_provided_workspace(pkg, oracle):
    """fp8gemm_launch_ws: the K slices' partial sums go to the caller's buffer; too small a
    buffer is refused with hipErrorOutOfMemory before anything is launched; results equal
    those of fp8gemm_launch bit for bit (same plan, same kernels)."""
    import torch
    L = pkg.lib()
    stream = torch.cuda.current_stream().cuda_stream
    for (M, K, N), stages in [((256, 8192, 2048), 2), ((64, 8192, 2048), 2), ((512, 1024, 768), 2),
                              ((256, 28672, 10240), 4), ((256, 4912, 6144), 4)]:
        need = L.fp8gemm_scratch_bytes(M, K, N)
        A = pkg.fill((M, K), 0, seed=0xA11CE + 500 + M, dist="normal", sigma=2.0)
        B = pkg.fill((N, K), 0, seed=0xB0B + 500 + M, dist="normal", sigma=2.0)
        dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
        ref = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        pkg.gemm(dA, dB, out=ref, a_fmt=0, b_fmt=0, stages=stages)
        got = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
        held = L.fp8gemm_scratch_held_bytes()
        code = L.fp8gemm_launch_ws(M, K, N, dA.data_ptr(), 0, dB.data_ptr(), 0, got.data_ptr(), stages,
                                   ws.data_ptr() if need else None, need, stream)
        assert code == 0
        torch.cuda.synchronize()
        assert L.fp8gemm_scratch_held_bytes() == held       # the library allocated nothing
        assert torch.equal(got, ref)
        assert_within_bound(oracle, got.cpu().numpy(), A, 0, B, 0)
        if need:
            got.fill_(float("nan"))
            assert L.fp8gemm_launch_ws(M, K, N, dA.data_ptr(), 0, dB.data_ptr(), 0, got.data_ptr(), stages,
                                       ws.data_ptr(), need - 1, stream) == 2
            assert L.fp8gemm_launch_ws(M, K, N, dA.data_ptr(), 0, dB.data_ptr(), 0, got.data_ptr(), stages,
                                       None, 0, stream) == 2
            assert L.fp8gemm_launch_ws(M, K, N, dA.data_ptr(), 0, dB.data_ptr(), 0, got.data_ptr(), stages,
                                       ws.data_ptr() + 4, need, stream) == 1      # misaligned workspace
            torch.cuda.synchronize()
            assert bool(torch.isnan(got).all())             # nothing was launched


def test_k_slices_summed_inside_the_kernel_equal_the_reduction_kernel(pkg):
    """With the library's own scratch the slice of a tile that arrives last adds the slices up
    inside the kernel; with a caller's workspace (whose arrival counters cannot be relied on) a
    reduction kernel follows.  Both add in slice order: equal bit for bit, on ragged shapes, on
    every tile shape the planner picks for them, and on every one of several launches in a row
    (the counters are back at zero after each)."""
    import torch
    L = pkg.lib()
    stream = torch.cuda.current_stream().cuda_stream
    shapes = [(300, 4096, 500), (100, 8192, 1000), (257, 4096, 1023), (1000, 8192, 1000), (64, 28672, 8192),
              (64, 8192, 10240), (256, 8192, 10240), (7168, 7168, 7168)]
    for (M, K, N) in shapes:
        assert pkg.plan(M, K, N)[0] == pkg.ALGO_TILE and pkg.plan(M, K, N)[2] > 1
        need = L.fp8gemm_scratch_bytes(M, K, N)
        dA = torch.from_numpy(pkg.fill((M, K), 0, seed=0xA11CE + 900 + M, dist="normal", sigma=2.0)).cuda()
        dB = torch.from_numpy(pkg.fill((N, K), 1, seed=0xB0B + 900 + N, dist="normal", sigma=2.0)).cuda()
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        ref = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        assert L.fp8gemm_launch_ws(M, K, N, dA.data_ptr(), 0, dB.data_ptr(), 1, ref.data_ptr(), 2,
                                   ws.data_ptr(), need, stream) == 0
        # (many launches back to back on the small shapes: a slice whose partial sums were not yet
        # visible to the workgroup that adds them up would show as a mismatch now and then)
        outs = [torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda") for _ in range(60 if M * N <= 1 << 20 else 4)]
        for out in outs:
            pkg.gemm(dA, dB, out=out, a_fmt=0, b_fmt=1)
        torch.cuda.synchronize()
        assert not bool(torch.isnan(ref).any())
        for out in outs:
            assert torch.equal(out, ref), (M, K, N)
        del dA, dB, ws, ref, outs


@pytest.mark.parametrize("fw,fx", PAIRS)
@pytest.mark.parametrize("shape", [(4096, 4096), (10240, 8192), (1000, 8192), (512, 1040), (333, 777), (28672, 2048)])
def test_gemv_entry_point(pkg, oracle, fw, fx, shape):
    """fp8gemm_gemv: y = W x against the CPU loop with one row of A (all four pairings; shapes
    the streaming kernel takes, shapes that fall to the tiled kernel and to the general one),
    and bit-equal to fp8gemm_launch with m = 1."""
    import torch
    L = pkg.lib()
    N, K = shape
    W = pkg.fill((N, K), fw, seed=0xB0B + 1100 + N, dist="normal", sigma=2.0)
    x = pkg.fill((1, K), fx, seed=0xA11CE + 1100 + K, dist="normal", sigma=2.0)
    dW, dx = torch.from_numpy(W).cuda(), torch.from_numpy(x).cuda()
    y = torch.full((N,), float("nan"), dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    assert L.fp8gemm_gemv(N, K, dW.data_ptr(), fw, dx.data_ptr(), fx, y.data_ptr(), stream) == 0
    ref = torch.full((1, N), float("nan"), dtype=torch.float32, device="cuda")
    assert L.fp8gemm_launch(1, K, N, dx.data_ptr(), fx, dW.data_ptr(), fw, ref.data_ptr(), 2, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(y, ref[0])
    assert_within_bound(oracle, y.cpu().numpy()[None, :], x, fx, W, fw, hw_term=K < 1024)
    assert L.fp8gemm_gemv(0, K, dW.data_ptr(), fw, dx.data_ptr(), fx, y.data_ptr(), stream) == 1
    assert L.fp8gemm_gemv(N, K, None, fw, dx.data_ptr(), fx, y.data_ptr(), stream) == 1


def test_back_to_back_launches_without_synchronisation(pkg, oracle):
    """Twenty launches of alternating shapes queued on one stream with no host
    synchronisation in between (stream order is the only ordering): each output is right."""
    import torch
    cases = []
    for idx in range(20):
        M, K, N = [(16, 2048, 1024), (512, 1024, 768), (256, 8192, 1024), (1, 4096, 256)][idx % 4]
        A = pkg.fill((M, K), idx % 2, seed=0xA11CE + 200 + idx, dist="normal", sigma=2.0)
        B = pkg.fill((N, K), 0, seed=0xB0B + 200 + idx, dist="normal", sigma=2.0)
        cases.append((A, B, torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(),
                      torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda"), idx % 2))
    torch.cuda.synchronize()
    for A, B, dA, dB, out, fa in cases:
        pkg.gemm(dA, dB, out=out, a_fmt=fa, b_fmt=0)
    torch.cuda.synchronize()
    for A, B, dA, dB, out, fa in cases:
        assert_within_bound(oracle, out.cpu().numpy(), A, fa, B, 0)


def test_random_shapes_against_the_general_kernel(pkg, oracle):
    """Eighty seeded random shapes, pairings and stage counts through the automatic selection,
    each compared on the GPU with the general kernel (one wave per 32 x 32 tile, no LDS, a
    different summation order) within twice the fp32 reordering bound; the general kernel
    itself is pinned against the CPU oracle by the tests above."""
    import torch
    rng = np.random.default_rng(20240611)
    luts = [torch.from_numpy(oracle.decode(np.arange(256, dtype=np.uint8), f).astype(np.float64)).cuda() for f in (0, 1)]
    families = set()
    for case in range(80):
        kind = rng.integers(0, 4)
        if kind == 0:      # mid / large, K a multiple of 16
            M, N, K = int(rng.integers(65, 3000)), int(rng.integers(1, 3000)), 16 * int(rng.integers(1, 300))
        elif kind == 1:    # few rows
            M, N, K = int(rng.integers(1, 65)), 16 * int(rng.integers(1, 400)), 128 * int(rng.integers(1, 64))
        elif kind == 2:    # anything
            M, N, K = int(rng.integers(1, 700)), int(rng.integers(1, 700)), int(rng.integers(1, 1500))
        else:              # long K, few tiles
            M, N, K = int(rng.integers(1, 600)), int(rng.integers(1, 1200)), 128 * int(rng.integers(32, 160))
        fa, fb = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        stages = int(rng.choice([2, 4]))
        families.add(pkg.plan(M, K, N, stages)[0])
        A = pkg.fill((M, K), fa, seed=1000 + case, dist="normal", sigma=2.0)
        B = pkg.fill((N, K), fb, seed=2000 + case, dist="normal", sigma=2.0)
        dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
        got = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        ref = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        pkg.gemm(dA, dB, out=got, a_fmt=fa, b_fmt=fb, stages=stages)
        pkg.gemm(dA, dB, out=ref, a_fmt=fa, b_fmt=fb, algo=ALGOS["direct"])
        torch.cuda.synchronize()
        S = luts[fa][dA.long()].abs() @ luts[fb][dB.long()].abs().T
        bound = 2.0 * (2.0 * K * 2.0 ** -24) * S + 1e-30
        err = (got.double() - ref.double()).abs()
        assert bool(torch.isfinite(got).all()), (case, M, K, N)
        # small K: the MFMA's internal alignment window (about 2^-13 of a block's largest product) shows
        window = 2.0 ** -12 * S if K < 1024 else 0.0
        ok = err <= bound + window
        assert bool(ok.all()), (case, M, K, N, fa, fb, stages, float((err / (bound + window + 1e-30)).max()))
    assert families == {1, 2, 3}          # the draw exercised all three kernel families
