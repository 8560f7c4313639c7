"""The CPU oracle's GEMM (restating GEMM/gemm_main.cpp:39-53 of the reference): pinned by
cases whose answer arithmetic fixes without rerunning the oracle's own formula."""
import numpy as np
import pytest

from conftest import finite_codes, random_codes

PAIRS = [(0, 0), (1, 1), (0, 1), (1, 0)]


def tame(codes, fmt):
    """Keep e5m2 magnitudes below 2^10 so that fp32 sums stay finite."""
    if fmt == 1:
        return np.where(((codes >> 2) & 0x1F) > 24, codes & 0x83 | 0x3C, codes).astype(np.uint8)
    return codes


@pytest.mark.parametrize("fa,fb", PAIRS)
def test_fast_form_is_bit_identical_to_the_reference_loop_order(oracle, fa, fb):
    rng = np.random.default_rng(1 + fa * 2 + fb)
    for (M, K, N) in [(64, 256, 96), (33, 100, 70), (1, 7, 1), (256, 256, 256), (5, 1024, 37)]:
        A = tame(random_codes(rng, (M, K), fa), fa)
        B = tame(random_codes(rng, (N, K), fb), fb)
        C0 = oracle.gemm_verbatim(A, fa, B, fb)
        C1, S = oracle.gemm(A, fa, B, fb, with_scale=True)
        assert np.array_equal(C0.view(np.uint32), C1.view(np.uint32))
        rows = np.array([M - 1, 0], dtype=np.int32)
        C2 = oracle.gemm(A, fa, B, fb, rows=rows)
        assert np.array_equal(C2.view(np.uint32), C0[rows].view(np.uint32))


@pytest.mark.parametrize("fa,fb", PAIRS)
def test_all_ones_gives_k(oracle, fa, fb):
    one = {0: 0x38, 1: 0x3C}
    M, K, N = 9, 777, 11
    A = np.full((M, K), one[fa], dtype=np.uint8)
    B = np.full((N, K), one[fb], dtype=np.uint8)
    assert np.array_equal(oracle.gemm(A, fa, B, fb), np.full((M, N), float(K), dtype=np.float32))
    assert np.array_equal(oracle.gemm_verbatim(A, fa, B, fb), np.full((M, N), float(K), dtype=np.float32))


@pytest.mark.parametrize("fa,fb", PAIRS)
def test_one_hot_rows_select_entries_of_b(oracle, fa, fb):
    """A has a single 1.0 per row: C[i, j] must be exactly the decoded B[j, k_i] -- a transposed
    operand, a wrong stride or a k/n mix-up cannot survive this."""
    one = {0: 0x38, 1: 0x3C}
    rng = np.random.default_rng(3)
    M, K, N = 40, 96, 50
    ks = rng.integers(0, K, M)
    A = np.zeros((M, K), dtype=np.uint8)
    A[np.arange(M), ks] = one[fa]
    codes = finite_codes(fb)
    B = codes[rng.integers(0, codes.size, (N, K))]
    table = np.arange(256, dtype=np.uint8)
    if fb == 0:   # value table from the OCP definition, independent of the oracle's decoder
        E, Mn = (table >> 3) & 0xF, table & 7
        mag = np.where(E == 0, Mn / 8.0 * 2.0 ** -6, (1 + Mn / 8.0) * 2.0 ** (E.astype(np.float64) - 7))
    else:
        E, Mn = (table >> 2) & 0x1F, table & 3
        mag = np.where(E == 0, Mn / 4.0 * 2.0 ** -14, (1 + Mn / 4.0) * 2.0 ** (E.astype(np.float64) - 15))
    val = np.where(table & 0x80, -mag, mag)
    want = val[B][:, ks].T.astype(np.float32)
    for C in (oracle.gemm(A, fa, B, fb), oracle.gemm_verbatim(A, fa, B, fb)):
        assert np.array_equal(C, want)


def test_small_integers_equal_integer_matmul(oracle):
    rng = np.random.default_rng(4)
    vals = np.arange(-8, 9, dtype=np.float32)
    M, K, N = 31, 1000, 29
    a = vals[rng.integers(0, vals.size, (M, K))]
    b = vals[rng.integers(0, vals.size, (N, K))]
    A, B = oracle.encode(a, 0), oracle.encode(b, 1)
    want = a.astype(np.int64) @ b.astype(np.int64).T            # |sum| <= 64000 < 2^24: exact in fp32
    assert np.array_equal(oracle.gemm(A, 0, B, 1).astype(np.int64), want)
    assert np.array_equal(oracle.gemm_verbatim(A, 0, B, 1).astype(np.int64), want)


def test_matches_sequential_fp32_accumulation_done_in_numpy(oracle):
    """Brute force on a tiny case: products formed in float64 (exact), summed k-ascending with
    an explicit float32 rounding after each addition."""
    rng = np.random.default_rng(6)
    M, K, N = 6, 300, 5
    A = random_codes(rng, (M, K), 0)
    B = tame(random_codes(rng, (N, K), 1), 1)
    a = oracle.decode(A, 0).astype(np.float64)
    b = oracle.decode(B, 1).astype(np.float64)
    want = np.zeros((M, N), dtype=np.float32)
    for k in range(K):
        want = (want.astype(np.float64) + np.outer(a[:, k], b[:, k])).astype(np.float32)
    assert np.array_equal(oracle.gemm(A, 0, B, 1).view(np.uint32), want.view(np.uint32))


def test_tolerance_scale_is_sum_of_absolute_products(oracle):
    rng = np.random.default_rng(8)
    M, K, N = 17, 513, 23
    A = random_codes(rng, (M, K), 0)
    B = random_codes(rng, (N, K), 0)
    _, S = oracle.gemm(A, 0, B, 0, with_scale=True)
    want = np.abs(oracle.decode(A, 0).astype(np.float64)) @ np.abs(oracle.decode(B, 0).astype(np.float64)).T
    assert np.allclose(S, want, rtol=1e-6, atol=0)
    assert np.array_equal(oracle.tolerance(K, S), 2.0 * K * 2.0 ** -24 * S)


def test_config1_shape_runs_on_cpu(oracle, pkg):
    """The reference's own CPU-runnable case: M=N=K=1024, N(0,1) inputs rounded to e4m3."""
    M = N = K = 1024
    A = pkg.fill((M, K), 0, seed=0xA11CE + 1, dist="normal")
    B = pkg.fill((N, K), 0, seed=0xB0B + 1, dist="normal")
    C = oracle.gemm(A, 0, B, 0)
    rows = np.array([0, 511, 1023], dtype=np.int32)
    assert np.array_equal(oracle.gemm_verbatim(A[rows], 0, B, 0).view(np.uint32), C[rows].view(np.uint32))
    d = oracle.decode(A[rows], 0).astype(np.float64) @ oracle.decode(B, 0).astype(np.float64).T
    assert np.abs(C[rows] - d).max() <= 1024 * 2.0 ** -24 * np.abs(d).max() * 64
