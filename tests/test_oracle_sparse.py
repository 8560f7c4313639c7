"""The oracle's sparse-times-dense loop (oracle_spmm_csr), pinned without the reference.

The reference announces SpMM and SpMV (README.md:7) and holds only host helpers for their
operand formats (GEMM/include/bm_test_utils.h:48-128): no kernel, no CPU loop, no vector.
So parity is unpinned by the reference; the loop is pinned by what the arithmetic fixes:
equality with the dense loop on the densified operand, an independent sparse library on exact
small integers, one-hot selections, a numpy replay of the running fp32 sum.
"""
import numpy as np
import pytest
import scipy.sparse as sp

from conftest import finite_codes, random_codes
from sparse_util import random_bell, random_csr


@pytest.mark.parametrize("sfmt,bfmt", [(0, 0), (1, 1), (0, 1), (1, 0)])
@pytest.mark.parametrize("m,k,n,density", [(37, 100, 29, 0.1), (64, 256, 16, 0.5), (5, 33, 1, 0.3), (128, 64, 40, 0.02)])
def test_equals_the_dense_loop_on_the_densified_operand(oracle, sfmt, bfmt, m, k, n, density):
    """Distinct columns per row, any finite codes: leaving the zeros out changes no bit of
    the dense loop's result (the dense loop is pinned by tests/test_oracle_gemm.py)."""
    rng = np.random.default_rng(m * 1000 + k + 7 * sfmt + bfmt)
    vals, offs, col = random_csr(rng, m, k, density, sfmt, all_codes=True)
    B = random_codes(rng, (n, k), bfmt)
    if bfmt == 1:
        B = np.where(((B >> 2) & 0x1F) > 24, B & 0x83 | 0x3C, B).astype(np.uint8)     # keep the sums finite
    dense = np.zeros((m, k), dtype=np.uint8)
    for i in range(m):
        dense[i, col[offs[i]:offs[i + 1]]] = vals[offs[i]:offs[i + 1]]
    got = oracle.spmm_csr(vals, sfmt, offs, col, k, B, bfmt)
    want = oracle.gemm_verbatim(dense, sfmt, B, bfmt)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    if n == 1:
        assert np.array_equal(oracle.spmm_csr(vals, sfmt, offs, col, k, B[0], bfmt), got[:, 0])


def test_small_integers_against_an_independent_sparse_library(oracle):
    """|values| <= 8, duplicates and zero-valued padding entries included: every partial sum is
    an integer far below 2^24, so the loop must equal scipy's CSR product (which adds
    duplicates) computed in float64."""
    rng = np.random.default_rng(5)
    m, k, n = 60, 90, 33
    ints = np.arange(-8, 9, dtype=np.float32)
    offs = np.zeros(m + 1, dtype=np.int32)
    cols, vals = [], []
    for i in range(m):
        cnt = int(rng.integers(0, 25))
        c = np.sort(rng.integers(0, k, cnt))                 # sorted, duplicates likely
        cols.append(c)
        vals.append(ints[rng.integers(0, ints.size, cnt)])
        offs[i + 1] = offs[i] + cnt
    col = np.concatenate(cols).astype(np.int32)
    val_f = np.concatenate(vals).astype(np.float32)
    Bf = ints[rng.integers(0, ints.size, (n, k))]
    got = oracle.spmm_csr(oracle.encode(val_f, 0), 0, offs, col, k, oracle.encode(Bf, 1), 1)
    S = sp.csr_matrix((val_f.astype(np.float64), col, offs), shape=(m, k))
    want = S @ Bf.T.astype(np.float64)
    assert np.array_equal(got.astype(np.float64), np.asarray(want))


@pytest.mark.parametrize("sfmt,bfmt", [(0, 1), (1, 0)])
def test_one_hot_rows_select_single_entries(oracle, sfmt, bfmt):
    """One stored entry of value 1.0 per row: out[i][j] == decode(B[j][col_i]) for every finite code."""
    one = {0: 0x38, 1: 0x3C}
    k, n = 300, 256
    codes = finite_codes(bfmt)
    rng = np.random.default_rng(9)
    B = codes[rng.integers(0, codes.size, (n, k))]
    B[:, 17] = np.resize(codes, n)
    col = rng.integers(0, k, 50).astype(np.int32)
    col[0] = 17
    offs = np.arange(51, dtype=np.int32)
    vals = np.full(50, one[sfmt], dtype=np.uint8)
    got = oracle.spmm_csr(vals, sfmt, offs, col, k, B, bfmt)
    assert np.array_equal(got, oracle.decode(B, bfmt)[:, col].T)


def test_running_fp32_sum_in_storage_order(oracle):
    """Values whose sum depends on the order (2^16, small terms, -2^16): the result is the
    running fp32 sum in storage order, replayed here with numpy float32 scalars."""
    k, n = 64, 3
    rng = np.random.default_rng(11)
    val_f = np.array([2.0 ** 15, 2.0 ** -9, 2.0 ** -9, 2.0 ** -10, -(2.0 ** 15), 2.0 ** -6, 1.5], dtype=np.float32)
    col = np.array([3, 5, 9, 20, 33, 40, 63], dtype=np.int32)
    offs = np.array([0, 7], dtype=np.int32)
    Bf = np.ones((n, k), dtype=np.float32)
    Bf[1] = 2.0 ** 8
    Bf[2, :] = rng.choice([1.0, -1.0, 0.5], size=k)
    vals = oracle.encode(val_f, 1)
    assert np.array_equal(oracle.decode(vals, 1), val_f)         # all representable in e5m2
    got = oracle.spmm_csr(vals, 1, offs, col, k, oracle.encode(Bf, 1), 1)[0]
    for j in range(n):
        acc = np.float32(0.0)
        for v, c in zip(val_f, col):
            acc = np.float32(acc + np.float32(v * Bf[j, c]))
        assert got[j] == acc
    # 2^15 swallows 2^-9 (half an ulp, ties to even), 2^-9 and 2^-10: what is left is not the exact sum
    assert got[0] == np.float32(1.5 + 2.0 ** -6) and float(val_f.astype(np.float64).sum()) != float(got[0])


@pytest.mark.parametrize("block,ell", [(16, 3), (32, 2), (64, 1)])
def test_blocked_ell_as_csr_equals_the_dense_loop(oracle, block, ell):
    """bell_to_csr keeps every stored element of every block (padding blocks dropped), so the
    sparse loop on it equals the dense loop on the matrix the blocks spell out."""
    rng = np.random.default_rng(block)
    m, k, n = 4 * block, 6 * block, 24
    vals, bcols = random_bell(rng, m, k, block, ell, 0, pad_some=True)
    B = random_codes(rng, (n, k), 0)
    dense = np.zeros((m, k), dtype=np.uint8)
    for br in range(m // block):
        for j in range(ell):
            c = bcols[br, j]
            if c >= 0:
                dense[br * block:(br + 1) * block, c * block:(c + 1) * block] = vals[br * block:(br + 1) * block, j * block:(j + 1) * block]
    v, offs, col = oracle.bell_to_csr(vals, bcols, block)
    got = oracle.spmm_csr(v, 0, offs, col, k, B, 0)
    assert np.array_equal(got.view(np.uint32), oracle.gemm_verbatim(dense, 0, B, 0).view(np.uint32))


@pytest.mark.parametrize("lfmt,rfmt", [(0, 0), (1, 1), (0, 1), (1, 0)])
@pytest.mark.parametrize("m_vec,vec,k,n", [(9, 4, 100, 37), (5, 8, 256, 64), (3, 1, 33, 10), (4, 16, 64, 20)])
def test_sddmm_is_the_dense_product_sampled(oracle, lfmt, rfmt, m_vec, vec, k, n):
    """Every output of the sampled product is one element of lhs * rhs^T: bit-equal to the dense
    loop (pinned by tests/test_oracle_gemm.py) gathered at the stored positions, every finite code."""
    rng = np.random.default_rng(m_vec * 100 + vec + 7 * lfmt + rfmt)
    lhs = random_codes(rng, (m_vec * vec, k), lfmt)
    rhs = random_codes(rng, (n, k), rfmt)
    for a, f in ((lhs, lfmt), (rhs, rfmt)):
        if f == 1:
            a[...] = np.where(((a >> 2) & 0x1F) > 24, a & 0x83 | 0x3C, a)
    counts = rng.integers(0, n, m_vec)
    offs = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    col = np.concatenate([np.sort(rng.permutation(n)[:c]) for c in counts]).astype(np.int32)
    got = oracle.sddmm(offs, col, vec, lhs, lfmt, rhs, rfmt)
    dense = oracle.gemm_verbatim(lhs, lfmt, rhs, rfmt)                  # (m_vec*vec, n)
    for i in range(m_vec):
        for j in range(offs[i], offs[i + 1]):
            want = dense[i * vec:(i + 1) * vec, col[j]]
            assert np.array_equal(got[j].view(np.uint32), want.view(np.uint32))
