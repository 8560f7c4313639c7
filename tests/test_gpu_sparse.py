"""GPU parity of the sparse-times-dense entry points (blocked-ELL and CSR, SpMM and SpMV),
called through the C ABI, against the CPU oracle's sparse loop (oracle_spmm_csr, which
tests/test_oracle_sparse.py pins without the reference: the reference holds no SpMM / SpMV
kernel, loop or vector, only the generators of the operand formats,
GEMM/include/bm_test_utils.h:48-128).

Bar: |out_gpu - out_ref| <= 2 * L * 2^-24 * sum |a*b| per element, L = stored entries of the
row (reordered fp32 accumulation only; products are exact), plus the MFMA's alignment-window
term where the sums are short; bit-exact where no rounding can occur.
"""
import zlib

import numpy as np
import pytest

from conftest import finite_codes, random_codes
from sparse_util import random_bell, random_csr

pytestmark = pytest.mark.gpu

PAIRS = [(0, 0), (1, 1), (0, 1), (1, 0)]


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def bound(oracle, vals, sfmt, offs, col, k, B, bfmt, mfma=False):
    """Reference, and the tolerance per element."""
    ref, S = oracle.spmm_csr(vals, sfmt, offs, col, k, B, bfmt, with_scale=True)
    L = np.diff(offs).astype(np.float64)
    L = L if S.ndim == 1 else L[:, None]
    tol = 2.0 * np.maximum(L, 1.0) * 2.0 ** -24 * S
    if mfma:
        # the f8f6f4 MFMA adds groups of 8 products with 13 bits below the group's largest
        # (tests/test_gpu_mfma_numerics.py); bounded here by 2^-10 of the largest product times the group count
        amax = np.abs(oracle.decode(vals, sfmt)).max() if vals.size else 0.0
        bmax = np.abs(oracle.decode(B, bfmt)).max()
        tol = tol + 2.0 ** -10 * amax * bmax * np.maximum(L, 1.0) / 8.0
    return ref, tol


def check(out, ref, tol):
    assert np.isfinite(out).all()
    err = np.abs(out.astype(np.float64) - ref.astype(np.float64))
    assert (err <= tol).all(), "worst err/tol = %g" % float((err / np.maximum(tol, 1e-300)).max())


@pytest.mark.parametrize("fs,fb", PAIRS)
@pytest.mark.parametrize("block,ell,m,k,n", [(16, 3, 64, 160, 40), (32, 5, 128, 512, 100), (64, 2, 256, 1024, 64),
                                              (128, 3, 256, 2048, 33), (48, 2, 96, 480, 17), (16, 9, 32, 144, 16)])
def test_spmm_bell_all_finite_codes(pkg, oracle, fs, fb, block, ell, m, k, n):
    """Every finite code as a value, padding blocks included, block sizes that are and are not
    powers of two, stored rows that are not whole 128-byte K steps, n that overhangs the wave's
    column group."""
    rng = np.random.default_rng(zlib.crc32(repr((fs, fb, block, ell, m, k, n)).encode()))
    vals, bcols = random_bell(rng, m, k, block, ell, fs, pad_some=True)
    B = random_codes(rng, (n, k), fb)
    if fb == 1:
        B = np.where(((B >> 2) & 0x1F) > 24, B & 0x83 | 0x3C, B).astype(np.uint8)
    out = pkg.spmm_bell(dev(vals), dev(bcols), block, dev(B), k, s_fmt=fs, b_fmt=fb).cpu().numpy()
    v, offs, col = oracle.bell_to_csr(vals, bcols, block)
    ref, tol = bound(oracle, v, fs, offs, col, k, B, fb, mfma=True)
    check(out, ref, tol)


@pytest.mark.parametrize("fs,fb", PAIRS)
@pytest.mark.parametrize("block,ell,m,k,n", [(128, 4, 512, 4096, 300), (256, 2, 512, 2048, 256), (128, 40, 256, 8192, 512),
                                              (256, 16, 1024, 8192, 1024), (128, 1, 128, 128, 64), (384, 2, 768, 1536, 200),
                                              (128, 3, 2304, 2048, 2200)])
def test_spmm_bell_through_the_tiled_kernel(pkg, oracle, fs, fb, block, ell, m, k, n):
    """Blocks of whole 128-byte K tiles and whole tile rows run on the LDS-tiled persistent kernel:
    128- and 256-row tiles, both MFMA shapes, K slices (few tiles, long stored rows), more tiles
    than CUs with leftover tiles, a single K tile, padding blocks, n that overhangs the tile."""
    rng = np.random.default_rng(zlib.crc32(repr(("tiled", fs, fb, block, ell, m, k, n)).encode()))
    vals, bcols = random_bell(rng, m, k, block, ell, fs, pad_some=ell > 1)
    B = random_codes(rng, (n, k), fb)
    if fb == 1:
        B = np.where(((B >> 2) & 0x1F) > 24, B & 0x83 | 0x3C, B).astype(np.uint8)
    out = pkg.spmm_bell(dev(vals), dev(bcols), block, dev(B), k, s_fmt=fs, b_fmt=fb).cpu().numpy()
    v, offs, col = oracle.bell_to_csr(vals, bcols, block)
    ref, tol = bound(oracle, v, fs, offs, col, k, B, fb, mfma=True)
    check(out, ref, tol)


@pytest.mark.parametrize("fs,fb", PAIRS)
@pytest.mark.parametrize("block,ell,m,k,n", [(64, 40, 128, 4096, 300), (96, 3, 192, 960, 128), (192, 2, 384, 1536, 256),
                                              (32, 9, 2048, 1024, 2048), (32, 1, 32, 32, 64), (64, 3, 4096, 512, 1100),
                                              (160, 5, 320, 1600, 70)])
def test_spmm_bell_small_blocks_through_the_tiled_kernel(pkg, oracle, fs, fb, block, ell, m, k, n):
    """Blocks of 32 rows and multiples that are not multiples of 128 run on the tiled kernel with
    tiles as tall as a block (64 or 32 rows): a K tile then spans several stored blocks (or parts
    of blocks: 96, 160, 192), stored rows need not be whole K tiles, few tiles are cut into K
    slices, many run in rounds with leftover tiles; padding blocks everywhere."""
    rng = np.random.default_rng(zlib.crc32(repr(("small", fs, fb, block, ell, m, k, n)).encode()))
    vals, bcols = random_bell(rng, m, k, block, ell, fs, pad_some=ell > 1)
    B = random_codes(rng, (n, k), fb)
    if fb == 1:
        B = np.where(((B >> 2) & 0x1F) > 24, B & 0x83 | 0x3C, B).astype(np.uint8)
    out = pkg.spmm_bell(dev(vals), dev(bcols), block, dev(B), k, s_fmt=fs, b_fmt=fb).cpu().numpy()
    v, offs, col = oracle.bell_to_csr(vals, bcols, block)
    ref, tol = bound(oracle, v, fs, offs, col, k, B, fb, mfma=True)
    check(out, ref, tol)


@pytest.mark.parametrize("fs,fb", PAIRS)
@pytest.mark.parametrize("block", [32, 64, 128, 256])
def test_spmm_bell_tiled_one_hot_is_bit_exact(pkg, oracle, fs, fb, block):
    """The tiled kernel's gather through the block list, bit for bit: one value of 1.0 per row of S."""
    one = {0: 0x38, 1: 0x3C}
    ell, m, k, n = 3, 2 * block, 8 * block, 256
    rng = np.random.default_rng(177 + fs + block)
    _, bcols = random_bell(rng, m, k, block, ell, fs)
    vals = np.zeros((m, ell * block), dtype=np.uint8)
    pos = rng.integers(0, ell * block, m)
    vals[np.arange(m), pos] = one[fs]
    col = bcols[np.arange(m) // block, pos // block] * block + pos % block
    codes = finite_codes(fb)
    B = codes[rng.integers(0, codes.size, (n, k))]
    B[:, col[0]] = np.resize(codes, n)
    out = pkg.spmm_bell(dev(vals), dev(bcols), block, dev(B), k, s_fmt=fs, b_fmt=fb).cpu().numpy()
    assert np.array_equal(out, oracle.decode(B, fb)[:, col].T)


@pytest.mark.parametrize("fs,fb", PAIRS)
def test_spmm_bell_normal_values_plain_bound(pkg, oracle, fs, fb):
    """N(0,1)-like values, long stored rows: the plain reordering bound, no hardware term."""
    rng = np.random.default_rng(31 + fs * 2 + fb)
    m, k, n, block, ell = 512, 8192, 256, 64, 32
    vals, bcols = random_bell(rng, m, k, block, ell, fs, encode=oracle.encode, sigma=2.0)
    B = pkg.fill((n, k), fb, seed=0xB0B + 70 + fs, dist="normal", sigma=2.0)
    out = pkg.spmm_bell(dev(vals), dev(bcols), block, dev(B), k, s_fmt=fs, b_fmt=fb).cpu().numpy()
    v, offs, col = oracle.bell_to_csr(vals, bcols, block)
    ref, tol = bound(oracle, v, fs, offs, col, k, B, fb)
    check(out, ref, tol)


@pytest.mark.parametrize("fs,fb", PAIRS)
def test_spmm_bell_one_hot_is_bit_exact(pkg, oracle, fs, fb):
    """One value of 1.0 per row of S: out[i][j] == decode(b[j][that column]) for every finite
    code of b's format (decode through the MFMA, positions gathered through the block list)."""
    one = {0: 0x38, 1: 0x3C}
    block, ell, m, k, n = 16, 4, 64, 256, 256
    rng = np.random.default_rng(77 + fs)
    _, bcols = random_bell(rng, m, k, block, ell, fs)
    vals = np.zeros((m, ell * block), dtype=np.uint8)
    pos = rng.integers(0, ell * block, m)
    vals[np.arange(m), pos] = one[fs]
    col = bcols[np.arange(m) // block, pos // block] * block + pos % block
    codes = finite_codes(fb)
    B = codes[rng.integers(0, codes.size, (n, k))]
    B[:, col[0]] = np.resize(codes, n)
    out = pkg.spmm_bell(dev(vals), dev(bcols), block, dev(B), k, s_fmt=fs, b_fmt=fb).cpu().numpy()
    assert np.array_equal(out, oracle.decode(B, fb)[:, col].T)


@pytest.mark.parametrize("fs,fx", PAIRS)
@pytest.mark.parametrize("block,ell,m,k", [(16, 8, 1024, 2048), (128, 4, 512, 4096), (32, 1, 64, 64),
                                           (64, 112, 256, 8192),        # stored rows of 7 slots of 1 KiB (an odd count), two waves to a row
                                           (64, 256, 64, 16384),        # few long rows: four waves to a row
                                           (64, 24, 2048, 4096),        # a slot and a half per row, several rows per wave
                                           (48, 5, 960, 960),           # blocks that are no power of two, 16 lanes to a row
                                           (16, 3, 4096, 1024),         # rows shorter than the four lanes they get
                                           (256, 8, 16384, 4096)])      # more row items than resident waves
def test_spmv_bell(pkg, oracle, fs, fx, block, ell, m, k):
    """Row lengths on every side of the kernel's slot of 1024 bytes, row counts that choose each of its
    ways of sharing the work, padding blocks."""
    rng = np.random.default_rng(zlib.crc32(repr((fs, fx, block, ell, m, k)).encode()))
    vals, bcols = random_bell(rng, m, k, block, ell, fs, pad_some=True, encode=oracle.encode, sigma=2.0)
    x = pkg.fill((k,), fx, seed=0xA11CE + 80 + block, dist="normal", sigma=2.0)
    y = pkg.spmm_bell(dev(vals), dev(bcols), block, dev(x), k, s_fmt=fs, b_fmt=fx).cpu().numpy()
    v, offs, col = oracle.bell_to_csr(vals, bcols, block)
    ref, tol = bound(oracle, v, fs, offs, col, k, x, fx, mfma=True)
    check(y, ref, tol)


@pytest.mark.parametrize("fs,fx", PAIRS)
@pytest.mark.parametrize("m,k,density,pad", [(1000, 4096, 0.1, 0), (257, 1000, 0.3, 4), (64, 70000, 0.01, 0), (5, 7, 0.5, 0)])
def test_spmv_csr(pkg, oracle, fs, fx, m, k, density, pad):
    """Rows of very different lengths (empty ones included), row padding as the reference's
    generator appends it, every finite code; natural row order and longest-rows-first."""
    rng = np.random.default_rng(zlib.crc32(repr((fs, fx, m, k, density, pad)).encode()))
    vals, offs, col = random_csr(rng, m, k, density, fs, all_codes=True, row_padding=pad)
    x = random_codes(rng, (k,), fx)
    if fx == 1:
        x = np.where(((x >> 2) & 0x1F) > 24, x & 0x83 | 0x3C, x).astype(np.uint8)
    ref, tol = bound(oracle, vals, fs, offs, col, k, x, fx)
    dv, do, dc, dx = dev(vals), dev(offs), dev(col), dev(x)
    y = pkg.spmm_csr(dv, do, dc, dx, k, s_fmt=fs, b_fmt=fx).cpu().numpy()
    check(y, ref, tol)
    order = pkg.sorted_row_swizzle(offs)
    lengths = np.diff(offs)[order]
    assert sorted(order.tolist()) == list(range(m)) and (np.diff(lengths) <= 0).all()
    y2 = pkg.spmm_csr(dv, do, dc, dx, k, s_fmt=fs, b_fmt=fx, row_order=dev(order)).cpu().numpy()
    assert np.array_equal(y2, y)          # the order of the rows changes no row's sum


@pytest.mark.parametrize("fs,fx", PAIRS)
def test_spmv_csr_decodes_every_code_bit_for_bit(pkg, oracle, fs, fx):
    """One stored entry per row: a value of 1.0 against every code of x's format, and every code of the
    value's format against an x of 1.0 -- the kernel's own decode (conversion instructions) must give
    the oracle's value bit for bit, subnormals, -0 and the infinities of e5m2 included; NaN codes give NaN."""
    one = {0: 0x38, 1: 0x3C}
    k = 256
    codes = np.arange(256, dtype=np.uint8)
    offs = np.arange(257, dtype=np.int32)
    col = np.arange(256, dtype=np.int32)
    for vals, x, decoded in [(np.full(256, one[fs], np.uint8), codes, oracle.decode(codes, fx)),
                             (codes, np.full(256, one[fx], np.uint8), oracle.decode(codes, fs))]:
        want = oracle.spmm_csr(vals, fs, offs, col, k, x, fx)          # = the decoded values (a sum that starts at +0 turns -0 into +0)
        assert np.array_equal(np.nan_to_num(want, nan=7.0), np.nan_to_num(decoded + np.float32(0.0), nan=7.0))
        for aligned in (True, False):                      # the 16-byte-load kernel and the element-wise one
            dcol = dev(np.concatenate([[0], col]).astype(np.int32))[1:] if not aligned else dev(col)
            y = pkg.spmm_csr(dev(vals), dev(offs), dcol, dev(x), k, s_fmt=fs, b_fmt=fx).cpu().numpy()
            nan = np.isnan(want)
            assert np.array_equal(np.isnan(y), nan)
            assert np.array_equal(y[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_spmv_csr_small_integers_with_duplicates_exact(pkg, oracle):
    """|values| <= 8: every sum is an exact integer; entries that repeat a column are added."""
    rng = np.random.default_rng(3)
    m, k = 300, 500
    ints = np.arange(-8, 9, dtype=np.float32)
    counts = rng.integers(0, 200, m)
    offs = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    col = np.concatenate([np.sort(rng.integers(0, k, c)) for c in counts]).astype(np.int32)
    val_f = ints[rng.integers(0, ints.size, offs[-1])]
    x_f = ints[rng.integers(0, ints.size, k)]
    y = pkg.spmm_csr(dev(oracle.encode(val_f, 0)), dev(offs), dev(col), dev(oracle.encode(x_f, 1)), k, s_fmt=0, b_fmt=1).cpu().numpy()
    want = np.array([np.dot(val_f[offs[i]:offs[i + 1]].astype(np.float64), x_f[col[offs[i]:offs[i + 1]]]) for i in range(m)])
    assert np.array_equal(y.astype(np.float64), want)


@pytest.mark.parametrize("fs,fb", PAIRS)
@pytest.mark.parametrize("m,k,n,density,pad", [(256, 1024, 256, 0.1, 0), (300, 2048, 200, 0.05, 8), (64, 8192, 2048, 0.02, 0),
                                                (100, 100, 50, 0.3, 0)])
def test_spmm_csr(pkg, oracle, fs, fb, m, k, n, density, pad):
    """Through the dense scratch and the dense GEMM (tiled kernels with and without K slices,
    the general kernel for k % 16 != 0); zero-valued padding entries repeat a column and must
    not wipe the real entry there."""
    rng = np.random.default_rng(zlib.crc32(repr((fs, fb, m, k, n, density, pad)).encode()))
    vals, offs, col = random_csr(rng, m, k, density, fs, row_padding=pad, encode=oracle.encode, sigma=2.0)
    B = pkg.fill((n, k), fb, seed=0xB0B + 90 + m, dist="normal", sigma=2.0)
    out = pkg.spmm_csr(dev(vals), dev(offs), dev(col), dev(B), k, s_fmt=fs, b_fmt=fb).cpu().numpy()
    ref, S = oracle.spmm_csr(vals, fs, offs, col, k, B, fb, with_scale=True)
    # the dense GEMM adds over all k positions (zeros included): its bound is the dense one
    tol = oracle.tolerance(k, S) + (2.0 ** -10 * 16.0 * 16.0 if k < 1024 else 0.0)
    check(out, ref, tol)
    assert pkg.lib().fp8gemm_spmm_csr_scratch_bytes(m, k, n) >= m * k


@pytest.mark.parametrize("fl,fr", PAIRS)
@pytest.mark.parametrize("m_vec,vec,k,n,per_row", [(64, 8, 1024, 512, 40), (33, 16, 256, 100, 70), (20, 4, 4096, 64, 17),
                                                    (7, 1, 144, 30, 5), (5, 16, 8192, 48, 20), (10, 3, 100, 40, 9), (4, 20, 64, 32, 6)])
def test_sddmm(pkg, oracle, fl, fr, m_vec, vec, k, n, per_row):
    """Sampled dense-dense product against the oracle's loop (the reference's Host_sddmm): rows with
    more and fewer than 16 stored entries and empty ones, vector lengths up to 16 on the MFMA,
    k that is not a whole K step, rows of lhs too long to be held in LDS, and shapes only the
    one-thread-per-output kernel takes (k % 16 != 0, vec > 16)."""
    rng = np.random.default_rng(zlib.crc32(repr((fl, fr, m_vec, vec, k, n, per_row)).encode()))
    lhs = pkg.fill((m_vec * vec, k), fl, seed=0xA11CE + 40 + m_vec, dist="normal", sigma=2.0)
    rhs = pkg.fill((n, k), fr, seed=0xB0B + 40 + n, dist="normal", sigma=2.0)
    counts = rng.integers(0, min(n, 2 * per_row) + 1, m_vec)
    counts[0] = 0
    offs = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    col = np.concatenate([np.sort(rng.permutation(n)[:c]) for c in counts]).astype(np.int32)
    out = pkg.sddmm(dev(offs), dev(col), vec, dev(lhs), dev(rhs), l_fmt=fl, r_fmt=fr).cpu().numpy()
    ref, S = oracle.sddmm(offs, col, vec, lhs, fl, rhs, fr, with_scale=True)
    tol = oracle.tolerance(k, S) + (2.0 ** -10 * S if k < 1024 else 0.0)
    check(out, ref, tol)


def test_sddmm_at_benchmark_size_is_the_dense_product_sampled(pkg):
    """The benchmark's shape (8192 x 8192 outputs in vectors of 8, one in ten stored, K = 512), too large
    for the CPU loop: every stored output is an element of lhs * rhs^T, which the library's dense GEMM
    (held to the oracle by its own tests) computes in another order; the bound's sum of magnitudes comes
    from the same GEMM on the operands with their sign bits cleared."""
    import torch
    m_vec, vec, n, k = 1024, 8, 8192, 512
    rng = np.random.default_rng(77)
    mask = rng.random((m_vec, n)) < 0.10
    offs = np.concatenate([[0], np.cumsum(mask.sum(axis=1))]).astype(np.int32)
    rows, col = np.nonzero(mask)
    lhs = dev(pkg.fill((m_vec * vec, k), 0, seed=0xA11CE + 77, dist="normal"))
    rhs = dev(pkg.fill((n, k), 0, seed=0xB0B + 77, dist="normal"))
    out = pkg.sddmm(dev(offs), dev(col.astype(np.int32)), vec, lhs, rhs, l_fmt=0, r_fmt=0)
    dense = pkg.gemm(lhs, rhs, a_fmt=0, b_fmt=0)
    mags = pkg.gemm(lhs & 0x7F, rhs & 0x7F, a_fmt=0, b_fmt=0)
    torch.cuda.synchronize()
    r = torch.from_numpy(rows).to("cuda")[:, None] * vec + torch.arange(vec, device="cuda")[None, :]
    c = torch.from_numpy(col).to("cuda")[:, None].expand(-1, vec)
    want, S = dense[r, c], mags[r, c]
    assert out.shape == want.shape
    # both sides are reordered fp32 sums of the same exact products (each within the bound of the running sum)
    tol = 2.0 * (2.0 * k * 2.0 ** -24 + 2.0 ** -10) * S
    assert bool((torch.abs(out - want) <= tol).all())
    assert float(torch.abs(out).max()) > 0.0


def test_sddmm_small_integers_exact(pkg, oracle):
    rng = np.random.default_rng(12)
    m_vec, vec, k, n = 16, 8, 512, 128
    ints = np.arange(-8, 9, dtype=np.float32)
    lf, rf = ints[rng.integers(0, 17, (m_vec * vec, k))], ints[rng.integers(0, 17, (n, k))]
    counts = rng.integers(1, 60, m_vec)
    offs = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    col = np.concatenate([np.sort(rng.permutation(n)[:c]) for c in counts]).astype(np.int32)
    out = pkg.sddmm(dev(offs), dev(col), vec, dev(oracle.encode(lf, 0)), dev(oracle.encode(rf, 1)), l_fmt=0, r_fmt=1).cpu().numpy()
    dense = lf.astype(np.float64) @ rf.astype(np.float64).T
    for i in range(m_vec):
        for j in range(offs[i], offs[i + 1]):
            assert np.array_equal(out[j].astype(np.float64), dense[i * vec:(i + 1) * vec, col[j]])


def _bell_on_device(pkg, m, k, block, ell, seed):
    """A blocked-ELL operand of normal values, and the dense matrix its blocks spell out, both on the device."""
    import torch
    rng = np.random.default_rng(seed)
    nbr, nbc = m // block, k // block
    bcols = np.stack([np.sort(rng.permutation(nbc)[:ell]) for _ in range(nbr)]).astype(np.int32)
    vals = dev(pkg.fill((m, ell * block), 0, seed=0xA11CE + seed, dist="normal"))
    dense = torch.zeros((nbr, block, nbc, block), dtype=torch.uint8, device="cuda")
    rows = torch.arange(nbr, device="cuda")[:, None].expand(-1, ell)
    dense[rows, :, dev(bcols).long(), :] = vals.view(nbr, block, ell, block).permute(0, 2, 1, 3)
    return vals, bcols, dense.view(m, k)


def _within_reordering(out, want, mags, terms):
    """Two fp32 sums of the same exact products in different orders, `mags` the sum of their magnitudes."""
    import torch
    tol = 2.0 * (2.0 * terms * 2.0 ** -24 + 2.0 ** -10) * mags
    assert bool(torch.isfinite(out).all()) and bool((torch.abs(out - want) <= tol).all())
    assert float(torch.abs(out).max()) > 0.0


@pytest.mark.parametrize("m,k,n,block,ell", [(8192, 8192, 8192, 256, 8), (8192, 8192, 8192, 128, 16), (4096, 4096, 4096, 32, 32)])
def test_spmm_bell_at_benchmark_size_is_the_dense_gemm_on_the_blocks_spelled_out(pkg, m, k, n, block, ell):
    """The benchmark's blocked-ELL shapes, too large for the CPU loop: zeros add nothing, so the product
    equals the library's dense GEMM (held to the oracle by its own tests) on the dense matrix the stored
    blocks spell out, up to the order of the sum; the sum of magnitudes for the bound comes from the same
    GEMM on the operands with their sign bits cleared."""
    import torch
    vals, bcols, dense = _bell_on_device(pkg, m, k, block, ell, seed=block)
    B = dev(pkg.fill((n, k), 0, seed=0xB0B + block, dist="normal"))
    out = pkg.spmm_bell(vals, dev(bcols), block, B, k, s_fmt=0, b_fmt=0)
    want = pkg.gemm(dense, B, a_fmt=0, b_fmt=0)
    mags = pkg.gemm(dense & 0x7F, B & 0x7F, a_fmt=0, b_fmt=0)
    torch.cuda.synchronize()
    _within_reordering(out, want, mags, ell * block)


def test_spmv_at_benchmark_size_is_the_dense_matrix_vector_product(pkg):
    """The benchmark's two matrix-vector shapes (28672 x 8192: a quarter of the 64 x 64 blocks, and one
    element in ten in CSR) against the library's dense GEMV on the matrix the operand spells out."""
    import torch
    m, k = 28672, 8192
    x = dev(pkg.fill((k,), 0, seed=0x5BA, dist="normal"))
    L = pkg.lib()

    def gemv(w):
        y = torch.empty(m, dtype=torch.float32, device="cuda")
        pkg.check(L.fp8gemm_gemv(m, k, w.data_ptr(), 0, x.data_ptr(), 0, y.data_ptr(), None))
        return y
    vals, bcols, dense = _bell_on_device(pkg, m, k, 64, 32, seed=5)
    y = pkg.spmm_bell(vals, dev(bcols), 64, x, k, s_fmt=0, b_fmt=0)
    want = gemv(dense)
    magx = torch.empty_like(want)                          # sum of |a| * |x|: the same GEMV with the sign bits cleared
    xa = x & 0x7F
    pkg.check(L.fp8gemm_gemv(m, k, (dense & 0x7F).data_ptr(), 0, xa.data_ptr(), 0, magx.data_ptr(), None))
    torch.cuda.synchronize()
    _within_reordering(y, want, magx, 32 * 64)
    del vals, dense
    # CSR: one element in ten
    rng = np.random.default_rng(9)
    mask = torch.from_numpy(rng.random((m, k)) < 0.10).cuda()
    codes = dev(pkg.fill((m, k), 0, seed=0xA11CE + 9, dist="normal"))
    dense = torch.where(mask, codes, torch.zeros_like(codes))
    offs = torch.zeros(m + 1, dtype=torch.int32, device="cuda")
    offs[1:] = torch.cumsum(mask.sum(dim=1), 0).to(torch.int32)
    col = torch.nonzero(mask)[:, 1].to(torch.int32).contiguous()
    y = pkg.spmm_csr(codes[mask].contiguous(), offs, col, x, k, s_fmt=0, b_fmt=0)
    want = gemv(dense)
    pkg.check(L.fp8gemm_gemv(m, k, (dense & 0x7F).data_ptr(), 0, xa.data_ptr(), 0, magx.data_ptr(), None))
    torch.cuda.synchronize()
    _within_reordering(y, want, magx, 8192)


def test_sparse_launches_replay_in_a_hip_graph(pkg):
    """The matrix-vector products and the sampled product allocate nothing and clear nothing, and the blocked-ELL
    SpMM takes its scratch from the stream's pool, which a first eager call has sized: all four captured into
    one HIP graph and replayed on new operand values, with eager work between the replays, give the eager
    results bit for bit."""
    import torch
    rng = np.random.default_rng(4)
    m, k, n, block, ell = 2048, 4096, 512, 64, 8
    vals, bcols, _ = _bell_on_device(pkg, m, k, block, ell, seed=21)
    bc = dev(bcols)
    B = dev(pkg.fill((n, k), 0, seed=0xB0B + 21, dist="normal"))
    x = dev(pkg.fill((k,), 0, seed=0xB0B + 22, dist="normal"))
    mask = rng.random((m, k)) < 0.05
    offs = dev(np.concatenate([[0], np.cumsum(mask.sum(axis=1))]).astype(np.int32))
    col = dev(np.nonzero(mask)[1].astype(np.int32))
    cv = dev(pkg.fill((int(mask.sum()),), 0, seed=0xA11CE + 23, dist="normal"))
    vmask = rng.random((m // 8, n)) < 0.2
    voffs = dev(np.concatenate([[0], np.cumsum(vmask.sum(axis=1))]).astype(np.int32))
    vcol = dev(np.nonzero(vmask)[1].astype(np.int32))
    lhs = dev(pkg.fill((m, 256), 0, seed=0xA11CE + 24, dist="normal"))
    rhs = dev(pkg.fill((n, 256), 0, seed=0xB0B + 24, dist="normal"))
    outs = [torch.empty((m, n), dtype=torch.float32, device="cuda"), torch.empty(m, dtype=torch.float32, device="cuda"),
            torch.empty(m, dtype=torch.float32, device="cuda"), torch.empty((int(vmask.sum()), 8), dtype=torch.float32, device="cuda")]

    def launches(stream):
        pkg.spmm_bell(vals, bc, block, B, k, s_fmt=0, b_fmt=0, out=outs[0], stream=stream)
        pkg.spmm_bell(vals, bc, block, x, k, s_fmt=0, b_fmt=0, out=outs[1], stream=stream)
        pkg.spmm_csr(cv, offs, col, x, k, s_fmt=0, b_fmt=0, out=outs[2], stream=stream)
        pkg.sddmm(voffs, vcol, 8, lhs, rhs, l_fmt=0, r_fmt=0, out=outs[3], stream=stream)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launches(side)                                   # (sizes the stream's scratch pool before the capture)
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        launches(side)
    for rep in range(3):
        # new operand values in place, then eager work of the program's own, then the replay
        new = dev(pkg.fill((m, ell * block), 0, seed=0xA11CE + 30 + rep, dist="normal"))
        vals.copy_(new)
        x.copy_(dev(pkg.fill((k,), 0, seed=0xB0B + 30 + rep, dist="normal")))
        lhs.copy_(dev(pkg.fill((m, 256), 0, seed=0xA11CE + 40 + rep, dist="normal")))
        torch.cuda.synchronize()
        for o in outs:
            o.fill_(-1.0)
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        launches(None)
        torch.cuda.synchronize()
        for g, o in zip(got, outs):
            assert torch.equal(g, o)
    assert float(torch.abs(outs[0]).max()) > 0.0


def test_sparse_entry_points_refuse_bad_arguments(pkg):
    import torch
    L = pkg.lib()
    v = torch.zeros((64, 64), dtype=torch.uint8, device="cuda")
    c = torch.zeros((4, 4), dtype=torch.int32, device="cuda")
    b = torch.zeros((16, 64), dtype=torch.uint8, device="cuda")
    o = torch.zeros((64, 16), dtype=torch.float32, device="cuda")
    args = lambda block, m=64, k=64: (m, k, 16, block, 4, v.data_ptr(), 0, c.data_ptr(), b.data_ptr(), 0, o.data_ptr(), None)
    assert L.fp8gemm_spmm_bell(*args(16)) == 0
    assert L.fp8gemm_spmm_bell(*args(8)) == 1              # block not a multiple of 16
    assert L.fp8gemm_spmm_bell(*args(48)) == 1             # m, k not multiples of the block
    assert L.fp8gemm_spmm_bell(64, 64, 16, 16, 4, None, 0, c.data_ptr(), b.data_ptr(), 0, o.data_ptr(), None) == 1
    assert L.fp8gemm_spmm_bell(64, 64, 16, 16, 4, v.data_ptr(), 2, c.data_ptr(), b.data_ptr(), 0, o.data_ptr(), None) == 1
    assert L.fp8gemm_spmv_csr(0, 64, v.data_ptr(), 0, c.data_ptr(), c.data_ptr(), None, b.data_ptr(), 0, o.data_ptr(), None) == 1
    assert L.fp8gemm_spmm_csr(4, 64, 16, v.data_ptr(), 0, None, c.data_ptr(), b.data_ptr(), 0, o.data_ptr(), None) == 1
    # sampled product: a pattern with no stored entry at all is a launch that writes nothing
    offs = torch.zeros(5, dtype=torch.int32, device="cuda")
    o.fill_(7.0)
    assert L.fp8gemm_sddmm(4, 64, 16, offs.data_ptr(), c.data_ptr(), v.data_ptr(), 0, b.data_ptr(), 0, o.data_ptr(), None) == 0
    assert L.fp8gemm_sddmm(0, 64, 16, offs.data_ptr(), c.data_ptr(), v.data_ptr(), 0, b.data_ptr(), 0, o.data_ptr(), None) == 1
    assert L.fp8gemm_sddmm(4, 64, 0, offs.data_ptr(), c.data_ptr(), v.data_ptr(), 0, b.data_ptr(), 0, o.data_ptr(), None) == 1
    assert L.fp8gemm_sddmm(4, 64, 16, None, c.data_ptr(), v.data_ptr(), 0, b.data_ptr(), 0, o.data_ptr(), None) == 1
    assert L.fp8gemm_sddmm(4, 64, 16, offs.data_ptr(), c.data_ptr(), v.data_ptr(), 3, b.data_ptr(), 0, o.data_ptr(), None) == 1
    torch.cuda.synchronize()
    assert bool((o == 7.0).all())
