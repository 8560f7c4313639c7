"""Seeded sparse operands for the tests, in the two formats the reference's host helpers
produce (GEMM/include/bm_test_utils.h:48-68 blocked-ELL column lists, :71-128 CSR with optional
row padding)."""
import numpy as np

from conftest import random_codes


def random_csr(rng, m, k, density, fmt, all_codes=False, row_padding=0, sigma=1.0, encode=None):
    """Uniformly random sparsity mask with distinct, ascending columns per row.  Values: every
    finite code (all_codes) or N(0, sigma) through `encode`.  row_padding > 0 pads each row to
    a multiple of it with zero-valued entries that repeat the row's last column, as the
    reference's generator does."""
    mask = rng.random((m, k)) < density
    offs = [0]
    cols, vals = [], []
    for i in range(m):
        c = np.flatnonzero(mask[i]).astype(np.int32)
        if all_codes:
            v = random_codes(rng, (c.size,), fmt)
            if fmt == 1:
                v = np.where(((v >> 2) & 0x1F) > 24, v & 0x83 | 0x3C, v).astype(np.uint8)
        else:
            v = encode(rng.normal(0.0, sigma, c.size).astype(np.float32), fmt)
        if row_padding > 0 and c.size > 0:
            add = (-c.size) % row_padding
            c = np.concatenate([c, np.full(add, c[-1], dtype=np.int32)])
            v = np.concatenate([v, np.zeros(add, dtype=np.uint8)])
        cols.append(c)
        vals.append(v)
        offs.append(offs[-1] + c.size)
    return (np.concatenate(vals).astype(np.uint8), np.asarray(offs, dtype=np.int32),
            np.concatenate(cols).astype(np.int32))


def random_bell(rng, m, k, block, ell_cols, fmt, pad_some=False, encode=None, sigma=1.0):
    """Blocked-ELL: every block row stores ell_cols blocks at distinct, ascending block columns
    drawn uniformly (what GenerateUniformBlockedELLIndex produces); with pad_some the last
    stored block of some block rows is padding (-1).  Values: every finite code, or N(0, sigma)."""
    nbr, nbc = m // block, k // block
    assert m % block == 0 and k % block == 0 and ell_cols <= nbc
    bcols = np.stack([np.sort(rng.permutation(nbc)[:ell_cols]) for _ in range(nbr)]).astype(np.int32)
    if pad_some:
        bcols[rng.random(nbr) < 0.4, -1] = -1
    if encode is None:
        vals = random_codes(rng, (m, ell_cols * block), fmt)
        if fmt == 1:
            vals = np.where(((vals >> 2) & 0x1F) > 24, vals & 0x83 | 0x3C, vals).astype(np.uint8)
    else:
        vals = encode(rng.normal(0.0, sigma, (m, ell_cols * block)).astype(np.float32), fmt)
    return vals, bcols
