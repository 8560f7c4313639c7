"""ctypes front end of the CPU oracle (oracle/fp8_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke test and by the
cpu_baseline leg of bench.py as the checker.  The library and its harness never
import it.

The reference path it restates: GEMM/gemm_main.cpp:39-53 (fp32 CPU GEMM over
fp8 inputs) with the fp8 types of GEMM/include/gemm.cuh:6-7; the sparse-times-dense
loop is that loop over the stored entries of the reference's sparse operand formats
(GEMM/include/bm_test_utils.h:48-128), for which the reference holds no loop of its own.
"""
import ctypes
import os
import subprocess

import numpy as np

E4M3 = 0
E5M2 = 1

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None


def build(force=False):
    """Compile liboracle.so with gcc (a few seconds)."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        build()
    L = ctypes.CDLL(_LIB_PATH)
    u8p = ctypes.POINTER(ctypes.c_uint8)
    f32p = ctypes.POINTER(ctypes.c_float)
    f64p = ctypes.POINTER(ctypes.c_double)
    i32p = ctypes.POINTER(ctypes.c_int)
    L.oracle_fp8_decode.restype = ctypes.c_float
    L.oracle_fp8_decode.argtypes = [ctypes.c_uint8, ctypes.c_int]
    L.oracle_fp8_encode.restype = ctypes.c_uint8
    L.oracle_fp8_encode.argtypes = [ctypes.c_float, ctypes.c_int]
    L.oracle_fp8_encode_array.restype = None
    L.oracle_fp8_encode_array.argtypes = [f32p, u8p, ctypes.c_size_t, ctypes.c_int]
    L.oracle_fp8_decode_array.restype = None
    L.oracle_fp8_decode_array.argtypes = [u8p, f32p, ctypes.c_size_t, ctypes.c_int]
    L.oracle_gemm_verbatim.restype = None
    L.oracle_gemm_verbatim.argtypes = [ctypes.c_int] * 3 + [u8p, ctypes.c_int, u8p, ctypes.c_int, f32p]
    L.oracle_gemm_fast.restype = None
    L.oracle_gemm_fast.argtypes = [ctypes.c_int] * 3 + [u8p, ctypes.c_int, u8p, ctypes.c_int,
                                                        i32p, ctypes.c_int, f32p, f64p]
    L.oracle_spmm_csr.restype = None
    L.oracle_spmm_csr.argtypes = [ctypes.c_int] * 3 + [u8p, ctypes.c_int, i32p, i32p, u8p, ctypes.c_int, f32p, f64p]
    L.oracle_sddmm.restype = None
    L.oracle_sddmm.argtypes = [ctypes.c_int] * 3 + [i32p, i32p, u8p, ctypes.c_int, u8p, ctypes.c_int, f32p, f64p]
    L.oracle_num_threads.restype = ctypes.c_int
    L.oracle_set_num_threads.argtypes = [ctypes.c_int]
    _lib = L
    return L


def _p(a, ct):
    return a.ctypes.data_as(ctypes.POINTER(ct))


def decode(codes, fmt):
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    out = np.empty(codes.shape, dtype=np.float32)
    lib().oracle_fp8_decode_array(_p(codes, ctypes.c_uint8), _p(out, ctypes.c_float), codes.size, fmt)
    return out


def encode(values, fmt):
    values = np.ascontiguousarray(values, dtype=np.float32)
    out = np.empty(values.shape, dtype=np.uint8)
    lib().oracle_fp8_encode_array(_p(values, ctypes.c_float), _p(out, ctypes.c_uint8), values.size, fmt)
    return out


def gemm_verbatim(A, afmt, B, bfmt):
    """Single-thread loop in the reference's own order.  A: MxK u8, B: NxK u8."""
    A = np.ascontiguousarray(A, dtype=np.uint8)
    B = np.ascontiguousarray(B, dtype=np.uint8)
    M, K = A.shape
    N, K2 = B.shape
    assert K == K2
    C = np.empty((M, N), dtype=np.float32)
    lib().oracle_gemm_verbatim(M, K, N, _p(A, ctypes.c_uint8), afmt, _p(B, ctypes.c_uint8), bfmt,
                               _p(C, ctypes.c_float))
    return C


def gemm(A, afmt, B, bfmt, rows=None, with_scale=False):
    """Bit-identical fast variant.  rows: optional list of A rows to compute.

    Returns C (len(rows) x N fp32) and, when with_scale, S = sum_k |a*b| (fp64).
    """
    A = np.ascontiguousarray(A, dtype=np.uint8)
    B = np.ascontiguousarray(B, dtype=np.uint8)
    M, K = A.shape
    N, K2 = B.shape
    assert K == K2
    if rows is not None:
        rows = np.ascontiguousarray(rows, dtype=np.int32)
        assert rows.min() >= 0 and rows.max() < M
        R = rows.size
        rp = _p(rows, ctypes.c_int)
    else:
        R = M
        rp = None
    C = np.empty((R, N), dtype=np.float32)
    S = np.empty((R, N), dtype=np.float64) if with_scale else None
    lib().oracle_gemm_fast(M, K, N, _p(A, ctypes.c_uint8), afmt, _p(B, ctypes.c_uint8), bfmt,
                           rp, R, _p(C, ctypes.c_float), _p(S, ctypes.c_double) if with_scale else None)
    return (C, S) if with_scale else C


def spmm_csr(values, sfmt, row_offsets, col, k, B, bfmt, with_scale=False):
    """Sparse (CSR, m x k) times dense (B stored n x k) -> m x n fp32, entries of a row added in
    storage order as a running fp32 sum.  A one-dimensional B (k codes) is the SpMV and gives m floats."""
    values = np.ascontiguousarray(values, dtype=np.uint8)
    row_offsets = np.ascontiguousarray(row_offsets, dtype=np.int32)
    col = np.ascontiguousarray(col, dtype=np.int32)
    B = np.ascontiguousarray(B, dtype=np.uint8)
    vector = B.ndim == 1
    B2 = B.reshape(1, -1) if vector else B
    m, (n, k2) = row_offsets.size - 1, B2.shape
    assert k == k2 and row_offsets[0] == 0 and row_offsets[-1] == values.size == col.size
    assert col.size == 0 or (col.min() >= 0 and col.max() < k)
    out = np.empty((m, n), dtype=np.float32)
    S = np.empty((m, n), dtype=np.float64) if with_scale else None
    lib().oracle_spmm_csr(m, k, n, _p(values, ctypes.c_uint8), sfmt, _p(row_offsets, ctypes.c_int), _p(col, ctypes.c_int),
                          _p(B2, ctypes.c_uint8), bfmt, _p(out, ctypes.c_float), _p(S, ctypes.c_double) if with_scale else None)
    if vector:
        out = out[:, 0]
        S = S[:, 0] if with_scale else None
    return (out, S) if with_scale else out


def sddmm(row_offsets, col, vec, lhs, lfmt, rhs, rfmt, with_scale=False):
    """Sampled dense-dense product (the reference's Host_sddmm, GEMM/include/bm_test_utils.h:172-194):
    out[j*vec + v] = lhs[i*vec + v] . rhs[col[j]] for every stored entry j of vector row i.
    lhs: (m_vec*vec, k) codes, rhs: (n, k) codes.  Returns (nnz, vec) fp32."""
    row_offsets = np.ascontiguousarray(row_offsets, dtype=np.int32)
    col = np.ascontiguousarray(col, dtype=np.int32)
    lhs = np.ascontiguousarray(lhs, dtype=np.uint8)
    rhs = np.ascontiguousarray(rhs, dtype=np.uint8)
    m_vec, k = row_offsets.size - 1, lhs.shape[1]
    assert lhs.shape[0] == m_vec * vec and rhs.shape[1] == k and row_offsets[-1] == col.size
    assert col.size == 0 or (col.min() >= 0 and col.max() < rhs.shape[0])
    out = np.empty((col.size, vec), dtype=np.float32)
    S = np.empty((col.size, vec), dtype=np.float64) if with_scale else None
    lib().oracle_sddmm(m_vec, k, vec, _p(row_offsets, ctypes.c_int), _p(col, ctypes.c_int), _p(lhs, ctypes.c_uint8), lfmt,
                       _p(rhs, ctypes.c_uint8), rfmt, _p(out, ctypes.c_float), _p(S, ctypes.c_double) if with_scale else None)
    return (out, S) if with_scale else out


def bell_to_csr(values, block_cols, block):
    """Blocked-ELL (the format behind the reference's GenerateUniformBlockedELLIndex,
    GEMM/include/bm_test_utils.h:48-68: square blocks of `block`, every block row stores the same
    number of blocks; values m x (ell_cols*block) codes, block_cols (m/block) x ell_cols block
    column numbers, -1 = padding that holds nothing) -> (values, row_offsets, col) in CSR, every
    stored element of a block an entry (zeros included), in storage order."""
    values = np.ascontiguousarray(values, dtype=np.uint8)
    block_cols = np.ascontiguousarray(block_cols, dtype=np.int32)
    m, kell = values.shape
    nbr, ell = block_cols.shape
    assert m == nbr * block and kell == ell * block
    cols = (block_cols[:, :, None] * block + np.arange(block, dtype=np.int32)[None, None, :]).reshape(nbr, kell)
    keep = np.repeat(block_cols >= 0, block, axis=1)                    # (nbr, kell)
    keep_rows = np.repeat(keep, block, axis=0)                          # (m, kell)
    cols_rows = np.repeat(cols, block, axis=0)
    row_offsets = np.zeros(m + 1, dtype=np.int32)
    row_offsets[1:] = np.cumsum(keep_rows.sum(axis=1))
    return values[keep_rows], row_offsets, cols_rows[keep_rows].astype(np.int32)


def tolerance(K, S):
    """The parity bound: |C_gpu - C_ref| <= 2*K*2^-24 * sum_k |a_ik*b_kj|."""
    return 2.0 * K * 2.0 ** -24 * S


def num_threads():
    return lib().oracle_num_threads()


def set_num_threads(n):
    lib().oracle_set_num_threads(int(n))
