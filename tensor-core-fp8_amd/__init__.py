"""Python plumbing over the C ABI of the gfx950 FP8 GEMM library.

The product is the shared library ``lib/libfp8gemm.so`` (HIP kernels + C ABI,
``include/fp8gemm.h``) and the C++ harness under ``GEMM/``.  This module only
loads the library with ctypes and passes torch device pointers through, so
that tests and the benchmark can drive the same entry points a C++ caller
binds.  There is no fallback: if the library is missing, loading raises.

``GEMM`` / ``GEMM4`` mirror the reference's launch API
(GEMM/include/gemm.cuh:11-55): argument order (m, k, n, a, b, out), the
operand pairing chosen by the operand types (here: torch.float8_e4m3fn /
torch.float8_e5m2 tensors).
"""
import ctypes
import os
import subprocess

E4M3 = 0
E5M2 = 1
ALGO_AUTO, ALGO_DIRECT, ALGO_TILE, ALGO_SKINNY = 0, 1, 2, 3
NOALLOC_SCRATCH_BYTES = 64 << 20      # FP8GEMM_NOALLOC_SCRATCH_BYTES: the static array behind fp8gemm_launch_noalloc

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libfp8gemm.so")
HARNESS_DIR = os.path.join(_HERE, "GEMM")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "fp8gemm.h")

_lib = None

ENTRY_POINTS = [
    "fp8gemm_e4m3_e4m3_stage2", "fp8gemm_e4m3_e4m3_stage4",
    "fp8gemm_e5m2_e5m2_stage2", "fp8gemm_e5m2_e5m2_stage4",
    "fp8gemm_e4m3_e5m2_stage2", "fp8gemm_e4m3_e5m2_stage4",
    "fp8gemm_e5m2_e4m3_stage2", "fp8gemm_e5m2_e4m3_stage4",
]


class Fp8GemmError(RuntimeError):
    pass


def build(jobs=8):
    """Compile the library and the harness for gfx950 (hipcc; no GPU needed)."""
    subprocess.check_call(["make", "-C", HARNESS_DIR, "-j", str(jobs), "lib", "gemm", "hipblaslt"])


def lib():
    """The loaded C ABI.  Raises if the shared library has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise Fp8GemmError(
            "libfp8gemm.so is not built (%s); run __graft_entry__.build() or "
            "`make -C tensor-core-fp8_amd/GEMM lib`" % LIB_PATH)
    # torch ships its own copy of the HIP runtime; when both end up in one process the
    # copy loaded first is the one that owns the device, so let torch load first
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    L = ctypes.CDLL(LIB_PATH)
    vp, ci = ctypes.c_void_p, ctypes.c_int
    for name in ENTRY_POINTS:
        fn = getattr(L, name)
        fn.restype = ci
        fn.argtypes = [ci, ci, ci, vp, vp, vp]
    L.fp8gemm_launch.restype = ci
    L.fp8gemm_launch.argtypes = [ci, ci, ci, vp, ci, vp, ci, vp, ci, vp]
    L.fp8gemm_gemv.restype = ci
    L.fp8gemm_gemv.argtypes = [ci, ci, vp, ci, vp, ci, vp, vp]
    L.fp8gemm_launch_ws.restype = ci
    L.fp8gemm_launch_ws.argtypes = [ci, ci, ci, vp, ci, vp, ci, vp, ci, vp, ctypes.c_size_t, vp]
    L.fp8gemm_launch_noalloc.restype = ci
    L.fp8gemm_launch_noalloc.argtypes = [ci, ci, ci, vp, ci, vp, ci, vp, ci, vp]
    L.fp8gemm_release_scratch.restype = ci
    L.fp8gemm_release_scratch.argtypes = []
    L.fp8gemm_scratch_held_bytes.restype = ctypes.c_size_t
    L.fp8gemm_scratch_held_bytes.argtypes = []
    L.fp8gemm_launch_epilogue.restype = ci
    L.fp8gemm_launch_epilogue.argtypes = [ci, ci, ci, vp, ci, vp, ci, vp, ci, ctypes.c_float, ctypes.c_float, vp, ci,
                                          vp, vp, vp, vp, vp, vp]
    L.fp8gemm_launch_ex.restype = ci
    L.fp8gemm_launch_ex.argtypes = [ci, ci, ci, vp, ci, vp, ci, vp, ci, ctypes.c_float, vp, vp, vp]
    L.fp8gemm_launch_algo.restype = ci
    L.fp8gemm_launch_algo.argtypes = [ci, ci, ci, vp, ci, vp, ci, vp, ci, ci, vp]
    L.fp8gemm_launch_tuned.restype = ci
    L.fp8gemm_launch_tuned.argtypes = [ci, ci, ci, vp, ci, vp, ci, vp, ci, ci, ci, vp]
    L.fp8gemm_num_variants.restype = ci
    L.fp8gemm_num_variants.argtypes = [ci]
    L.fp8gemm_select_algo.restype = ci
    L.fp8gemm_select_algo.argtypes = [ci, ci, ci]
    L.fp8gemm_plan.restype = ci
    L.fp8gemm_plan.argtypes = [ci, ci, ci, ci, ctypes.POINTER(ci)]
    L.fp8gemm_scratch_bytes.restype = ctypes.c_size_t
    L.fp8gemm_scratch_bytes.argtypes = [ci, ci, ci]
    L.fp8gemm_device_info.restype = ci
    L.fp8gemm_device_info.argtypes = [ctypes.POINTER(ci)]
    L.fp8gemm_error_string.restype = ctypes.c_char_p
    L.fp8gemm_error_string.argtypes = [ci]
    L.fp8gemm_version.restype = ci
    L.fp8gemm_encode_one.restype = ctypes.c_uint8
    L.fp8gemm_encode_one.argtypes = [ctypes.c_float, ci]
    L.fp8gemm_decode_one.restype = ctypes.c_float
    L.fp8gemm_decode_one.argtypes = [ctypes.c_uint8, ci]
    L.fp8gemm_encode.restype = None
    L.fp8gemm_encode.argtypes = [vp, vp, ctypes.c_size_t, ci]
    L.fp8gemm_decode.restype = None
    L.fp8gemm_decode.argtypes = [vp, vp, ctypes.c_size_t, ci]
    L.fp8gemm_fill_uniform.restype = None
    L.fp8gemm_fill_uniform.argtypes = [vp, ctypes.c_size_t, ci, ctypes.c_uint64, ctypes.c_float, ctypes.c_float]
    L.fp8gemm_fill_normal.restype = None
    L.fp8gemm_fill_normal.argtypes = [vp, ctypes.c_size_t, ci, ctypes.c_uint64, ctypes.c_float, ctypes.c_float]
    L.fp8gemm_fill_weights.restype = None
    L.fp8gemm_fill_weights.argtypes = [vp, ctypes.c_size_t, ci, ctypes.c_uint64, ctypes.c_float]
    L.fp8gemm_fill_loguniform.restype = None
    L.fp8gemm_fill_loguniform.argtypes = [vp, ctypes.c_size_t, ci, ctypes.c_uint64]
    ip = ctypes.c_void_p
    L.fp8gemm_spmm_bell.restype = ci
    L.fp8gemm_spmm_bell.argtypes = [ci, ci, ci, ci, ci, vp, ci, ip, vp, ci, vp, vp]
    L.fp8gemm_spmv_bell.restype = ci
    L.fp8gemm_spmv_bell.argtypes = [ci, ci, ci, ci, vp, ci, ip, vp, ci, vp, vp]
    L.fp8gemm_spmv_csr.restype = ci
    L.fp8gemm_spmv_csr.argtypes = [ci, ci, vp, ci, ip, ip, ip, vp, ci, vp, vp]
    L.fp8gemm_spmm_csr.restype = ci
    L.fp8gemm_spmm_csr.argtypes = [ci, ci, ci, vp, ci, ip, ip, vp, ci, vp, vp]
    L.fp8gemm_spmm_csr_scratch_bytes.restype = ctypes.c_size_t
    L.fp8gemm_spmm_csr_scratch_bytes.argtypes = [ci, ci, ci]
    L.fp8gemm_sddmm.restype = ci
    L.fp8gemm_sddmm.argtypes = [ci, ci, ci, ip, ip, vp, ci, vp, ci, vp, vp]
    L.fp8gemm_sorted_row_swizzle.restype = None
    L.fp8gemm_sorted_row_swizzle.argtypes = [ci, ip, ip]
    _lib = L
    return L


def check(code):
    if code != 0:
        raise Fp8GemmError("fp8gemm error %d: %s" % (code, lib().fp8gemm_error_string(code).decode()))


def plan(m, k, n, stages=2):
    """(family, variant, K slices, columns per wave | rotation mode) that the automatic
    selection uses for a shape."""
    out = (ctypes.c_int * 4)()
    check(lib().fp8gemm_plan(m, k, n, stages, out))
    return tuple(out)


# ---------------------------------------------------------------- host codec
def encode(values, fmt):
    """float32 numpy array -> uint8 codes (RNE, saturate to finite)."""
    import numpy as np
    values = np.ascontiguousarray(values, dtype=np.float32)
    out = np.empty(values.shape, dtype=np.uint8)
    lib().fp8gemm_encode(values.ctypes.data, out.ctypes.data, values.size, fmt)
    return out


def decode(codes, fmt):
    import numpy as np
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    out = np.empty(codes.shape, dtype=np.float32)
    lib().fp8gemm_decode(codes.ctypes.data, out.ctypes.data, codes.size, fmt)
    return out


def fill(shape, fmt, seed, dist="normal", **kw):
    """Seeded synthetic fp8 matrix as a uint8 numpy array (host memory)."""
    import numpy as np
    out = np.empty(shape, dtype=np.uint8)
    L = lib()
    if dist == "normal":
        L.fp8gemm_fill_normal(out.ctypes.data, out.size, fmt, seed, kw.get("mean", 0.0), kw.get("sigma", 1.0))
    elif dist == "uniform":
        L.fp8gemm_fill_uniform(out.ctypes.data, out.size, fmt, seed, kw.get("lo", -1.0), kw.get("hi", 1.0))
    elif dist == "weights":
        L.fp8gemm_fill_weights(out.ctypes.data, out.size, fmt, seed, kw.get("sigma", 0.02))
    elif dist == "loguniform":
        L.fp8gemm_fill_loguniform(out.ctypes.data, out.size, fmt, seed)
    else:
        raise ValueError(dist)
    return out


# ---------------------------------------------------------------- device GEMM
def _fmt_of(t, fmt):
    import torch
    if fmt is not None:
        return fmt
    if t.dtype == torch.float8_e4m3fn:
        return E4M3
    if t.dtype == torch.float8_e5m2:
        return E5M2
    raise TypeError("operand must be float8_e4m3fn / float8_e5m2, or uint8 with an explicit format")


def _stream_handle(stream):
    import torch
    if stream is None:
        stream = torch.cuda.current_stream()
    return ctypes.c_void_p(stream.cuda_stream)


def gemm(a, b, out=None, a_fmt=None, b_fmt=None, stages=2, algo=ALGO_AUTO, variant=None,
         split_k=0, stream=None):
    """out[m, n] = sum_k a[m, k] * b[n, k] on the device holding a and b.

    a: (m, k), b: (n, k) contiguous device tensors of fp8 (or uint8 + format);
    out: (m, n) float32 device tensor, allocated when None.  Launches on
    `stream` (default: torch's current stream) and does not synchronise.
    """
    import torch
    if not (a.is_cuda and b.is_cuda):
        raise Fp8GemmError("operands must live in device memory")
    if not (a.is_contiguous() and b.is_contiguous()):
        raise Fp8GemmError("operands must be contiguous")
    m, k = a.shape
    n, k2 = b.shape
    if k != k2:
        raise Fp8GemmError("inner dimensions differ: %d vs %d" % (k, k2))
    fa, fb = _fmt_of(a, a_fmt), _fmt_of(b, b_fmt)
    if out is None:
        out = torch.empty((m, n), dtype=torch.float32, device=a.device)
    L = lib()
    s = _stream_handle(stream)
    if variant is None and split_k == 0:
        code = L.fp8gemm_launch_algo(m, k, n, a.data_ptr(), fa, b.data_ptr(), fb, out.data_ptr(), stages, algo, s)
    else:
        code = L.fp8gemm_launch_tuned(m, k, n, a.data_ptr(), fa, b.data_ptr(), fb, out.data_ptr(), algo,
                                      -1 if variant is None else variant, split_k, s)
    check(code)
    return out


OUT_F32, OUT_BF16, OUT_F16 = 0, 1, 2


def gemm_ex(a, b, out_dtype=None, out=None, alpha=1.0, a_scale=None, b_scale=None, a_fmt=None, b_fmt=None,
            stream=None):
    """out[m, n] = cast(alpha * a_scale * b_scale * sum_k a[m, k] * b[n, k]) through
    fp8gemm_launch_ex.  out_dtype: torch.float32 / bfloat16 / float16; a_scale, b_scale:
    one-element float32 device tensors or None."""
    import torch
    if not (a.is_cuda and b.is_cuda and a.is_contiguous() and b.is_contiguous()):
        raise Fp8GemmError("operands must be contiguous device tensors")
    m, k = a.shape
    n, k2 = b.shape
    if k != k2:
        raise Fp8GemmError("inner dimensions differ: %d vs %d" % (k, k2))
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype or torch.float32, device=a.device)
    code = {torch.float32: OUT_F32, torch.bfloat16: OUT_BF16, torch.float16: OUT_F16}[out.dtype]
    for s in (a_scale, b_scale):
        if s is not None and not (s.is_cuda and s.dtype == torch.float32 and s.numel() == 1):
            raise Fp8GemmError("scales are one-element float32 device tensors")
    check(lib().fp8gemm_launch_ex(m, k, n, a.data_ptr(), _fmt_of(a, a_fmt), b.data_ptr(), _fmt_of(b, b_fmt),
                                  out.data_ptr(), code, float(alpha),
                                  None if a_scale is None else a_scale.data_ptr(),
                                  None if b_scale is None else b_scale.data_ptr(), _stream_handle(stream)))
    return out


def gemm_epilogue(a, b, out_dtype=None, out=None, alpha=1.0, beta=0.0, c=None, a_scale=None, b_scale=None,
                  c_scale=None, d_scale=None, amax=None, a_fmt=None, b_fmt=None, stream=None):
    """d = cast(d_scale * (alpha * a_scale * b_scale * sum_k a b + beta * c_scale * c)) through
    fp8gemm_launch_epilogue; amax (a one-element float32 device tensor) receives the largest
    magnitude before d_scale.  c: (m, n) device tensor of float32 / bfloat16 / float16 or None;
    the scales are one-element float32 device tensors or None."""
    import torch
    if not (a.is_cuda and b.is_cuda and a.is_contiguous() and b.is_contiguous()):
        raise Fp8GemmError("operands must be contiguous device tensors")
    m, k = a.shape
    n, k2 = b.shape
    if k != k2:
        raise Fp8GemmError("inner dimensions differ: %d vs %d" % (k, k2))
    codes = {torch.float32: OUT_F32, torch.bfloat16: OUT_BF16, torch.float16: OUT_F16}
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype or torch.float32, device=a.device)
    for s in (a_scale, b_scale, c_scale, d_scale, amax):
        if s is not None and not (s.is_cuda and s.dtype == torch.float32 and s.numel() == 1):
            raise Fp8GemmError("scales and amax are one-element float32 device tensors")
    if c is not None and not (c.is_cuda and c.is_contiguous() and tuple(c.shape) == (m, n)):
        raise Fp8GemmError("c must be a contiguous (m, n) device tensor")
    ptr = lambda t: None if t is None else t.data_ptr()
    check(lib().fp8gemm_launch_epilogue(m, k, n, a.data_ptr(), _fmt_of(a, a_fmt), b.data_ptr(), _fmt_of(b, b_fmt),
                                        out.data_ptr(), codes[out.dtype], float(alpha), float(beta), ptr(c),
                                        codes[c.dtype] if c is not None else OUT_F32, ptr(a_scale), ptr(b_scale),
                                        ptr(c_scale), ptr(d_scale), ptr(amax), _stream_handle(stream)))
    return out


_PAIR = {(E4M3, E4M3): "e4m3_e4m3", (E5M2, E5M2): "e5m2_e5m2", (E4M3, E5M2): "e4m3_e5m2", (E5M2, E4M3): "e5m2_e4m3"}


def _entry(m, k, n, a, b, out, stage):
    fn = getattr(lib(), "fp8gemm_%s_stage%d" % (_PAIR[(_fmt_of(a, None), _fmt_of(b, None))], stage))
    return fn(m, k, n, a.data_ptr(), b.data_ptr(), out.data_ptr())


def GEMM(m, k, n, a, b, out):
    """gemm::GEMM of the reference (gemm.cuh:12-15, 24-27, 36-39, 47-50): default
    stream, returns the launch status."""
    return _entry(m, k, n, a, b, out, 2)


def GEMM4(m, k, n, a, b, out):
    """gemm::GEMM4 of the reference (gemm.cuh:18-21, 30-33, 41-44, 52-55)."""
    return _entry(m, k, n, a, b, out, 4)


# ---------------------------------------------------------------- sparse operands
def _dev_ints(t):
    import torch
    if not (t.is_cuda and t.dtype == torch.int32 and t.is_contiguous()):
        raise Fp8GemmError("index arrays are contiguous int32 device tensors")
    return t.data_ptr()


def spmm_bell(values, block_cols, block, b, k, s_fmt=None, b_fmt=None, out=None, stream=None):
    """out[m, n] = S b^T for S (m x k) in blocked-ELL: values (m, ell_cols*block) codes, block_cols
    (m/block, ell_cols) int32 block column numbers (-1 = padding), b (n, k) dense; device tensors.
    A one-dimensional b (k codes) is the matrix-vector product and gives m floats."""
    import torch
    m, kell = values.shape
    ell_cols = block_cols.shape[1]
    if kell != ell_cols * block or block_cols.shape[0] * block != m:
        raise Fp8GemmError("values / block_cols do not fit the block size")
    vector = b.dim() == 1
    n = 1 if vector else b.shape[0]
    if (b.shape[0] if vector else b.shape[1]) != k:
        raise Fp8GemmError("b does not have k columns")
    if out is None:
        out = torch.empty((m,) if vector else (m, n), dtype=torch.float32, device=values.device)
    L = lib()
    fs, fb = _fmt_of(values, s_fmt), _fmt_of(b, b_fmt)
    if vector:
        code = L.fp8gemm_spmv_bell(m, k, block, ell_cols, values.data_ptr(), fs, _dev_ints(block_cols), b.data_ptr(), fb,
                                   out.data_ptr(), _stream_handle(stream))
    else:
        code = L.fp8gemm_spmm_bell(m, k, n, block, ell_cols, values.data_ptr(), fs, _dev_ints(block_cols), b.data_ptr(), fb,
                                   out.data_ptr(), _stream_handle(stream))
    check(code)
    return out


def spmm_csr(values, row_offsets, col_idx, b, k, s_fmt=None, b_fmt=None, out=None, row_order=None, stream=None):
    """out = S b^T for S (m x k) in compressed sparse rows (values codes, row_offsets m+1 and col_idx
    int32; device tensors), b (n, k) dense, or a vector of k codes for the matrix-vector product
    (row_order: optional int32 permutation of the rows, the order the waves take them in)."""
    import torch
    m = row_offsets.numel() - 1
    vector = b.dim() == 1
    n = 1 if vector else b.shape[0]
    if (b.shape[0] if vector else b.shape[1]) != k:
        raise Fp8GemmError("b does not have k columns")
    if out is None:
        out = torch.empty((m,) if vector else (m, n), dtype=torch.float32, device=values.device)
    L = lib()
    fs, fb = _fmt_of(values, s_fmt), _fmt_of(b, b_fmt)
    if vector:
        code = L.fp8gemm_spmv_csr(m, k, values.data_ptr(), fs, _dev_ints(row_offsets), _dev_ints(col_idx),
                                  None if row_order is None else _dev_ints(row_order), b.data_ptr(), fb, out.data_ptr(),
                                  _stream_handle(stream))
    else:
        code = L.fp8gemm_spmm_csr(m, k, n, values.data_ptr(), fs, _dev_ints(row_offsets), _dev_ints(col_idx), b.data_ptr(), fb,
                                  out.data_ptr(), _stream_handle(stream))
    check(code)
    return out


def sorted_row_swizzle(row_offsets):
    """Host: rows ordered by falling number of stored entries (numpy int32 in, numpy int32 out)."""
    import numpy as np
    row_offsets = np.ascontiguousarray(row_offsets, dtype=np.int32)
    out = np.empty(row_offsets.size - 1, dtype=np.int32)
    lib().fp8gemm_sorted_row_swizzle(out.size, row_offsets.ctypes.data, out.ctypes.data)
    return out


def sddmm(row_offsets, col_idx, vec_length, lhs, rhs, l_fmt=None, r_fmt=None, out=None, stream=None):
    """out[j, v] = lhs[i*vec_length + v] . rhs[col_idx[j]] for every stored entry j of vector row i
    (row_offsets, col_idx int32 device tensors; lhs (m_vec*vec_length, k), rhs (n, k) codes)."""
    import torch
    m_vec = row_offsets.numel() - 1
    k = lhs.shape[1]
    if lhs.shape[0] != m_vec * vec_length or rhs.shape[1] != k:
        raise Fp8GemmError("lhs / rhs do not fit the pattern")
    if out is None:
        out = torch.empty((col_idx.numel(), vec_length), dtype=torch.float32, device=lhs.device)
    check(lib().fp8gemm_sddmm(m_vec, k, vec_length, _dev_ints(row_offsets), _dev_ints(col_idx), lhs.data_ptr(), _fmt_of(lhs, l_fmt),
                              rhs.data_ptr(), _fmt_of(rhs, r_fmt), out.data_ptr(), _stream_handle(stream)))
    return out
