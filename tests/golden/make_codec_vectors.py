"""Writes tests/golden/codec_vectors.npz: float32 inputs and the fp8 codes two
independent library implementations assign to them.

Sources of the expected codes (neither is the code under test, neither is the
reference):
  * ROCm's host-side OCP FP8 conversion, hip/hip_fp8.h
    (__hip_cvt_float_to_fp8, saturate-to-finite), through hipfp8_ref.cpp;
  * PyTorch's float32 -> float8_e4m3fn / float8_e5m2 casts, on the inputs
    where a cast is defined the same way (finite, inside the finite range).
The script asserts that the two agree wherever both apply, then stores ROCm's
codes.  +-Inf is left out on purpose: ROCm maps it to NaN/Inf codes, the
reference's CUDA conversion saturates it; that case is covered by a hand-written
threshold test instead.

Run from the repository root:  python tests/golden/make_codec_vectors.py
"""
import ctypes
import os
import subprocess
import tempfile

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def build_helper():
    so = os.path.join(tempfile.mkdtemp(), "libhipfp8_ref.so")
    subprocess.check_call(["hipcc", "-std=c++17", "-O2", "-fPIC", "-shared", "--offload-arch=gfx950", "-x", "hip",
                           os.path.join(HERE, "hipfp8_ref.cpp"), "-o", so], stderr=subprocess.DEVNULL)
    return ctypes.CDLL(so)


def rocm_encode(L, x, fmt):
    out = np.zeros(x.size, dtype=np.uint8)
    L.hipfp8_encode(x.ctypes.data_as(ctypes.c_void_p), out.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(x.size), fmt)
    return out


def finite_values(fmt):
    """Every finite value of the format, from the OCP definition (sign, exponent, mantissa)."""
    mbits, bias, top = (3, 7, 0x7E) if fmt == 0 else (2, 15, 0x7B)
    vals = []
    for c in range(top + 1):
        E, Mn = c >> mbits, c & ((1 << mbits) - 1)
        v = Mn * 2.0 ** (1 - bias - mbits) if E == 0 else (1 + Mn / (1 << mbits)) * 2.0 ** (E - bias)
        vals.append(v)
    return np.array(vals, dtype=np.float64)


def main():
    L = build_helper()
    rng = np.random.default_rng(20240607)
    pieces = []
    for fmt in (0, 1):
        v = finite_values(fmt)
        mid = (v[:-1] + v[1:]) / 2                      # exact ties between neighbours
        for arr in (v, mid):
            f = arr.astype(np.float32)
            pieces += [f, np.nextafter(f, np.float32(np.inf)), np.nextafter(f, np.float32(-np.inf))]
        top = v[-1]
        ulp = v[-1] - v[-2]
        pieces.append(np.array([top + ulp / 4, top + ulp / 2, top + ulp, 2 * top, 1e9, 3e38], dtype=np.float32))
    mag = np.exp2(rng.uniform(-20, 17, 20000)).astype(np.float32)
    pieces.append(mag * rng.choice([-1.0, 1.0], mag.size).astype(np.float32))
    pieces.append(rng.standard_normal(5000).astype(np.float32))
    pieces.append(np.array([0.0, -0.0, np.float32(1e-45), np.float32(-1e-45), np.float32(1.1754944e-38)], dtype=np.float32))
    x = np.concatenate(pieces).astype(np.float32)
    x = np.concatenate([x, -x])
    x = x[np.isfinite(x)]

    expect = {}
    for fmt, dt, top in ((0, torch.float8_e4m3fn, 448.0), (1, torch.float8_e5m2, 57344.0)):
        r = rocm_encode(L, x, fmt)
        t = torch.from_numpy(x).to(dt).view(torch.uint8).numpy()
        inside = np.abs(x) <= top                       # torch does not saturate: compare inside the range only
        bad = np.nonzero(inside & (r != t))[0]
        assert bad.size == 0, "ROCm and torch disagree on %d inputs, first %r" % (bad.size, x[bad[:5]])
        expect[fmt] = r
    np.savez_compressed(os.path.join(HERE, "codec_vectors.npz"), x=x, e4m3=expect[0], e5m2=expect[1])
    print("wrote %d vectors" % x.size)


if __name__ == "__main__":
    main()
