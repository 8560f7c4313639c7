"""GPU parity of the extended epilogue (fp8gemm_launch_ex): scaled, 16-bit output.

Expected value = cast(alpha * a_scale * b_scale * C_ref) with C_ref from the CPU oracle.  The
GPU sum differs from the oracle's by at most tol = 2*K*2^-24*sum|a*b| before scaling, so
    |out - scale*C_ref| <= |scale|*tol + (half an output ulp at |scale*C_ref| + |scale|*tol),
and where the fp32 sums are exact (small integers) the 16-bit result is bit-exact.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def ulp16(x, mant_bits, min_exp):
    """Spacing of the 16-bit format (mant_bits explicit mantissa bits) at |x|."""
    ax = np.maximum(np.abs(x), 2.0 ** min_exp)
    return 2.0 ** (np.floor(np.log2(ax)) - mant_bits)


FORMATS = {"float32": (23, -126), "bfloat16": (7, -126), "float16": (10, -14)}


def run_ex(pkg, A, fa, B, fb, dtype, alpha, sa, sb):
    import torch
    dA = torch.from_numpy(A).cuda()
    dB = torch.from_numpy(B).cuda()
    tdtype = getattr(torch, dtype)
    out = torch.full((A.shape[0], B.shape[0]), float("nan"), dtype=tdtype, device="cuda")
    ta = None if sa is None else torch.tensor([sa], dtype=torch.float32, device="cuda")
    tb = None if sb is None else torch.tensor([sb], dtype=torch.float32, device="cuda")
    pkg.gemm_ex(dA, dB, out=out, alpha=alpha, a_scale=ta, b_scale=tb, a_fmt=fa, b_fmt=fb)
    torch.cuda.synchronize()
    return out.float().cpu().numpy().astype(np.float64)


SHAPES = [
    (256, 1024, 512),       # persistent tiled kernel, whole tiles
    (300, 2048, 250),       # tiles that overhang C (n not a multiple of 4: guarded element stores)
    (16, 4096, 1024),       # weight-streaming kernel
    (48, 8192, 256),        # weight-streaming kernel with K slices + reduction
    (256, 8192, 1024),      # tiled kernel with K slices + tile-slot reduction
    (70, 200, 90),          # general kernel (k not a multiple of 16)
    (512, 1040, 384),       # K tile overhanging K
    (3584, 256, 3584),      # 256 x 256 tiles on the 16x16x128 MFMA
    (3072, 384, 3072),      # 192 x 256 tiles on the 16x16x128 MFMA, odd count of K tiles
]


@pytest.mark.parametrize("dtype", ["bfloat16", "float16", "float32"])
@pytest.mark.parametrize("shape", SHAPES)
def test_scaled_16_bit_output(pkg, oracle, dtype, shape):
    M, K, N = shape
    fa, fb = (0, 1) if K % 3 else (1, 0)
    A = pkg.fill((M, K), fa, seed=0xA11CE + 300 + K, dist="normal", sigma=1.0)
    B = pkg.fill((N, K), fb, seed=0xB0B + 300 + K, dist="normal", sigma=1.0)
    alpha, sa, sb = 0.5, 0.125, 3.0
    scale = float(np.float32(np.float32(alpha) * np.float32(sa)) * np.float32(sb))
    got = run_ex(pkg, A, fa, B, fb, dtype, alpha, sa, sb)
    Cref, S = oracle.gemm(A, fa, B, fb, with_scale=True)
    want = scale * Cref.astype(np.float64)
    tol = abs(scale) * oracle.tolerance(K, S)
    mant, emin = FORMATS[dtype]
    bound = tol + 0.5 * ulp16(np.abs(want) + tol, mant, emin) + np.abs(want) * 2.0 ** -23
    assert np.isfinite(got).all()
    err = np.abs(got - want)
    assert (err <= bound).all(), "worst err/bound = %g" % float((err / bound).max())


@pytest.mark.parametrize("dtype", ["bfloat16", "float16"])
@pytest.mark.parametrize("shape", [(256, 512, 256), (16, 1024, 512), (100, 256, 60), (64, 112, 64)])
def test_exact_sums_round_to_nearest_even(pkg, oracle, dtype, shape):
    """Small-integer operands: the fp32 sum is exact, so the 16-bit output must be exactly the
    round-to-nearest-even of scale * sum (torch's own float32 -> 16-bit cast as the referee)."""
    import torch
    M, K, N = shape
    rng = np.random.default_rng(K + N)
    va = rng.integers(-4, 5, size=(M, K)).astype(np.float32)
    vb = rng.integers(-4, 5, size=(N, K)).astype(np.float32)
    A, B = pkg.encode(va, 0), pkg.encode(vb, 0)
    exact = va.astype(np.int64) @ vb.astype(np.int64).T
    alpha = 0.3125        # not a power of two: products need rounding in the 16-bit formats
    got = run_ex(pkg, A, 0, B, 0, dtype, alpha, None, None)
    want32 = (np.float32(alpha) * exact.astype(np.float32)).astype(np.float32)       # exact in fp32 (|sum| < 2^14)
    want = torch.from_numpy(want32).to(getattr(torch, dtype)).float().numpy().astype(np.float64)
    assert np.array_equal(got, want)


def test_plain_call_equals_ex_with_unit_scales(pkg, oracle):
    """fp8gemm_launch and fp8gemm_launch_ex(fp32, alpha = 1, no scales) give identical bits."""
    import torch
    for (M, K, N) in [(512, 1024, 512), (16, 2048, 512), (70, 200, 90), (256, 8192, 1024)]:
        A = pkg.fill((M, K), 0, seed=0xA11CE + 400 + K, dist="normal")
        B = pkg.fill((N, K), 0, seed=0xB0B + 400 + K, dist="normal")
        dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
        plain = pkg.gemm(dA, dB, a_fmt=0, b_fmt=0)
        ex = pkg.gemm_ex(dA, dB, out_dtype=torch.float32, a_fmt=0, b_fmt=0)
        torch.cuda.synchronize()
        assert torch.equal(plain, ex), (M, K, N)
