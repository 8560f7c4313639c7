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
    (48, 8192, 256),        # 64 x 128 weight-streaming tiles with K slices, summed inside the kernel
    (256, 8192, 1024),      # 128 x 128 tiles with K slices, summed inside the kernel
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


# ------------------------------------------------------------------ beta * C, D scale, amax
def run_full(pkg, A, fa, B, fb, d_dtype, alpha, beta, Cin, c_dtype, sa, sb, sc, sd, want_amax=True, in_place=False):
    import torch
    dA = torch.from_numpy(A).cuda()
    dB = torch.from_numpy(B).cuda()
    one = lambda v: None if v is None else torch.tensor([v], dtype=torch.float32, device="cuda")
    dC = None if Cin is None else torch.from_numpy(Cin).cuda().to(getattr(torch, c_dtype))
    if in_place:
        out = dC
    else:
        out = torch.full((A.shape[0], B.shape[0]), float("nan"), dtype=getattr(torch, d_dtype), device="cuda")
    amax = torch.full((1,), -7.0, dtype=torch.float32, device="cuda") if want_amax else None    # stale value: must be overwritten
    c_used = None if dC is None else dC.float().cpu().numpy().astype(np.float64)                # C as the kernel reads it
    pkg.gemm_epilogue(dA, dB, out=out, alpha=alpha, beta=beta, c=dC, a_scale=one(sa), b_scale=one(sb), c_scale=one(sc),
                      d_scale=one(sd), amax=amax, a_fmt=fa, b_fmt=fb)
    torch.cuda.synchronize()
    return out.float().cpu().numpy().astype(np.float64), (None if amax is None else float(amax.item())), c_used


EPI_SHAPES = [
    (256, 1024, 512),       # persistent tiled kernel, whole tiles
    (300, 2048, 250),       # tiles that overhang C, n not a multiple of 4
    (16, 4096, 1024),       # weight-streaming kernel
    (48, 8192, 256),        # 64 x 128 weight-streaming tiles with K slices, summed inside the kernel
    (256, 8192, 1024),      # 128 x 128 tiles with K slices, summed inside the kernel
    (70, 200, 90),          # general kernel
    (3584, 256, 3584),      # 256 x 256 tiles on the 16x16x128 MFMA
]


def check_full_epilogue(pkg, oracle, shape, d_dtype, c_dtype, rows=None):
    """d = cast(sd * (alpha*sa*sb*sum + beta*sc*C)), amax = max|.| before sd: against the oracle's
    sum within the fp32 reordering bound carried through the epilogue, plus the rounding of the
    epilogue's own fp32 operations and half an ulp of the output format.  rows: check these rows
    of the result only (amax is then bounded from below by them)."""
    M, K, N = shape
    fa, fb = (0, 1) if K % 3 else (1, 0)
    A = pkg.fill((M, K), fa, seed=0xA11CE + 600 + K, dist="normal", sigma=1.0)
    B = pkg.fill((N, K), fb, seed=0xB0B + 600 + K, dist="normal", sigma=1.0)
    rng = np.random.default_rng(M * 7 + N)
    Cin = (rng.standard_normal((M, N)) * 40.0).astype(np.float32)
    alpha, beta, sa, sb, sc, sd = 0.5, -1.5, 0.125, 3.0, 0.75, 0.0625
    got, amax, c_used = run_full(pkg, A, fa, B, fb, d_dtype, alpha, beta, Cin, c_dtype, sa, sb, sc, sd)
    assert np.isfinite(got).all()
    if rows is None:
        Cref, S = oracle.gemm(A, fa, B, fb, with_scale=True)
    else:
        Cref, S = oracle.gemm(A, fa, B, fb, rows=rows, with_scale=True)
        got, c_used = got[rows], c_used[rows]
    fab = float(np.float32(np.float32(alpha) * np.float32(sa)) * np.float32(sb))
    fc = float(np.float32(beta) * np.float32(sc))
    y = fab * Cref.astype(np.float64) + fc * c_used
    mag = np.abs(fab * Cref.astype(np.float64)) + np.abs(fc * c_used)
    ytol = abs(fab) * oracle.tolerance(K, S) + 3.0 * mag * 2.0 ** -24            # three fp32 roundings
    want = sd * y
    mant, emin = FORMATS[d_dtype]
    bound = sd * ytol + 0.5 * ulp16(np.abs(want) + sd * ytol, mant, emin) + np.abs(want) * 2.0 ** -23
    err = np.abs(got - want)
    assert (err <= bound).all(), "worst err/bound = %g" % float((err / bound).max())
    # amax: the largest |y| (before sd), within the tolerance of the element that attains it
    assert amax is not None and amax > 0
    if rows is None:
        assert abs(amax - np.abs(y).max()) <= ytol.max() + np.abs(y).max() * 2.0 ** -22
    else:
        assert amax >= np.abs(y).max() - ytol.max() - np.abs(y).max() * 2.0 ** -22


@pytest.mark.parametrize("d_dtype,c_dtype", [("float32", "float32"), ("bfloat16", "float32"), ("float16", "bfloat16"),
                                             ("float32", "float16")])
@pytest.mark.parametrize("shape", EPI_SHAPES)
def test_beta_c_d_scale_and_amax(pkg, oracle, shape, d_dtype, c_dtype):
    check_full_epilogue(pkg, oracle, shape, d_dtype, c_dtype)


@pytest.mark.parametrize("d_dtype,c_dtype", [("bfloat16", "float32"), ("float32", "float16")])
def test_epilogue_in_the_reduction_kernel(pkg, oracle, d_dtype, c_dtype):
    """128 x 256 tiles in 8 K slices: too large for the in-kernel sum, so the slices are added up,
    and the epilogue applied, by the reduction kernel (sampled rows against the oracle)."""
    shape = (256, 16384, 4096)
    fam, var, slices, _ = pkg.plan(*shape)
    assert fam == pkg.ALGO_TILE and var in (5, 8, 0, 13) and slices > 1
    check_full_epilogue(pkg, oracle, shape, d_dtype, c_dtype, rows=np.arange(0, 256, 8, dtype=np.int32))


@pytest.mark.parametrize("shape", [(256, 512, 256), (16, 1024, 512), (100, 256, 60), (48, 8192, 256), (256, 8192, 1024)])
def test_epilogue_is_exact_on_small_integers(pkg, oracle, shape):
    """Small-integer operands and C, power-of-two scales: every step is exact in fp32, so d and
    amax equal the integer arithmetic bit for bit; in place (c == d) gives the same."""
    M, K, N = shape
    rng = np.random.default_rng(K + 3 * N)
    va = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
    vb = rng.integers(-3, 4, size=(N, K)).astype(np.float32)
    Cin = rng.integers(-1000, 1001, size=(M, N)).astype(np.float32)
    A, B = pkg.encode(va, 0), pkg.encode(vb, 1)
    exact = (va.astype(np.int64) @ vb.astype(np.int64).T).astype(np.float64)
    alpha, beta, sa, sb, sc, sd = 2.0, -0.5, 0.5, 4.0, 2.0, 0.25
    y = alpha * sa * sb * exact + beta * sc * Cin.astype(np.float64)
    got, amax, _ = run_full(pkg, A, 0, B, 1, "float32", alpha, beta, Cin, "float32", sa, sb, sc, sd)
    assert np.array_equal(got, sd * y)
    assert amax == np.abs(y).max()
    got2, amax2, _ = run_full(pkg, A, 0, B, 1, "float32", alpha, beta, Cin, "float32", sa, sb, sc, sd, in_place=True)
    assert np.array_equal(got2, sd * y) and amax2 == amax
    # without C: beta and c_scale are ignored; without amax: nothing is written there
    got3, amax3, _ = run_full(pkg, A, 0, B, 1, "float32", alpha, 123.0, None, "float32", sa, sb, 55.0, sd, want_amax=False)
    assert np.array_equal(got3, sd * alpha * sa * sb * exact) and amax3 is None


def test_epilogue_argument_validation(pkg):
    import ctypes
    L = pkg.lib()
    p = ctypes.c_void_p(0x1000)
    q = ctypes.c_void_p(0x2000)
    args = lambda d_type, alpha, beta, c, c_type, d=p: (128, 128, 128, p, 0, p, 0, d, d_type, alpha, beta, c, c_type,
                                                        None, None, None, None, None, None)
    assert L.fp8gemm_launch_epilogue(*args(3, 1.0, 0.0, None, 0)) == 1            # bad output type
    assert L.fp8gemm_launch_epilogue(*args(0, 1.0, 0.0, q, 5)) == 1               # bad C type
    assert L.fp8gemm_launch_epilogue(*args(0, 1.0, float("nan"), q, 0)) == 1      # NaN beta
    assert L.fp8gemm_launch_epilogue(*args(1, 1.0, 1.0, p, 0)) == 1               # in place with two element types
    assert L.fp8gemm_launch_epilogue(*args(0, 1.0, 0.0, None, 0, d=None)) == 1    # no output
