"""The entry point that allocates nothing (fp8gemm_launch_noalloc): K-slice partial sums go
to a static device array of the library, so callers that cannot call hipMalloc (graph
capture, tight serving loops) can still run K-sliced shapes.  Checked through the C ABI
against fp8gemm_launch: same plan, same kernels, so the outputs agree bit for bit."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

STATIC_SCRATCH_BYTES = 64 << 20


def _bind(L):
    return L.fp8gemm_launch_noalloc


def test_noalloc_entry_matches_the_allocating_one_on_two_calls_in_a_row(pkg, oracle):
    import torch
    L = pkg.lib()
    noalloc = _bind(L)
    stream = torch.cuda.current_stream().cuda_stream
    held_before = L.fp8gemm_scratch_held_bytes()
    # the second call is smaller than the first: it finds the first call's partial sums in the
    # array and must not be disturbed by them; the third needs no scratch at all; the fourth
    # is a weight-streaming shape whose K is cut
    shapes = [(256, 8192, 2048, 0, 0), (256, 8192, 1024, 0, 1), (512, 1024, 768, 1, 0), (64, 8192, 2048, 1, 1)]
    outs = []
    for (M, K, N, fa, fb) in shapes:
        assert (L.fp8gemm_scratch_bytes(M, K, N) > 0) == (pkg.plan(M, K, N)[2] > 1)
        A = pkg.fill((M, K), fa, seed=0xA11CE + 700 + N, dist="normal", sigma=2.0)
        B = pkg.fill((N, K), fb, seed=0xB0B + 700 + N, dist="normal", sigma=2.0)
        dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
        got = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        outs.append((A, B, dA, dB, got, fa, fb))
    torch.cuda.synchronize()
    held = L.fp8gemm_scratch_held_bytes()
    for (M, K, N, fa, fb), (A, B, dA, dB, got, _, _) in zip(shapes, outs):
        assert noalloc(M, K, N, dA.data_ptr(), fa, dB.data_ptr(), fb, got.data_ptr(), 2, stream) == 0
    torch.cuda.synchronize()
    assert L.fp8gemm_scratch_held_bytes() == held == held_before      # nothing was allocated
    for (M, K, N, fa, fb), (A, B, dA, dB, got, _, _) in zip(shapes, outs):
        ref = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        pkg.gemm(dA, dB, out=ref, a_fmt=fa, b_fmt=fb)
        torch.cuda.synchronize()
        assert torch.equal(got, ref), (M, K, N)
        Cref, S = oracle.gemm(A, fa, B, fb, with_scale=True)
        err = np.abs(got.cpu().numpy().astype(np.float64) - Cref)
        assert (err <= oracle.tolerance(K, S)).all()


def test_noalloc_entry_refuses_what_the_static_array_cannot_hold(pkg):
    """A plan whose partial sums exceed the array is rejected with hipErrorOutOfMemory before
    anything is launched; bad arguments are rejected as everywhere else."""
    import torch
    L = pkg.lib()
    noalloc = _bind(L)
    stream = torch.cuda.current_stream().cuda_stream
    M, K, N = 768, 32768, 12288
    need = L.fp8gemm_scratch_bytes(M, K, N)
    assert need > STATIC_SCRATCH_BYTES
    dA = torch.zeros((M, K), dtype=torch.uint8, device="cuda")
    dB = torch.zeros((N, K), dtype=torch.uint8, device="cuda")
    out = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    assert noalloc(M, K, N, dA.data_ptr(), 0, dB.data_ptr(), 0, out.data_ptr(), 2, stream) == 2
    torch.cuda.synchronize()
    assert bool(torch.isnan(out).all())
    assert noalloc(0, K, N, dA.data_ptr(), 0, dB.data_ptr(), 0, out.data_ptr(), 2, stream) == 1
    assert noalloc(M, K, N, None, 0, dB.data_ptr(), 0, out.data_ptr(), 2, stream) == 1
