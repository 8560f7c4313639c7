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


def test_noalloc_entry_under_graph_capture_and_replay(pkg):
    """What the entry point is for: K-sliced launches captured into a HIP graph (tiles whose
    slices are added up inside the kernel, and tiles that take the reduction kernel), replayed
    several times with eager launches of other shapes and synchronisations in between.  Every
    replay must reproduce the eager result bit for bit: the arrival counters are back at zero
    after each launch, nothing is cleared from the host, nothing is allocated."""
    import torch
    L = pkg.lib()
    noalloc = _bind(L)
    shapes = [(64, 8192, 2048), (256, 8192, 2048), (100, 8192, 1000), (16, 4096, 512)]
    side = torch.cuda.Stream()
    cases = []
    for (M, K, N) in shapes:
        dA = torch.from_numpy(pkg.fill((M, K), 0, seed=0xA11CE + 800 + N, dist="normal", sigma=2.0)).cuda()
        dB = torch.from_numpy(pkg.fill((N, K), 1, seed=0xB0B + 800 + N, dist="normal", sigma=2.0)).cuda()
        ref = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        pkg.gemm(dA, dB, out=ref, a_fmt=0, b_fmt=1)
        got = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        cases.append((M, K, N, dA, dB, ref, got))
    assert any(pkg.plan(M, K, N)[2] > 1 for (M, K, N) in shapes)
    torch.cuda.synchronize()

    def enqueue():
        for (M, K, N, dA, dB, ref, got) in cases:
            assert noalloc(M, K, N, dA.data_ptr(), 0, dB.data_ptr(), 1, got.data_ptr(), 2, side.cuda_stream) == 0
    with torch.cuda.stream(side):
        enqueue()                  # eager, before the capture: the static array's address is looked up here
    side.synchronize()
    for (M, K, N, dA, dB, ref, got) in cases:
        assert torch.equal(got, ref), ("eager", M, K, N)
    held = L.fp8gemm_scratch_held_bytes()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        enqueue()
    other = cases[1]
    for replay in range(4):
        for (M, K, N, dA, dB, ref, got) in cases:
            got.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for (M, K, N, dA, dB, ref, got) in cases:
            assert torch.equal(got, ref), (replay, M, K, N)
        # eager work of the program's own between the replays, on the default stream
        tmp = torch.empty_like(other[5])
        pkg.gemm(other[3], other[4], out=tmp, a_fmt=0, b_fmt=1)
        torch.cuda.synchronize()
        assert torch.equal(tmp, other[5])
    assert L.fp8gemm_scratch_held_bytes() == held
