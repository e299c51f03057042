"""clblasSgemmNoAlloc (the entry point that allocates nothing) against clblasSgemm, through the C
ABI, bit for bit: both run the same kernels, one on the library's fixed scratch array, the other
on a per-stream buffer.  Each case is two calls in a row, the second on a smaller problem, so
that what the first call left in the shared array is there when the second runs."""
import numpy as np
import pytest
import torch

import clblas_amd
import oracle
from gpu_util import debug_env
from helpers import COL, ROW, NOTRANS, TRANS

pytestmark = pytest.mark.gpu


def _run_both(order, tA, tB, M, N, K, alpha, beta, seed, pad=3, offs=(5, 7, 11)):
    """Returns (status, C) of clblasSgemm and of clblasSgemmNoAlloc on the same inputs."""
    col = order == COL
    ra, ca = ((M, K) if (tA == NOTRANS) == col else (K, M))
    rb, cb = ((K, N) if (tB == NOTRANS) == col else (N, K))
    rc, cc = (M, N) if col else (N, M)
    lda, ldb, ldc = ra + pad, rb + pad, rc + pad
    A = oracle.uniform(offs[0] + lda * ca, seed, np.float32)
    B = oracle.uniform(offs[1] + ldb * cb, seed + 1, np.float32)
    C = oracle.uniform(offs[2] + ldc * cc, seed + 2, np.float32)
    dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    out = []
    for fn in (clblas_amd.sgemm, clblas_amd.sgemm_noalloc):
        dC = torch.from_numpy(C).cuda()
        st = fn(order, tA, tB, M, N, K, alpha, dA, offs[0], lda, dB, offs[1], ldb, beta, dC, offs[2], ldc)
        torch.cuda.synchronize()
        out.append((st, dC.cpu().numpy(), clblas_amd.last_dispatch()[0]))
    return out


# (first problem, second and smaller problem); K ranges and sliced tails both use the scratch array
CASES = [
    ("split-K, deep K",      (COL, NOTRANS, NOTRANS, 127, 129, 8192), (COL, TRANS, NOTRANS, 65, 70, 4100)),
    ("split-K, larger tile", (COL, NOTRANS, TRANS, 1024, 1024, 8192), (ROW, NOTRANS, NOTRANS, 500, 300, 6000)),
    ("sliced tail",          (COL, NOTRANS, NOTRANS, 2304, 2304, 640), (COL, TRANS, TRANS, 1100, 1000, 520)),
    ("no scratch needed",    (COL, NOTRANS, NOTRANS, 2048, 2048, 300), (ROW, TRANS, NOTRANS, 64, 64, 64)),
]


@pytest.mark.parametrize("name,first,second", CASES, ids=[c[0] for c in CASES])
def test_noalloc_equals_sgemm_twice_in_a_row(name, first, second):
    assert clblas_amd.setup() == 0
    used_scratch = False
    for i, (order, tA, tB, M, N, K) in enumerate((first, second)):
        (st0, c0, d0), (st1, c1, d1) = _run_both(order, tA, tB, M, N, K, 0.7, -1.3, 100 + 10 * i)
        assert st0 == 0 and st1 == 0, (name, st0, st1)
        assert d0 == d1, (d0, d1)  # same kernel, tile, K ranges and slices
        used_scratch |= "splits=1 " not in d1 or "tail_slices=1" not in d1
        assert np.array_equal(c0, c1), (name, i, d1)
        assert np.isfinite(c1).all()
    assert used_scratch == (name != "no scratch needed"), name


def test_noalloc_checks_arguments_like_sgemm():
    A = torch.zeros(64, device="cuda")
    assert clblas_amd.sgemm_noalloc(COL, NOTRANS, NOTRANS, 8, 8, 8, 1.0, None, 0, 8, A, 0, 8, 0.0, A, 0, 8) == -1022
    assert clblas_amd.sgemm_noalloc(COL, NOTRANS, NOTRANS, 8, 8, 8, 1.0, A, 0, 7, A, 0, 8, 0.0, A, 0, 8) == -1016
    assert clblas_amd.sgemm_noalloc(COL, NOTRANS, NOTRANS, 0, 8, 8, 1.0, A, 0, 8, A, 0, 8, 0.0, A, 0, 8) == -1017


def test_noalloc_rejects_what_does_not_fit_its_scratch():
    """64 K ranges of a 1024 x 1024 product are 256 MiB of partial sums: more than the fixed
    array holds, so the call is refused (clblasOutOfResources) and C is left alone, while
    clblasSgemm, which may allocate, runs it."""
    M = N = 1024
    K = 16384
    A = torch.from_numpy(oracle.uniform(M * K, 1, np.float32)).cuda()
    B = torch.from_numpy(oracle.uniform(K * N, 2, np.float32)).cuda()
    C = torch.full((M * N,), 3.0, device="cuda")
    with debug_env(CLBLAS_AMD_GEMM_TILE=6, CLBLAS_AMD_GEMM_SPLITS=64):   # the 64x64 tile, last in the FP32 table
        st = clblas_amd.sgemm_noalloc(COL, NOTRANS, NOTRANS, M, N, K, 1.0, A, 0, M, B, 0, K, 0.0, C, 0, M)
        torch.cuda.synchronize()
        assert st == clblas_amd.Status.OutOfResources
        assert bool((C == 3.0).all().item())
        st = clblas_amd.sgemm(COL, NOTRANS, NOTRANS, M, N, K, 1.0, A, 0, M, B, 0, K, 0.0, C, 0, M)
        torch.cuda.synchronize()
        assert st == 0 and "splits=64" in clblas_amd.last_dispatch()[0]
    # afterwards the entry point still works, and still agrees with clblasSgemm
    C2 = torch.empty_like(C)
    assert clblas_amd.sgemm_noalloc(COL, NOTRANS, NOTRANS, M, N, K, 1.0, A, 0, M, B, 0, K, 0.0, C2, 0, M) == 0
    C3 = torch.empty_like(C)
    assert clblas_amd.sgemm(COL, NOTRANS, NOTRANS, M, N, K, 1.0, A, 0, M, B, 0, K, 0.0, C3, 0, M) == 0
    torch.cuda.synchronize()
    assert torch.equal(C2, C3)


def test_noalloc_can_be_the_first_thing_in_a_graph():
    """No warm-up call on the capturing stream: the entry point must not need one."""
    assert clblas_amd.setup() == 0
    M, N, K = 200, 150, 8192
    A = torch.from_numpy(oracle.uniform(M * K, 4, np.float32)).cuda()
    B = torch.from_numpy(oracle.uniform(K * N, 5, np.float32)).cuda()
    C = torch.zeros(M * N, device="cuda")
    want = torch.zeros(M * N, device="cuda")
    assert clblas_amd.sgemm(COL, NOTRANS, NOTRANS, M, N, K, 1.0, A, 0, M, B, 0, K, 0.0, want, 0, M) == 0
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    stats = clblas_amd.workspace_stats()
    with torch.cuda.stream(s):
        with torch.cuda.graph(g, stream=s):
            st = clblas_amd.sgemm_noalloc(COL, NOTRANS, NOTRANS, M, N, K, 1.0, A, 0, M, B, 0, K, 0.0, C, 0, M, stream=s)
    assert st == 0
    assert "splits=1 " not in clblas_amd.last_dispatch()[0] + " ", "the case is meant to use the scratch array"
    assert clblas_amd.workspace_stats() == stats, "the entry point must not touch the per-stream buffers"
    for _ in range(3):
        C.fill_(-1.0)
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(C, want)
