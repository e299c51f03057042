"""The substitution leaf of TRSM synchronises its wavefronts through flags in LDS, and a wait for a flag
is bounded so that a mistake in the library cannot hang the GPU; a wait that gives up is counted on
the device (clblasAmdTrsmPollTimeouts).  This file is named to be collected near the end of the GPU
tests: when the whole suite runs in one process the first assertion covers every TRSM call the earlier
files made (the reference's own test family, all variants, the 8192 configuration)."""
import numpy as np
import pytest

from helpers import COL, NOTRANS, LOWER, NONUNIT, LEFT, RIGHT

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    import gpu_util
    import torch
    assert torch.cuda.is_available()
    return gpu_util


def test_flag_waits_never_reach_their_poll_limit(gpu):
    """No wait has given up in anything this process ran before, nor in one solve per type with every kind
    of leaf (16 and 32 right-hand sides per workgroup, both sides, short last blocks).  With the bound
    forced down to a single poll a solve does give up - the counter counts - and every kernel still ends."""
    import torch
    import clblas_amd
    import oracle
    assert clblas_amd.setup() == 0
    assert clblas_amd.trsm_poll_timeouts() == 0, "a flag wait of an earlier TRSM call in this process gave up"
    for dtype, fn, alpha in ((np.float32, clblas_amd.strsm, 1.0), (np.float64, clblas_amd.dtrsm, 1.0),
                             (np.complex64, clblas_amd.ctrsm, 1.0), (np.complex128, clblas_amd.ztrsm, 1.0)):
        real = np.float32 if dtype in (np.float32, np.complex64) else np.float64
        for side, M, N in ((LEFT, 700, 4200), (RIGHT, 300, 600), (LEFT, 1100, 48)):
            n = M if side == LEFT else N
            A = oracle.triangular(n, n, True, 31, real).astype(dtype)
            B = oracle.uniform(M * N, 32, dtype)
            dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
            assert fn(COL, side, LOWER, NOTRANS, NONUNIT, M, N, alpha, dA, 0, n, dB, 0, M) == 0
            torch.cuda.synchronize()
            assert bool(torch.isfinite(torch.view_as_real(dB) if dB.is_complex() else dB).all())
    assert clblas_amd.trsm_poll_timeouts() == 0
    # forced: one poll per wait (complex types always use the substitution leaf)
    n, N = 256, 64
    A = oracle.triangular(n, n, True, 33, np.float64).astype(np.complex128)
    B = oracle.uniform(n * N, 34, np.complex128)
    dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    with gpu.debug_env(CLBLAS_AMD_TRSM_POLL_LIMIT=1):
        assert clblas_amd.ztrsm(COL, LEFT, LOWER, NOTRANS, NONUNIT, n, N, 1.0, dA, 0, n, dB, 0, n) == 0
        torch.cuda.synchronize()
    assert clblas_amd.trsm_poll_timeouts(reset=True) > 0
    assert clblas_amd.trsm_poll_timeouts() == 0
