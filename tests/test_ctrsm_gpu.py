"""GPU parity tests for clblasCtrsm / clblasZtrsm through the C ABI: the reference sample's fixed
input, and every order / side / triangle / transpose (incl. conjugate) / diagonal combination
against the oracle's naive complex solver on the same seeded inputs - normwise backward error
<= 2 n eps and agreement with the oracle within 32 n eps * max|X| (same bars as the real routines)."""
import itertools

import numpy as np
import pytest

import oracle
from helpers import COL, ROW, NOTRANS, TRANS, CONJ, UPPER, LOWER, UNIT, NONUNIT, LEFT, RIGHT, golden_cases, logical_view
from l3_util import CPLX, ctrsm_inputs, trsm_backward_error

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    import gpu_util
    import torch
    assert torch.cuda.is_available()
    return gpu_util


def test_sample_ctrsm(gpu):
    c = golden_cases()["sample_ctrsm_offsets"]
    A, B = np.array(c["A"], dtype=np.complex64), np.array(c["B"], dtype=np.complex64)
    st, out = gpu.trsm(c["order"], c["side"], c["uplo"], c["transA"], c["diag"], c["M"], c["N"], c["alpha"], A,
                       c["offA"], c["lda"], B, c["offB"], c["ldb"])
    assert st == 0
    tol = 16 * np.finfo(np.float32).eps
    np.testing.assert_allclose(out.real.astype(np.float64), np.array(c["expected"]), rtol=tol, atol=tol)
    np.testing.assert_allclose(out.imag.astype(np.float64), 0, atol=tol)


VARIANTS = list(itertools.product([LEFT, RIGHT], [UPPER, LOWER], [NOTRANS, TRANS, CONJ], [UNIT, NONUNIT]))
SIZES = [(1, 1), (5, 3), (37, 29), (130, 17), (23, 300), (257, 64), (300, 520), (513, 40), (48, 1030)]


@pytest.mark.parametrize("dtype", CPLX)
@pytest.mark.parametrize("order", [ROW, COL])
@pytest.mark.parametrize("side,uplo,tA,diag", VARIANTS)
def test_all_variants(gpu, dtype, order, side, uplo, tA, diag):
    eps = np.finfo(dtype).eps
    alpha = 0.75 - 0.5j
    for (M, N) in SIZES:
        A, lda, B, ldb = ctrsm_inputs(order, side, uplo, diag, M, N, dtype, 11)
        want = B.copy()
        assert oracle.trsm_naive(order, side, uplo, tA, diag, M, N, alpha, A, 5, lda, want, 7, ldb) == 0
        st, got = gpu.trsm(order, side, uplo, tA, diag, M, N, alpha, A, 5, lda, B, 7, ldb)
        assert st == 0
        n = M if side == LEFT else N
        Xg = logical_view(got, order, NOTRANS, M, N, 7, ldb)
        assert not np.isnan(Xg).any(), "poisoned triangle or unit diagonal was read (%d,%d)" % (M, N)
        be = trsm_backward_error(order, side, uplo, tA, diag, M, N, alpha, A, 5, lda, B, got, 7, ldb)
        assert be <= 2 * n * eps, ((M, N), be)
        Xw = logical_view(want, order, NOTRANS, M, N, 7, ldb)
        assert np.abs(Xg - Xw).max() <= 32 * n * eps * np.abs(Xw).max(), (M, N)
        mask = np.ones(B.size, dtype=bool)
        logical_view(mask, order, NOTRANS, M, N, 7, ldb)[:] = False
        np.testing.assert_array_equal(got[mask].view(np.uint8), B[mask].view(np.uint8))


@pytest.mark.parametrize("dtype", CPLX)
def test_trmm_then_trsm_round_trip_2048(gpu, dtype):
    """Size-independent property at a size the CPU oracle does not reach: B -> op(A) B -> solve
    returns B (left, lower, conjugate transpose)."""
    import torch
    import clblas_amd
    n = 2048
    real = np.float32 if dtype == np.complex64 else np.float64
    A, lda, B, ldb = ctrsm_inputs(COL, LEFT, LOWER, NONUNIT, n, n, dtype, 21, offA=0, offB=0)
    dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    pre = "C" if dtype == np.complex64 else "Z"
    trsm = clblas_amd.ctrsm if dtype == np.complex64 else clblas_amd.ztrsm
    assert clblas_amd.trmm(pre, COL, LEFT, LOWER, CONJ, NONUNIT, n, n, 1.0, dA, 0, lda, dB, 0, ldb) == 0
    assert trsm(COL, LEFT, LOWER, CONJ, NONUNIT, n, n, 1.0, dA, 0, lda, dB, 0, ldb) == 0
    torch.cuda.synchronize()
    got = logical_view(dB.cpu().numpy(), COL, NOTRANS, n, n, 0, ldb)
    ref = logical_view(B, COL, NOTRANS, n, n, 0, ldb)
    assert np.abs(got - ref).max() <= 64 * n * np.finfo(real).eps * np.abs(ref).max()
