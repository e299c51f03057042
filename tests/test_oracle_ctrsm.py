"""Pins the oracle's complex TRSM (oracle_{c,z}trsm_naive) on the CPU: the reference sample's fixed
input (src/samples/example_ctrsm.c) against its exact solution, the reference's own naive
trsm<FloatComplex/DoubleComplex> (src/library/tools/ktest/naive/naive_blas.cpp:632-684, built into
oracle/_ref), and the defining equation op(A) X = alpha B evaluated independently with numpy for
every order / side / triangle / transpose / diagonal combination."""
import itertools

import numpy as np
import pytest

import oracle
from helpers import COL, ROW, NOTRANS, TRANS, CONJ, UPPER, LOWER, UNIT, NONUNIT, LEFT, RIGHT, golden_cases, logical_view
from l3_util import CPLX, ctrsm_inputs, trsm_backward_error

VARIANTS = list(itertools.product([ROW, COL], [LEFT, RIGHT], [UPPER, LOWER], [NOTRANS, TRANS, CONJ], [UNIT, NONUNIT]))


def test_sample_ctrsm_exact():
    c = golden_cases()["sample_ctrsm_offsets"]
    A, B = np.array(c["A"], dtype=np.complex64), np.array(c["B"], dtype=np.complex64)
    st = oracle.trsm_naive(c["order"], c["side"], c["uplo"], c["transA"], c["diag"], c["M"], c["N"], c["alpha"], A,
                           c["offA"], c["lda"], B, c["offB"], c["ldb"])
    assert st == 0
    tol = 16 * np.finfo(np.float32).eps  # as for the STRSM sample
    np.testing.assert_allclose(B.real.astype(np.float64), np.array(c["expected"]), rtol=tol, atol=tol)
    assert (B.imag == 0).all()


@pytest.mark.parametrize("dtype", CPLX)
@pytest.mark.parametrize("order,side,uplo,tA,diag", VARIANTS)
def test_against_reference_naive_and_definition(dtype, order, side, uplo, tA, diag):
    eps = np.finfo(dtype).eps
    alpha = 0.75 - 0.5j
    for (M, N) in [(1, 1), (7, 4), (33, 18), (20, 41)]:
        A, lda, B, ldb = ctrsm_inputs(order, side, uplo, diag, M, N, dtype, 5)
        X = B.copy()
        assert oracle.trsm_naive(order, side, uplo, tA, diag, M, N, alpha, A, 5, lda, X, 7, ldb) == 0
        Xv = logical_view(X, order, NOTRANS, M, N, 7, ldb)
        assert not np.isnan(Xv).any(), "poisoned triangle or unit diagonal was read"
        n = M if side == LEFT else N
        # the defining equation, evaluated independently (numpy, complex128)
        be = trsm_backward_error(order, side, uplo, tA, diag, M, N, alpha, A, 5, lda, B, X, 7, ldb)
        assert be <= 2 * n * eps, ((M, N), be)
        # the reference's own naive routine: same operations in the same order (only the
        # compiler's fused multiply-adds may differ)
        Xr = B[7:].copy()
        oracle.ref_trsm(order, side, uplo, tA, diag, M, N, alpha, A[5:].copy(), lda, Xr, ldb)
        Xrv = logical_view(Xr, order, NOTRANS, M, N, 0, ldb)
        assert np.abs(Xv - Xrv).max() <= 8 * n * eps * np.abs(Xrv).max(), (M, N)
        # nothing outside the M x N block is written
        mask = np.ones(B.size, dtype=bool)
        logical_view(mask, order, NOTRANS, M, N, 7, ldb)[:] = False
        np.testing.assert_array_equal(X[mask].view(np.uint8), B[mask].view(np.uint8))


@pytest.mark.parametrize("dtype", CPLX)
def test_conjugation_identity(dtype):
    """Solving with A^H equals conj(solving conj(B) with A^T and conj(alpha)): conj(A^T x) = A^H conj(x)."""
    M, N = 19, 6
    A, lda, B, ldb = ctrsm_inputs(COL, LEFT, LOWER, NONUNIT, M, N, dtype, 9)
    alpha = 1.25 + 0.5j
    X1 = B.copy()
    assert oracle.trsm_naive(COL, LEFT, LOWER, CONJ, NONUNIT, M, N, alpha, A, 5, lda, X1, 7, ldb) == 0
    X2 = B.conj().copy()
    Ac = A.conj().copy()
    assert oracle.trsm_naive(COL, LEFT, LOWER, CONJ, NONUNIT, M, N, np.conj(alpha), Ac, 5, lda, X2, 7, ldb) == 0
    X3 = B.copy()
    assert oracle.trsm_naive(COL, LEFT, LOWER, TRANS, NONUNIT, M, N, alpha, Ac, 5, lda, X3, 7, ldb) == 0
    v = lambda Z: logical_view(Z, COL, NOTRANS, M, N, 7, ldb)
    np.testing.assert_array_equal(v(X1), v(X3))          # A^H == (conj A)^T, bit for bit
    np.testing.assert_array_equal(v(X2), v(X1).conj())   # conjugating everything conjugates the answer


def test_validation_is_the_real_one():
    A = np.zeros(64, dtype=np.complex64)
    B = np.zeros(64, dtype=np.complex64)
    assert oracle.trsm_naive(COL, LEFT, UPPER, NOTRANS, NONUNIT, 8, 8, 1.0, None, 0, 8, B, 0, 8) == -1022
    assert oracle.trsm_naive(COL, LEFT, UPPER, NOTRANS, NONUNIT, 8, 8, 1.0, A, 0, 8, None, 0, 8) == -1021
    assert oracle.trsm_naive(COL, LEFT, UPPER, NOTRANS, NONUNIT, 8, 8, 1.0, A, 0, 7, B, 0, 8) == \
        oracle.check_trsm(COL, LEFT, NOTRANS, 8, 8, 1, 0, 7, 0, 1, 0, 8, 0)
