"""Pins the CPU oracle's SYRK / TRMM / SYMM (oracle/level3.inc) for all four types:
exact-integer inputs against exact products over every order / side / triangle / transpose /
diagonal combination with the unused triangle NaN-poisoned, the reference's own naive syrk
and trmm (oracle/_ref), SYMM against GEMM on the symmetrised matrix, TRMM undone by TRSM, and
the argument checks.  CPU only."""
import itertools

import numpy as np
import pytest

import oracle
from helpers import COL, ROW, NOTRANS, TRANS, CONJ, UPPER, LOWER, UNIT, NONUNIT, LEFT, RIGHT, logical_view
from l3_util import (ALL, REAL, abs1, bound, err, is_cplx, matrix, nan_of, op, poison_triangle, real_scalars, scalars,
                     sym_dense, tri_dense, tri_mask)

needs_ref = pytest.mark.skipif(oracle.ref_lib() is None, reason="oracle/_ref not built (no reference tree)")
WIDE = lambda dt: np.complex128 if is_cplx(dt) else np.float64


def syrk_transposes(dtype):
    return [NOTRANS, TRANS] if is_cplx(dtype) else [NOTRANS, TRANS, CONJ]


# ------------------------------------------------------------------------------- SYRK
@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("order,uplo", list(itertools.product([ROW, COL], [UPPER, LOWER])))
def test_syrk_integer_exact(dtype, order, uplo):
    alpha, beta = scalars(dtype)
    for trans in syrk_transposes(dtype):
        for si, (N, K) in enumerate([(1, 1), (5, 3), (17, 33), (64, 20), (70, 129)]):
            rows, cols = (N, K) if trans == NOTRANS else (K, N)
            A, lda = matrix(order, rows, cols, 5, 3, 10 + si, dtype, True)
            C, ldc = matrix(order, N, N, 7, 2, 20 + si, dtype, True)
            keep = tri_mask(N, uplo == LOWER)
            logical_view(C, order, NOTRANS, N, N, 7, ldc)[~keep] = nan_of(dtype)  # must stay untouched
            C0 = C.copy()
            assert oracle.syrk(order, uplo, trans, N, K, alpha, A, 5, lda, beta, C, 7, ldc) == 0
            Av = logical_view(A, order, NOTRANS, rows, cols, 5, lda).astype(WIDE(dtype))
            Aop = Av if trans == NOTRANS else Av.T
            want = alpha * (Aop @ Aop.T) + beta * np.where(keep, logical_view(C0, order, NOTRANS, N, N, 7, ldc), 0)
            got = logical_view(C, order, NOTRANS, N, N, 7, ldc)
            np.testing.assert_array_equal(got[keep].astype(WIDE(dtype)), want[keep])
            # everything outside the stored triangle, padding included, is bit-identical (NaNs too)
            idx = logical_view(np.arange(C.size), order, NOTRANS, N, N, 7, ldc)[keep]
            rest = np.ones(C.size, dtype=bool)
            rest[idx] = False
            np.testing.assert_array_equal(C[rest].view(np.uint8), C0[rest].view(np.uint8))


@pytest.mark.parametrize("dtype", ALL)
def test_syrk_beta_zero_and_checks(dtype):
    N, K = 9, 4
    A, lda = matrix(COL, N, K, 0, 0, 1, dtype, True)
    C = np.full(N * N, nan_of(dtype), dtype=dtype)
    assert oracle.syrk(COL, LOWER, NOTRANS, N, K, 1, A, 0, lda, 0, C, 0, N) == 0
    Cv = C.reshape(N, N, order="F")
    Av = A.reshape(N, K, order="F").astype(WIDE(dtype))
    keep = tri_mask(N, True)
    np.testing.assert_array_equal(Cv[keep].astype(WIDE(dtype)), (Av @ Av.T)[keep])
    assert np.isnan(Cv[~keep].real).all()
    assert oracle.syrk(COL, LOWER, NOTRANS, N, K, 1, None, 0, lda, 0, C, 0, N) == -1022
    assert oracle.syrk(COL, LOWER, NOTRANS, N, K, 1, A, 0, lda, 0, None, 0, N) == -1020
    assert oracle.syrk(COL, LOWER, NOTRANS, N, 0, 1, A, 0, lda, 0, C, 0, N) == -1017
    assert oracle.syrk(COL, LOWER, NOTRANS, N, K, 1, A, 0, N - 1, 0, C, 0, N) == -1016
    assert oracle.syrk(COL, LOWER, TRANS, N, K, 1, A, 0, K - 1, 0, C, 0, N) == -1016
    assert oracle.syrk(COL, LOWER, NOTRANS, N, K, 1, A, 0, lda, 0, C, 0, N - 1) == -1014
    assert oracle.syrk(COL, LOWER, CONJ, N, K, 1, A, 0, K, 0, C, 0, N) == (-30 if is_cplx(dtype) else 0)


@needs_ref
@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("order,uplo,trans", list(itertools.product([ROW, COL], [UPPER, LOWER], [NOTRANS, TRANS])))
def test_syrk_vs_reference_naive(dtype, order, uplo, trans):
    N, K = 37, 45
    rows, cols = (N, K) if trans == NOTRANS else (K, N)
    for integer in (True, False):
        alpha, beta = scalars(dtype) if integer else real_scalars(dtype)
        A, lda = matrix(order, rows, cols, 0, 2, 1, dtype, integer)
        C, ldc = matrix(order, N, N, 0, 1, 2, dtype, integer)
        Cr = C.copy()
        oracle.ref_syrk(order, uplo, trans, N, K, alpha, A, lda, beta, Cr, ldc)
        assert oracle.syrk(order, uplo, trans, N, K, alpha, A, 0, lda, beta, C, 0, ldc) == 0
        if integer:
            np.testing.assert_array_equal(C, Cr)
        else:
            np.testing.assert_allclose(C, Cr, rtol=0, atol=8 * K * np.finfo(dtype).eps * 4)


# ------------------------------------------------------------------------------- TRMM
TRMM_CASES = list(itertools.product([LEFT, RIGHT], [UPPER, LOWER], [NOTRANS, TRANS, CONJ], [UNIT, NONUNIT]))


def trmm_want(order, side, uplo, trans, diag, M, N, alpha, A, offA, lda, B0, offB, ldb):
    n = M if side == LEFT else N
    T = op(tri_dense(A, order, n, offA, lda, uplo, diag == UNIT), trans)
    Bv = logical_view(B0, order, NOTRANS, M, N, offB, ldb).astype(T.dtype)
    return alpha * (T @ Bv if side == LEFT else Bv @ T), T, Bv


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("order", [ROW, COL])
@pytest.mark.parametrize("side,uplo,trans,diag", TRMM_CASES)
def test_trmm_integer_exact(dtype, order, side, uplo, trans, diag):
    alpha, _ = scalars(dtype)
    for si, (M, N) in enumerate([(1, 1), (3, 7), (16, 17), (33, 20), (70, 45)]):
        n = M if side == LEFT else N
        A, lda = matrix(order, n, n, 5, 3, 30 + si, dtype, True, limit=4)
        poison_triangle(A, order, n, 5, lda, uplo, unit=diag == UNIT)
        B, ldb = matrix(order, M, N, 7, 2, 40 + si, dtype, True, limit=4)
        B0 = B.copy()
        assert oracle.trmm(order, side, uplo, trans, diag, M, N, alpha, A, 5, lda, B, 7, ldb) == 0
        want, _, _ = trmm_want(order, side, uplo, trans, diag, M, N, alpha, A, 5, lda, B0, 7, ldb)
        got = logical_view(B, order, NOTRANS, M, N, 7, ldb)
        np.testing.assert_array_equal(got.astype(want.dtype), want)
        idx = logical_view(np.arange(B.size), order, NOTRANS, M, N, 7, ldb).ravel()
        rest = np.ones(B.size, dtype=bool)
        rest[idx] = False
        np.testing.assert_array_equal(B[rest], B0[rest])


@needs_ref
@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("order", [ROW, COL])
@pytest.mark.parametrize("side,uplo,trans,diag", TRMM_CASES)
def test_trmm_vs_reference_naive(dtype, order, side, uplo, trans, diag):
    M, N = 29, 23
    n = M if side == LEFT else N
    for integer in (True, False):
        alpha = scalars(dtype)[0] if integer else real_scalars(dtype)[0]
        A, lda = matrix(order, n, n, 0, 1, 3, dtype, integer, limit=4)
        B, ldb = matrix(order, M, N, 0, 2, 4, dtype, integer, limit=4)
        Br = B.copy()
        oracle.ref_trmm(order, side, uplo, trans, diag, M, N, alpha, A, lda, Br, ldb)
        assert oracle.trmm(order, side, uplo, trans, diag, M, N, alpha, A, 0, lda, B, 0, ldb) == 0
        if integer:
            np.testing.assert_array_equal(B, Br)
        else:
            np.testing.assert_allclose(B, Br, rtol=0, atol=16 * n * np.finfo(dtype).eps)


@pytest.mark.parametrize("dtype", REAL)
@pytest.mark.parametrize("order", [ROW, COL])
@pytest.mark.parametrize("side,uplo,trans,diag", TRMM_CASES)
def test_trmm_is_undone_by_trsm(dtype, order, side, uplo, trans, diag):
    M, N = 40, 27
    n = M if side == LEFT else N
    inner = n  # square: ld = n in both orders
    A = oracle.triangular(n, inner, (uplo == LOWER) == (order == COL), 7, dtype)
    B, ldb = matrix(order, M, N, 0, 0, 8, dtype, False)
    B0 = B.copy()
    assert oracle.trmm(order, side, uplo, trans, diag, M, N, 1.0, A, 0, inner, B, 0, ldb) == 0
    assert oracle.trsm_naive(order, side, uplo, trans, diag, M, N, 1.0, A, 0, inner, B, 0, ldb) == 0
    np.testing.assert_allclose(B, B0, rtol=0, atol=64 * n * np.finfo(dtype).eps)


def test_trmm_checks():
    A = np.ones(16, dtype=np.float64)
    B = np.ones(16, dtype=np.float64)
    assert oracle.trmm(COL, LEFT, UPPER, NOTRANS, NONUNIT, 4, 4, 1.0, None, 0, 4, B, 0, 4) == -1022
    assert oracle.trmm(COL, LEFT, UPPER, NOTRANS, NONUNIT, 4, 4, 1.0, A, 0, 4, None, 0, 4) == -1021
    assert oracle.trmm(COL, LEFT, UPPER, NOTRANS, NONUNIT, 0, 4, 1.0, A, 0, 4, B, 0, 4) == -1017
    assert oracle.trmm(COL, LEFT, UPPER, NOTRANS, NONUNIT, 4, 4, 1.0, A, 0, 3, B, 0, 4) == -1016
    assert oracle.trmm(COL, RIGHT, UPPER, NOTRANS, NONUNIT, 2, 4, 1.0, A, 0, 3, B, 0, 4) == -1016
    assert oracle.trmm(COL, LEFT, UPPER, NOTRANS, NONUNIT, 4, 4, 1.0, A, 0, 4, B, 0, 3) == -1015


# ------------------------------------------------------------------------------- SYMM
@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("order,side,uplo", list(itertools.product([ROW, COL], [LEFT, RIGHT], [UPPER, LOWER])))
def test_symm_integer_exact(dtype, order, side, uplo):
    alpha, beta = scalars(dtype)
    for si, (M, N) in enumerate([(1, 1), (3, 7), (16, 17), (33, 20), (70, 45)]):
        n = M if side == LEFT else N
        A, lda = matrix(order, n, n, 5, 3, 50 + si, dtype, True)
        poison_triangle(A, order, n, 5, lda, uplo)
        B, ldb = matrix(order, M, N, 7, 2, 60 + si, dtype, True)
        C, ldc = matrix(order, M, N, 11, 1, 70 + si, dtype, True)
        C0 = C.copy()
        assert oracle.symm(order, side, uplo, M, N, alpha, A, 5, lda, B, 7, ldb, beta, C, 11, ldc) == 0
        S = sym_dense(A, order, n, 5, lda, uplo)
        Bv = logical_view(B, order, NOTRANS, M, N, 7, ldb).astype(S.dtype)
        want = alpha * (S @ Bv if side == LEFT else Bv @ S) + beta * logical_view(C0, order, NOTRANS, M, N, 11, ldc)
        np.testing.assert_array_equal(logical_view(C, order, NOTRANS, M, N, 11, ldc).astype(S.dtype), want)
        idx = logical_view(np.arange(C.size), order, NOTRANS, M, N, 11, ldc).ravel()
        rest = np.ones(C.size, dtype=bool)
        rest[idx] = False
        np.testing.assert_array_equal(C[rest], C0[rest])


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("order,side,uplo", list(itertools.product([ROW, COL], [LEFT, RIGHT], [UPPER, LOWER])))
def test_symm_equals_gemm_on_symmetrised_matrix(dtype, order, side, uplo):
    """SYMM has no naive statement in the reference; pin it on the (separately pinned) GEMM."""
    M, N = 31, 26
    n = M if side == LEFT else N
    alpha, beta = real_scalars(dtype)
    A, lda = matrix(order, n, n, 0, 0, 5, dtype, False)
    B, ldb = matrix(order, M, N, 0, 2, 6, dtype, False)
    C, ldc = matrix(order, M, N, 0, 1, 7, dtype, False)
    Cg = C.copy()
    full = sym_dense(A, order, n, 0, lda, uplo).astype(dtype)
    Afull = np.ascontiguousarray(full).ravel()  # symmetric: either order reads the same matrix
    poison_triangle(A, order, n, 0, lda, uplo)
    assert oracle.symm(order, side, uplo, M, N, alpha, A, 0, lda, B, 0, ldb, beta, C, 0, ldc) == 0
    if side == LEFT:
        assert oracle.gemm(order, NOTRANS, NOTRANS, M, N, M, alpha, Afull, 0, n, B, 0, ldb, beta, Cg, 0, ldc) == 0
    else:
        assert oracle.gemm(order, NOTRANS, NOTRANS, M, N, N, alpha, B, 0, ldb, Afull, 0, n, beta, Cg, 0, ldc) == 0
    np.testing.assert_allclose(C, Cg, rtol=0, atol=32 * n * np.finfo(dtype).eps)
    # beta == 0 never reads C
    Cn = np.full(C.size, nan_of(dtype), dtype=dtype)
    assert oracle.symm(order, side, uplo, M, N, alpha, A, 0, lda, B, 0, ldb, 0, Cn, 0, ldc) == 0
    assert np.isfinite(logical_view(Cn, order, NOTRANS, M, N, 0, ldc).real).all()


def test_symm_checks():
    A = np.ones(16, dtype=np.float32)
    assert oracle.symm(COL, LEFT, UPPER, 4, 4, 1.0, None, 0, 4, A, 0, 4, 0.0, A, 0, 4) == -1022
    assert oracle.symm(COL, LEFT, UPPER, 4, 4, 1.0, A, 0, 4, None, 0, 4, 0.0, A, 0, 4) == -1021
    assert oracle.symm(COL, LEFT, UPPER, 4, 4, 1.0, A, 0, 4, A, 0, 4, 0.0, None, 0, 4) == -1020
    assert oracle.symm(COL, LEFT, UPPER, 4, 0, 1.0, A, 0, 4, A, 0, 4, 0.0, A, 0, 4) == -1017
    assert oracle.symm(COL, LEFT, UPPER, 4, 4, 1.0, A, 0, 3, A, 0, 4, 0.0, A, 0, 4) == -1016
    assert oracle.symm(COL, RIGHT, UPPER, 2, 4, 1.0, A, 0, 3, A, 0, 4, 0.0, A, 0, 4) == -1016
    assert oracle.symm(COL, LEFT, UPPER, 4, 4, 1.0, A, 0, 4, A, 0, 3, 0.0, A, 0, 4) == -1015
    assert oracle.symm(COL, LEFT, UPPER, 4, 4, 1.0, A, 0, 4, A, 0, 4, 0.0, A, 0, 3) == -1014


# ------------------------------------------------------------------------------- golden fixtures
def _run_golden(mod_syrk, mod_trmm, mod_symm, c):
    """Runs one fixed case (inputs from the reference's sample programs, expected values in
    exact arithmetic) through the given routines; returns (status, result buffer)."""
    dt = np.float32
    A = np.array(c["A"], dtype=dt)
    if c["kind"] == "syrk":
        C = np.array(c["C"], dtype=dt)
        return mod_syrk(c["order"], c["uplo"], c["transA"], c["N"], c["K"], c["alpha"], A, c["offA"], c["lda"],
                        c["beta"], C, c["offC"], c["ldc"]), C
    if c["kind"] == "trmm":
        B = np.array(c["B"], dtype=dt)
        return mod_trmm(c["order"], c["side"], c["uplo"], c["transA"], c["diag"], c["M"], c["N"], c["alpha"], A,
                        c["offA"], c["lda"], B, c["offB"], c["ldb"]), B
    B, C = np.array(c["B"], dtype=dt), np.array(c["C"], dtype=dt)
    return mod_symm(c["order"], c["side"], c["uplo"], c["M"], c["N"], c["alpha"], A, c["offA"], c["lda"], B, c["offB"],
                    c["ldb"], c["beta"], C, c["offC"], c["ldc"]), C


@pytest.mark.parametrize("name", ["sample_ssymm", "sample_ssyrk_offsets", "sample_strmm_offsets"])
def test_level3_golden(name):
    """Fixed inputs of src/samples/example_ssymm.c, example_ssyrk.c, example_strmm.c (integers:
    the results are exact)."""
    from helpers import golden_cases
    c = golden_cases()[name]
    st, out = _run_golden(oracle.syrk, oracle.trmm, oracle.symm, c)
    assert st == 0
    np.testing.assert_array_equal(out, np.array(c["expected"], dtype=np.float32))
