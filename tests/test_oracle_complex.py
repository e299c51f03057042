"""Pins the complex GEMM of the CPU oracle (oracle_cgemm / oracle_zgemm and their
high-precision yardsticks): Gaussian-integer inputs against exact integer arithmetic for every
order x transpose x conjugate combination (the reference tests' exact-integer method,
src/tests/include/blas-random.h:60-93, applied to complex data), closed forms, conjugation and
layout identities, and the reference's own naive complex gemm (oracle/_ref).  CPU only."""
import itertools

import numpy as np
import pytest

import oracle
from helpers import COL, ROW, NOTRANS, TRANS, CONJ, cgemm_bound, logical_view, mem_dims

CDT = [np.complex64, np.complex128]
ALL_T = [NOTRANS, TRANS, CONJ]
SHAPES = [(1, 1, 1), (2, 1, 3), (8, 16, 17), (17, 32, 62), (64, 33, 128), (65, 67, 5)]


def op_view(buf, order, trans, rows, cols, off, ld):
    v = logical_view(buf, order, trans, rows, cols, off, ld)
    return np.conj(v) if trans == CONJ else v


def layout(order, tA, tB, M, N, K, pad, offs):
    ia, oa = mem_dims(order, tA, M, K)
    ib, ob = mem_dims(order, tB, K, N)
    ic, oc = mem_dims(order, NOTRANS, M, N)
    lda, ldb, ldc = ia + pad, ib + pad, ic + pad
    return lda, ldb, ldc, offs[0] + oa * lda, offs[1] + ob * ldb, offs[2] + oc * ldc


@pytest.mark.parametrize("dtype", CDT)
@pytest.mark.parametrize("order", [ROW, COL])
@pytest.mark.parametrize("tA,tB", list(itertools.product(ALL_T, ALL_T)))
def test_cgemm_gaussian_integer_exact(dtype, order, tA, tB):
    alpha, beta = 2 - 1j, -1 + 2j
    for si, (M, N, K) in enumerate(SHAPES):
        offs = (5, 7, 11)
        lda, ldb, ldc, na, nb, nc = layout(order, tA, tB, M, N, K, 3, offs)
        # |parts| <= 8: every partial sum stays far below 2^23, so any order of the mads is exact
        A = oracle.integers(na, 100 + si, 8, dtype)
        B = oracle.integers(nb, 200 + si, 8, dtype)
        C = oracle.integers(nc, 300 + si, 8, dtype)
        C0 = C.copy()
        assert oracle.gemm(order, tA, tB, M, N, K, alpha, A, offs[0], lda, B, offs[1], ldb, beta, C, offs[2], ldc) == 0
        Av = op_view(A, order, tA, M, K, offs[0], lda).astype(np.complex128)
        Bv = op_view(B, order, tB, K, N, offs[1], ldb).astype(np.complex128)
        Cv0 = logical_view(C0, order, NOTRANS, M, N, offs[2], ldc).astype(np.complex128)
        want = alpha * (Av @ Bv) + beta * Cv0  # small integers: exact in float64
        got = logical_view(C, order, NOTRANS, M, N, offs[2], ldc)
        np.testing.assert_array_equal(got.astype(np.complex128), want)
        mask = np.ones(C.size, dtype=bool)
        mask[logical_view(np.arange(C.size), order, NOTRANS, M, N, offs[2], ldc).ravel()] = False
        np.testing.assert_array_equal(C[mask], C0[mask])
        if order == COL:
            rows, cols = np.meshgrid(np.arange(M), np.arange(N), indexing="ij")
            ex, mag = oracle.gemm_exact(tA, tB, K, alpha, A[offs[0]:], lda, B[offs[1]:], ldb, beta, C0[offs[2]:], ldc,
                                        rows.ravel(), cols.ravel())
            np.testing.assert_array_equal(ex.reshape(M, N), want)
            assert np.all(mag.reshape(M, N) >= np.maximum(np.abs(want.real), np.abs(want.imag)))


@pytest.mark.parametrize("dtype", CDT)
def test_cgemm_closed_forms(dtype):
    n = 29
    X = oracle.uniform(n * n, 1, dtype)
    I = np.eye(n, dtype=dtype).ravel(order="F").copy()
    iI = (1j * np.eye(n)).astype(dtype).ravel(order="F").copy()
    # (iI)(iI) = -I, exactly
    C = np.full(n * n, np.nan + 1j * np.nan, dtype=dtype)
    assert oracle.gemm(COL, NOTRANS, NOTRANS, n, n, n, 1, iI, 0, n, iI, 0, n, 0, C, 0, n) == 0
    np.testing.assert_array_equal(C, -I)
    # X * I, beta = 0 with NaN-filled C: C is never read, result is X bit for bit
    C = np.full(n * n, np.nan + 1j * np.nan, dtype=dtype)
    assert oracle.gemm(COL, NOTRANS, NOTRANS, n, n, n, 1, X, 0, n, I, 0, n, 0, C, 0, n) == 0
    np.testing.assert_array_equal(C, X)
    # alpha = i rotates: i * X exactly (re' = -im, im' = re)
    C = np.zeros(n * n, dtype=dtype)
    assert oracle.gemm(COL, NOTRANS, NOTRANS, n, n, n, 1j, X, 0, n, I, 0, n, 0, C, 0, n) == 0
    np.testing.assert_array_equal(C.real, -X.imag)
    np.testing.assert_array_equal(C.imag, X.real)
    # alpha = 0, beta = i: C <- i * C exactly; beta = 1: unchanged
    C = X.copy()
    assert oracle.gemm(COL, TRANS, CONJ, n, n, n, 0, X, 0, n, X, 0, n, 1j, C, 0, n) == 0
    np.testing.assert_array_equal(C.real, -X.imag)
    np.testing.assert_array_equal(C.imag, X.real)
    C = X.copy()
    assert oracle.gemm(COL, NOTRANS, NOTRANS, n, n, n, 0, X, 0, n, X, 0, n, 1, C, 0, n) == 0
    np.testing.assert_array_equal(C, X)
    # X^H X is Hermitian with a real, non-negative diagonal
    C = np.zeros(n * n, dtype=dtype)
    assert oracle.gemm(COL, CONJ, NOTRANS, n, n, n, 1, X, 0, n, X, 0, n, 0, C, 0, n) == 0
    G = C.reshape(n, n, order="F")
    eps = np.finfo(dtype).eps
    assert np.all(np.abs(np.diag(G).imag) <= 2 * n * eps) and np.all(np.diag(G).real > 0)
    assert np.all(np.abs(G - G.conj().T) <= 4 * n * eps * n)
    # a real beta with zero imaginary part but nonzero real part still reads C
    C = np.full(n * n, np.nan, dtype=dtype)
    assert oracle.gemm(COL, NOTRANS, NOTRANS, n, n, n, 1, X, 0, n, I, 0, n, 1e-30, C, 0, n) == 0
    assert np.isnan(C.real).all()
    C = np.full(n * n, np.nan, dtype=dtype)
    assert oracle.gemm(COL, NOTRANS, NOTRANS, n, n, n, 1, X, 0, n, I, 0, n, 1e-30j, C, 0, n) == 0
    assert np.isnan(C.real).all()


@pytest.mark.parametrize("dtype", CDT)
def test_cgemm_conjugation_and_layout_identities(dtype):
    M, N, K = 23, 19, 31
    A = oracle.uniform(M * K, 3, dtype).reshape(M, K)
    B = oracle.uniform(K * N, 4, dtype).reshape(K, N)
    C0 = oracle.uniform(M * N, 5, dtype).reshape(M, N)
    alpha, beta = 0.7 - 0.2j, -1.3 + 0.4j
    results = []
    for order, tA, tB in itertools.product([ROW, COL], ALL_T, ALL_T):
        # store whatever makes op(stored) == A, resp. B
        a = A if tA == NOTRANS else (A.T if tA == TRANS else A.conj().T)
        b = B if tB == NOTRANS else (B.T if tB == TRANS else B.conj().T)
        lay = "C" if order == ROW else "F"
        abuf, bbuf, cbuf = (x.ravel(order=lay).copy() for x in (a, b, C0))
        lda = a.shape[1] if order == ROW else a.shape[0]
        ldb = b.shape[1] if order == ROW else b.shape[0]
        ldc = N if order == ROW else M
        assert oracle.gemm(order, tA, tB, M, N, K, alpha, abuf, 0, lda, bbuf, 0, ldb, beta, cbuf, 0, ldc) == 0
        results.append(cbuf.reshape(M, N, order=lay))
    # the same logical product with the same k order (negation is exact): identical bits within
    # one order.  Row-major calls run with the operands swapped (xgemm.cc:40-61), which swaps the
    # two mads of the imaginary part of the accumulator, so across orders the bits may differ.
    per_order = len(results) // 2
    for r in results[1:per_order]:
        np.testing.assert_array_equal(r, results[0])
    for r in results[per_order + 1:]:
        np.testing.assert_array_equal(r, results[per_order])
    col_major = results[per_order]
    assert np.all(np.abs(results[0] - col_major) <= 8 * K * np.finfo(dtype).eps)
    results[0] = col_major
    # conj(alpha A B + beta C) == conj(alpha) conj(A) conj(B) + conj(beta) conj(C), bit for bit
    abuf, bbuf, cbuf = (np.conj(x).ravel(order="F").copy() for x in (A, B, C0))
    assert oracle.gemm(COL, NOTRANS, NOTRANS, M, N, K, np.conj(alpha), abuf, 0, M, bbuf, 0, K, np.conj(beta), cbuf, 0,
                       M) == 0
    np.testing.assert_array_equal(np.conj(cbuf.reshape(M, N, order="F")), results[0])
    A1, B1, C1 = (x.astype(np.complex128) for x in (A, B, C0))
    want = alpha * (A1 @ B1) + beta * C1
    mag = (abs(alpha.real) + abs(alpha.imag)) * ((np.abs(A1.real) + np.abs(A1.imag)) @ (np.abs(B1.real) + np.abs(B1.imag))) \
        + (abs(beta.real) + abs(beta.imag)) * (np.abs(C1.real) + np.abs(C1.imag))
    err = np.maximum(np.abs(results[0].real - want.real), np.abs(results[0].imag - want.imag))
    assert np.all(err <= cgemm_bound(K, mag, dtype, c=1.0))
    # the yardstick agrees with numpy's complex128 product
    rows, cols = np.meshgrid(np.arange(M), np.arange(N), indexing="ij")
    ex, mg = oracle.gemm_exact(NOTRANS, NOTRANS, K, alpha, A.ravel(order="F").copy(), M, B.ravel(order="F").copy(), K,
                               beta, C0.ravel(order="F").copy(), M, rows.ravel(), cols.ravel())
    al, be = complex(dtype(alpha)), complex(dtype(beta))  # the routines see alpha / beta rounded to the working precision
    want = al * (A1 @ B1) + be * C1
    assert np.all(np.abs(ex.reshape(M, N) - want) <= 1e-13 * mag)
    np.testing.assert_allclose(mg.reshape(M, N), (abs(al.real) + abs(al.imag)) * (
        (np.abs(A1.real) + np.abs(A1.imag)) @ (np.abs(B1.real) + np.abs(B1.imag))) + (abs(be.real) + abs(be.imag)) * (
        np.abs(C1.real) + np.abs(C1.imag)), rtol=1e-12)


needs_ref = pytest.mark.skipif(oracle.ref_lib() is None, reason="oracle/_ref not built (no reference tree)")


@needs_ref
@pytest.mark.parametrize("dtype", CDT)
@pytest.mark.parametrize("order", [ROW, COL])
@pytest.mark.parametrize("tA,tB", list(itertools.product(ALL_T, ALL_T)))
def test_cgemm_vs_reference_naive(dtype, order, tA, tB):
    M, N, K = 45, 37, 53
    lda, ldb, ldc, na, nb, nc = layout(order, tA, tB, M, N, K, 2, (0, 0, 0))
    for exact in (True, False):
        if exact:
            A, B, C = oracle.integers(na, 1, 8, dtype), oracle.integers(nb, 2, 8, dtype), oracle.integers(nc, 3, 8, dtype)
            alpha, beta = 2 + 1j, 3 - 2j
        else:
            A, B, C = oracle.uniform(na, 1, dtype), oracle.uniform(nb, 2, dtype), oracle.uniform(nc, 3, dtype)
            alpha, beta = 0.7 + 0.1j, -1.3 + 0.6j
        C0 = C.copy()
        Cr = C.copy()
        oracle.ref_gemm(order, tA, tB, M, N, K, alpha, A, lda, B, ldb, beta, Cr, ldc)
        assert oracle.gemm(order, tA, tB, M, N, K, alpha, A, 0, lda, B, 0, ldb, beta, C, 0, ldc) == 0
        if exact:
            np.testing.assert_array_equal(C, Cr)
        else:
            Av = op_view(A, order, tA, M, K, 0, lda).astype(np.complex128)
            Bv = op_view(B, order, tB, K, N, 0, ldb).astype(np.complex128)
            Cv = logical_view(C0, order, NOTRANS, M, N, 0, ldc).astype(np.complex128)
            mag = (abs(alpha.real) + abs(alpha.imag)) * (
                (np.abs(Av.real) + np.abs(Av.imag)) @ (np.abs(Bv.real) + np.abs(Bv.imag))) + (
                abs(beta.real) + abs(beta.imag)) * (np.abs(Cv.real) + np.abs(Cv.imag))
            got = logical_view(C, order, NOTRANS, M, N, 0, ldc).astype(np.complex128)
            ref = logical_view(Cr, order, NOTRANS, M, N, 0, ldc).astype(np.complex128)
            err = np.maximum(np.abs(got.real - ref.real), np.abs(got.imag - ref.imag))
            assert np.all(err <= cgemm_bound(K, mag, dtype))
