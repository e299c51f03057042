"""Pins the restatement of the reference's TRSM test family (oracle/trsm_reftest.inc,
tests/helpers.trsm_ref_delta): what src/tests/include/blas-random.h:205-372 fixes about the
generated matrices, the long double solver against exact rational solutions, numpy and the
reference's own naive trsm, and the vectorised bound against the reference's loops."""
import itertools
from fractions import Fraction

import numpy as np
import pytest

import oracle
from helpers import (COL, ROW, NOTRANS, TRANS, CONJ, LEFT, RIGHT, UPPER, LOWER, UNIT, NONUNIT, logical_view,
                     trsm_ref_delta, trsm_ref_delta_loops)

TYPES = [np.float32, np.float64, np.complex64, np.complex128]


def _views(dtype, order, side, M, N, A, offA, lda, B, offB, ldb):
    n = M if side == LEFT else N
    return (logical_view(A, order, NOTRANS, n, n, offA, lda), logical_view(B, order, NOTRANS, M, N, offB, ldb))


@pytest.mark.parametrize("dtype", TYPES)
def test_generated_family_has_the_reference_properties(dtype):
    dtype = np.dtype(dtype)
    cplx = dtype.kind == "c"
    lim_a = 128.0 if dtype in (np.dtype(np.float32), np.dtype(np.complex64)) else 32.0
    lim_b = 2.0 ** 16 if lim_a == 128.0 else 2.0 ** 47
    mod = np.abs
    for order, side, uplo, diag in itertools.product([ROW, COL], [LEFT, RIGHT], [UPPER, LOWER], [UNIT, NONUNIT]):
        M, N = 150, 70
        n = M if side == LEFT else N
        offA, offB, lda = 3, 5, n + 4
        ldb = (M if order == COL else N) + 2
        A, B = oracle.trsm_ref_inputs(dtype, order, side, uplo, diag, M, N, 1.0, offA, lda, offB, ldb, 77)
        Av, Bv = _views(dtype, order, side, M, N, A, offA, lda, B, offB, ldb)
        used = np.tril(np.ones((n, n), bool), -1) if uplo == LOWER else np.triu(np.ones((n, n), bool), 1)
        # NaN wherever the routine must not read (blas-random.h:289-293, 343-348), padding included
        assert np.isnan(Av[~used & ~np.eye(n, dtype=bool)]).all()
        assert np.isnan(A[:offA]).all() and np.isnan(B[:offB]).all()
        d = np.diagonal(Av)
        assert np.isnan(d).all() if diag == UNIT else np.isfinite(d).all()
        off = Av[used]
        assert np.isfinite(off).all() and np.isfinite(Bv).all()
        # integer entries (random<T>(limit) = +-(r % limit))
        assert (off.real == np.round(off.real)).all() and (off.imag == np.round(off.imag)).all()
        assert (Bv.real == np.round(Bv.real)).all()
        if diag == UNIT:
            assert (off == 0).all()  # budget 1: limit sum/sqrt(n-j) <= 1, and r % 1 == 0
            dmod = np.ones(n)
        else:
            dmod = mod(d)
            mx = dmod[0]
            comp = np.sqrt(2.0) if cplx else 1.0
            assert 1.0 <= mx < lim_a * comp
            assert (dmod >= mx / 100 * 0.999).all() and (dmod < mx * comp * 1.0001).all()
            # the budget rule row by row (:264-287): entry j bounded by what is left / sqrt(n - j)
            saw_nonzero = False
            for r in range(n):
                left = dmod[r]
                cols = range(r) if uplo == LOWER else range(r + 1, n)
                for j in cols:
                    x = Av[r, j]
                    if left >= 1.0:
                        lim = left / np.sqrt(n - j)
                        assert abs(x.real) < max(lim, 1) and abs(x.imag) < max(lim, 1)
                        left -= mod(x)
                    else:
                        assert x == 0
                    saw_nonzero |= x != 0
            assert saw_nonzero
        # right-hand sides (:297-341): |y| < sum * |a_pp| / sqrt(len - p) with sum <= TRSM_LIMIT_B
        along = Bv if side == LEFT else Bv.T    # (len, nrhs)
        ln = along.shape[0]
        bound = lim_b * dmod / np.sqrt(ln - np.arange(ln))
        assert (np.abs(along.real) <= bound[:, None]).all()
        assert np.abs(along).max() > 100


def test_alpha_divides_the_right_hand_sides():
    A1, B1 = oracle.trsm_ref_inputs(np.float64, COL, LEFT, LOWER, NONUNIT, 40, 30, 1.0, 0, 40, 0, 40, 5)
    A2, B2 = oracle.trsm_ref_inputs(np.float64, COL, LEFT, LOWER, NONUNIT, 40, 30, 4.0, 0, 40, 0, 40, 5)
    assert np.array_equal(np.nan_to_num(A1), np.nan_to_num(A2)) and np.array_equal(B1 / 4.0, B2)
    A3, B3 = oracle.trsm_ref_inputs(np.complex128, COL, RIGHT, UPPER, NONUNIT, 40, 30, 2 - 1j, 0, 30, 0, 40, 5)
    A4, B4 = oracle.trsm_ref_inputs(np.complex128, COL, RIGHT, UPPER, NONUNIT, 40, 30, 1.0, 0, 30, 0, 40, 5)
    assert np.allclose(B3 * (2 - 1j), B4, rtol=1e-15)


def _exact_solve(E, rhs):
    """Substitution in rational arithmetic; E lower or upper triangular (list of lists of Fraction pairs)."""
    n = len(E)
    lower = all(E[i][j] == 0 for i in range(n) for j in range(i + 1, n))
    x = [None] * n
    for s in range(n):
        i = s if lower else n - 1 - s
        acc = rhs[i]
        for t in range(s):
            k = t if lower else n - 1 - t
            acc = acc - E[i][k] * x[k]
        x[i] = acc / E[i][i]
    return x


class _CFrac:
    """Complex number with rational parts."""
    def __init__(self, re, im=0):
        self.re, self.im = Fraction(re), Fraction(im)
    def __mul__(self, o): return _CFrac(self.re * o.re - self.im * o.im, self.re * o.im + self.im * o.re)
    def __sub__(self, o): return _CFrac(self.re - o.re, self.im - o.im)
    def __truediv__(self, o):
        d = o.re * o.re + o.im * o.im
        return _CFrac((self.re * o.re + self.im * o.im) / d, (self.im * o.re - self.re * o.im) / d)
    def __eq__(self, o): return (self.re, self.im) == ((o, 0) if isinstance(o, int) else (o.re, o.im))


@pytest.mark.parametrize("dtype", TYPES)
def test_hp_solver_against_exact_rational_solutions(dtype):
    """Small systems from the reference family solved exactly; the long double result must be the
    correctly rounded double of the exact solution up to a few ulps of long double."""
    dtype = np.dtype(dtype)
    transes = [NOTRANS, TRANS, CONJ]
    for order, side, uplo, tA, diag in itertools.product([ROW, COL], [LEFT, RIGHT], [UPPER, LOWER], transes,
                                                         [UNIT, NONUNIT]):
        M, N = (9, 4) if side == LEFT else (4, 9)
        n = 9
        alpha = 3 - 2j if dtype.kind == "c" else -3.0
        lda, ldb = n + 1, (M if order == COL else N) + 2
        A, B = oracle.trsm_ref_inputs(dtype, order, side, uplo, diag, M, N, 1.0, 2, lda, 1, ldb, 31 + tA)
        Av, Bv = _views(dtype, order, side, M, N, A, 2, lda, B, 1, ldb)
        if diag == UNIT:  # give the unit-diagonal systems some off-diagonal entries
            mask = np.tril(np.ones((n, n), bool), -1) if uplo == LOWER else np.triu(np.ones((n, n), bool), 1)
            Av[mask] = (np.arange(mask.sum()) % 5 - 2).astype(dtype)
        rhs = [0, 3] if True else None
        X = oracle.trsm_hp(order, side, uplo, tA, diag, M, N, alpha, A, 2, lda, B, 1, ldb, rhs)
        # effective matrix E with E x = alpha b
        op = Av.T if tA != NOTRANS else Av
        if tA == CONJ:
            op = op.conj()
        E = op if side == LEFT else op.T
        tri = np.tril if ((uplo == LOWER) != (tA != NOTRANS)) != (side == RIGHT) else np.triu
        Em = tri(np.nan_to_num(E))
        if diag == UNIT:
            Em = Em - np.diag(np.diag(Em)) + np.eye(n)
        Ef = [[_CFrac(Fraction(float(Em[i, j].real)), Fraction(float(Em[i, j].imag))) for j in range(n)] for i in range(n)]
        for qi, q in enumerate(rhs):
            b = Bv[:, q] if side == LEFT else Bv[q, :]
            al = _CFrac(Fraction(complex(alpha).real), Fraction(complex(alpha).imag))
            bf = [al * _CFrac(Fraction(float(v.real)), Fraction(float(v.imag))) for v in b]
            xe = _exact_solve(Ef, bf)
            for p in range(n):
                want = complex(float(xe[p].re), float(xe[p].im))
                got = complex(X[qi, p])
                scale = max(abs(want), 1e-300)
                assert abs(got - want) <= 4 * 2.0 ** -53 * scale, (order, side, uplo, tA, diag, q, p, got, want)


@pytest.mark.parametrize("dtype", TYPES)
def test_hp_solver_against_numpy_and_the_reference_naive_trsm(dtype):
    import scipy.linalg
    dtype = np.dtype(dtype)
    rng = np.random.default_rng(5)
    for order, side, uplo, tA, diag in itertools.product([ROW, COL], [LEFT, RIGHT], [UPPER, LOWER],
                                                         [NOTRANS, TRANS, CONJ], [UNIT, NONUNIT]):
        M, N = (45, 7) if side == LEFT else (7, 45)
        n = 45
        alpha = 0.5 + 0.25j if dtype.kind == "c" else 0.5
        lda, ldb = n, (M if order == COL else N)
        A = oracle.triangular(n, n, True, 3, np.float64).astype(dtype)   # values only; layout set below
        Afull = rng.uniform(-1, 1, (n, n)) / n + np.diag(rng.uniform(1, 2, n))
        if dtype.kind == "c":
            Afull = Afull + 1j * rng.uniform(-1, 1, (n, n)) / n
        Bfull = rng.uniform(-1, 1, (M, N)) + (1j * rng.uniform(-1, 1, (M, N)) if dtype.kind == "c" else 0)
        A = np.ascontiguousarray(Afull.T if order == COL else Afull).astype(dtype).ravel()
        B = np.ascontiguousarray(Bfull.T if order == COL else Bfull).astype(dtype).ravel()
        Av = logical_view(A, order, NOTRANS, n, n, 0, lda).astype(np.complex128)
        Bv = logical_view(B, order, NOTRANS, M, N, 0, ldb).astype(np.complex128)
        T = np.tril(Av) if uplo == LOWER else np.triu(Av)
        if diag == UNIT:
            T = T - np.diag(np.diag(T)) + np.eye(n)
        op = T if tA == NOTRANS else (T.T if tA == TRANS else T.conj().T)
        want = np.linalg.solve(op, alpha * Bv) if side == LEFT else np.linalg.solve(op.T, (alpha * Bv).T).T
        rhs = list(range(N if side == LEFT else M))
        X = oracle.trsm_hp(order, side, uplo, tA, diag, M, N, alpha, A, 0, lda, B, 0, ldb, rhs)
        got = X.T if side == LEFT else X
        assert np.abs(got - want).max() <= 1e-12 * np.abs(want).max(), (order, side, uplo, tA, diag)
        # the reference's naive trsm in the working precision stays within n * eps of it
        if tA != CONJ or dtype.kind == "c":
            Bn = B.copy()
            oracle.ref_trsm(order, side, uplo, tA, diag, M, N, alpha, A, lda, Bn, ldb)
            naive = logical_view(Bn, order, NOTRANS, M, N, 0, ldb)
            eps = np.finfo(dtype).eps
            assert np.abs(naive - got).max() <= 8 * n * eps * np.abs(want).max()


@pytest.mark.parametrize("dtype", TYPES)
def test_vectorised_delta_equals_the_reference_loops(dtype):
    rng = np.random.default_rng(9)
    for n in (1, 5, 31, 32, 33, 100):
        absd = rng.uniform(0.3, 30, n)
        absb = rng.uniform(0, 1000, (3, n))
        for side, uplo, tA, diag in itertools.product([LEFT, RIGHT], [UPPER, LOWER], [NOTRANS, TRANS, CONJ],
                                                      [UNIT, NONUNIT]):
            a = trsm_ref_delta(dtype, side, uplo, tA, diag, 1.5, absd, absb)
            b = trsm_ref_delta_loops(dtype, side, uplo, tA, diag, 1.5, absd, absb)
            assert np.allclose(a, b, rtol=1e-12, atol=0), (n, side, uplo, tA, diag)
