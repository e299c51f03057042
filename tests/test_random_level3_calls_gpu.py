"""Randomised calls of SYRK, SYR2K, TRMM, SYMM (S, D, C, Z) and HERK, HER2K, HEMM (C, Z) through the C
ABI, every argument drawn from a seeded generator.  Small integer data (Gaussian integers for the complex
types) make the result independent of the summation order, so it must EQUAL the product formed by numpy
in a wider type from the definition of each routine (clBLAS.h: the BLAS level 3 argument conventions).
Elements that a routine must not read hold NaN (padding, the other triangle of a triangular / symmetric /
Hermitian operand, a unit diagonal, all of C's triangle when beta == 0); the other triangle of C and every
padding element of the output must come back untouched."""
import numpy as np
import pytest

from helpers import COL
from test_random_calls_gpu import _dim, _ints, _op, _store, _view

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    import gpu_util
    import torch
    assert torch.cuda.is_available()
    import clblas_amd
    assert clblas_amd.setup() == 0
    return gpu_util


def _tri(n, lower, strict=False):
    i, j = np.indices((n, n))
    return (i > j if strict else i >= j) if lower else (i < j if strict else i <= j)


def _scalar(rng, cplx, choices):
    a = choices[int(rng.integers(0, len(choices)))]
    return a + 1j * int(rng.integers(-1, 2)) if cplx else a


def _check_triangle(out, before, off, ld, n, order, keep, want, what):
    """The `keep` part of the n x n result equals `want`; everything else in the buffer is unchanged."""
    got = _view(out, off, ld, n, n, order)
    assert np.array_equal(got[keep].astype(want.dtype), want[keep]), what
    a, b = out.copy(), before.copy()
    _view(a, off, ld, n, n, order)[keep] = 0
    _view(b, off, ld, n, n, order)[keep] = 0
    assert np.array_equal(a, b, equal_nan=True), what + " (outside the triangle)"


def _sym_operand(rng, n, dt, lower, hermitian):
    """(dense symmetric / Hermitian matrix in the wide type, stored matrix with NaN in the other triangle)."""
    cplx = np.dtype(dt).kind == "c"
    wide = np.complex128 if cplx else np.float64
    t = _ints(rng, n * n, dt).reshape(n, n)
    if hermitian:
        t[np.arange(n), np.arange(n)] = t.diagonal().real
    keep = _tri(n, lower)
    half = np.where(keep, t, 0).astype(wide)
    strict = np.where(_tri(n, lower, True), t, 0).astype(wide)
    dense = half + (strict.conj().T if hermitian else strict.T)
    stored = np.full((n, n), np.nan, dtype=dt)
    stored[keep] = t[keep]
    return dense, stored


@pytest.mark.parametrize("seed", [1, 2])
def test_random_rank_k_updates_integer_exact(gpu, seed):
    """SYRK, SYR2K (trans N / T), HERK, HER2K (trans N / C)."""
    rng = np.random.default_rng(200 + seed)
    for case in range(900):
        routine = ["syrk", "syr2k", "herk", "her2k"][int(rng.integers(0, 4))]
        herm = routine in ("herk", "her2k")
        dt = [np.complex64, np.complex128][int(rng.integers(0, 2))] if herm else \
            [np.float32, np.float64, np.complex64, np.complex128][int(rng.integers(0, 4))]
        cplx = np.dtype(dt).kind == "c"
        wide = np.complex128 if cplx else np.float64
        order, uplo = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        trans = [0, 2 if herm else 1][int(rng.integers(0, 2))]
        N, K = _dim(rng, 1500), _dim(rng, 3000)
        alpha = _scalar(rng, cplx and routine != "herk", [0, 1, -2, 3])
        beta = _scalar(rng, cplx and not herm, [0, 1, -1, 2])
        Al, Bl = _ints(rng, N * K, dt).reshape(N, K), _ints(rng, N * K, dt).reshape(N, K)
        Cl = _ints(rng, N * N, dt).reshape(N, N)
        if herm:
            Cl[np.arange(N), np.arange(N)] = Cl.diagonal().real
        A, offA, lda = _store(rng, _op(Al, trans), order, dt, np.nan)
        B, offB, ldb = _store(rng, _op(Bl, trans), order, dt, np.nan)
        keep = _tri(N, uplo == 1)
        Cs = np.where(keep, Cl, 99).astype(dt)
        if beta == 0:
            Cs[keep] = np.nan
        C, offC, ldc = _store(rng, Cs, order, dt, 77)
        what = "seed %d case %d: %s %s order %d uplo %d trans %d  N %d K %d alpha %s beta %s" % (
            seed, case, routine, np.dtype(dt).name, order, uplo, trans, N, K, alpha, beta)
        Aw, Bw = Al.astype(wide), Bl.astype(wide)
        if routine == "syrk":
            st, out = gpu.syrk(order, uplo, trans, N, K, alpha, A, offA, lda, beta, C, offC, ldc)
            want = alpha * (Aw @ Aw.T)
        elif routine == "syr2k":
            st, out = gpu.syr2k(order, uplo, trans, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc)
            want = alpha * (Aw @ Bw.T) + alpha * (Bw @ Aw.T)
        elif routine == "herk":
            st, out = gpu.herk(order, uplo, trans, N, K, alpha, A, offA, lda, beta, C, offC, ldc)
            want = alpha * (Aw @ Aw.conj().T)
        else:
            st, out = gpu.her2k(order, uplo, trans, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc)
            want = alpha * (Aw @ Bw.conj().T) + np.conj(alpha) * (Bw @ Aw.conj().T)
        assert st == 0, what
        if beta != 0:
            want = want + beta * Cl.astype(wide)
        want = np.asarray(want, dtype=wide)
        _check_triangle(out, C, offC, ldc, N, order, keep, want, what)


@pytest.mark.parametrize("seed", [1, 2])
def test_random_trmm_symm_hemm_integer_exact(gpu, seed):
    rng = np.random.default_rng(300 + seed)
    for case in range(900):
        routine = ["trmm", "symm", "hemm"][int(rng.integers(0, 3))]
        dt = [np.complex64, np.complex128][int(rng.integers(0, 2))] if routine == "hemm" else \
            [np.float32, np.float64, np.complex64, np.complex128][int(rng.integers(0, 4))]
        cplx = np.dtype(dt).kind == "c"
        wide = np.complex128 if cplx else np.float64
        order, side, uplo = int(rng.integers(0, 2)), int(rng.integers(0, 2)), int(rng.integers(0, 2))
        M, N = _dim(rng, 1500), _dim(rng, 1500)
        n = M if side == 0 else N
        alpha = _scalar(rng, cplx, [0, 1, -2, 3])
        Bl = _ints(rng, M * N, dt).reshape(M, N)
        B, offB, ldb = _store(rng, Bl, order, dt, 55 if routine == "trmm" else np.nan)
        full = np.ones((M, N), bool)
        if routine == "trmm":
            tA, diag = int(rng.integers(0, 3)), int(rng.integers(0, 2))
            t = _ints(rng, n * n, dt).reshape(n, n)
            strict = _tri(n, uplo == 1, True)
            on_diag = np.ones(n) if diag == 0 else t.diagonal().astype(wide)
            dense = np.where(strict, t, 0).astype(wide) + np.diag(on_diag)
            stored = np.full((n, n), np.nan, dtype=dt)
            stored[strict] = t[strict]
            if diag == 1:
                stored[np.arange(n), np.arange(n)] = t.diagonal()
            A, offA, lda = _store(rng, stored, order, dt, np.nan)
            what = "seed %d case %d: trmm %s order %d side %d uplo %d trans %d diag %d  %d x %d alpha %s" % (
                seed, case, np.dtype(dt).name, order, side, uplo, tA, diag, M, N, alpha)
            st, out = gpu.trmm(order, side, uplo, tA, diag, M, N, alpha, A, offA, lda, B, offB, ldb)
            assert st == 0, what
            opA = _op(dense, tA)
            want = alpha * (opA @ Bl.astype(wide) if side == 0 else Bl.astype(wide) @ opA)
            _check_rect(out, B, offB, ldb, M, N, order, np.asarray(want, dtype=wide), what)
            continue
        beta = _scalar(rng, cplx, [0, 1, -1, 2])
        dense, stored = _sym_operand(rng, n, dt, uplo == 1, routine == "hemm")
        A, offA, lda = _store(rng, stored, order, dt, np.nan)
        Cl = _ints(rng, M * N, dt).reshape(M, N)
        Cs = Cl.copy()
        if beta == 0:
            Cs[full] = np.nan
        C, offC, ldc = _store(rng, Cs, order, dt, 77)
        what = "seed %d case %d: %s %s order %d side %d uplo %d  %d x %d alpha %s beta %s" % (
            seed, case, routine, np.dtype(dt).name, order, side, uplo, M, N, alpha, beta)
        fn = gpu.symm if routine == "symm" else gpu.hemm
        st, out = fn(order, side, uplo, M, N, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc)
        assert st == 0, what
        want = alpha * (dense @ Bl.astype(wide) if side == 0 else Bl.astype(wide) @ dense)
        if beta != 0:
            want = want + beta * Cl.astype(wide)
        _check_rect(out, C, offC, ldc, M, N, order, np.asarray(want, dtype=wide), what)


def _check_rect(out, before, off, ld, r, c, order, want, what):
    got = _view(out, off, ld, r, c, order)
    assert np.array_equal(got.astype(want.dtype), want), what
    a, b = out.copy(), before.copy()
    _view(a, off, ld, r, c, order)[...] = 0
    _view(b, off, ld, r, c, order)[...] = 0
    assert np.array_equal(a, b, equal_nan=True), what + " (padding)"
