"""Randomised calls of the GEMM and TRSM entry points (S, D, C, Z) through the C ABI: every argument
drawn from a seeded generator - order, transposes, side/uplo/diag, shapes from 1 to a few thousand,
offsets, padded leading dimensions, alpha/beta including 0.

GEMM uses the reference tests' exact-integer method (corr-gemm.cpp:192, matrix.h:322-327): small
integer data make every summation order give the same bits, so the result must EQUAL the integer
product computed in a wider type.  The padding of A and B and, when beta == 0, all of C hold NaN
(never to be used); the padding of C must come back untouched.
TRSM checks the componentwise backward error |op(A) X - alpha B| <= (n+2) u (|op(A)||X| + |alpha||B|),
with the unreferenced triangle (and a unit diagonal) of A holding NaN."""
import numpy as np
import pytest

from helpers import COL

pytestmark = pytest.mark.gpu

DT = [np.float32, np.float64, np.complex64, np.complex128]


@pytest.fixture(scope="module")
def gpu():
    import gpu_util
    import torch
    assert torch.cuda.is_available()
    import clblas_amd
    assert clblas_amd.setup() == 0
    return gpu_util


def _dim(rng, big):
    r = rng.random()
    if r < 0.1:
        return int(rng.integers(1, 4))
    if r < 0.6:
        return int(rng.integers(1, 200))
    if r < 0.93:
        return int(rng.integers(1, 700))
    return int(rng.integers(1, big))


def _ints(rng, n, dt):
    x = rng.integers(-4, 5, n).astype(dt)
    if np.dtype(dt).kind == "c":
        x = (x + 1j * rng.integers(-4, 5, n)).astype(dt)
    return x


def _store(rng, mat, order, dt, fill):
    """Buffer holding the logical matrix `mat` with a random offset and leading dimension."""
    r, c = mat.shape
    fast, slow = (r, c) if order == COL else (c, r)
    ld = fast + int(rng.integers(0, 7))
    off = int(rng.integers(0, 13))
    buf = np.full(off + slow * ld + 3, fill, dtype=dt)
    buf[off:off + slow * ld].reshape(slow, ld)[:, :fast] = mat.T if order == COL else mat
    return buf, off, ld


def _view(buf, off, ld, r, c, order):
    fast, slow = (r, c) if order == COL else (c, r)
    v = buf[off:off + slow * ld].reshape(slow, ld)[:, :fast]
    return v.T if order == COL else v


def _op(x, t):
    return x if t == 0 else (x.T if t == 1 else x.conj().T)


def _padding_untouched(out, before, off, ld, r, c, order):
    a, b = out.copy(), before.copy()
    _view(a, off, ld, r, c, order)[...] = 0
    _view(b, off, ld, r, c, order)[...] = 0
    return np.array_equal(a, b)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_gemm_calls_integer_exact(gpu, seed):
    rng = np.random.default_rng(seed)
    for case in range(1500):
        dt = DT[int(rng.integers(0, 4))]
        cplx = np.dtype(dt).kind == "c"
        wide = np.complex128 if cplx else np.float64
        order, tA, tB = int(rng.integers(0, 2)), int(rng.integers(0, 3)), int(rng.integers(0, 3))
        M, N, K = _dim(rng, 2000), _dim(rng, 2000), _dim(rng, 6000)
        alpha = [0, 1, -2, 3][int(rng.integers(0, 4))]
        beta = [0, 1, -1, 2][int(rng.integers(0, 4))]
        if cplx:
            alpha = alpha + 1j * int(rng.integers(-1, 2))
            beta = beta + (1j * int(rng.integers(-1, 2)) if beta != 0 else 0)
        Al = _ints(rng, M * K, dt).reshape(M, K)
        Bl = _ints(rng, K * N, dt).reshape(K, N)
        Cl = _ints(rng, M * N, dt).reshape(M, N)
        # op(stored A) = Al: store the (conjugate) transpose when the call transposes
        A, offA, lda = _store(rng, _op(Al, tA), order, dt, np.nan)
        B, offB, ldb = _store(rng, _op(Bl, tB), order, dt, np.nan)
        C, offC, ldc = _store(rng, Cl, order, dt, 77)
        if beta == 0:
            _view(C, offC, ldc, M, N, order)[...] = np.nan
        what = "seed %d case %d: %s order %d trans %d %d  %d x %d x %d alpha %s beta %s" % (
            seed, case, np.dtype(dt).name, order, tA, tB, M, N, K, alpha, beta)
        st, out = gpu.gemm(order, tA, tB, M, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc)
        assert st == 0, what
        want = alpha * (Al.astype(wide) @ Bl.astype(wide)) + (beta * Cl.astype(wide) if beta != 0 else 0)
        got = _view(out, offC, ldc, M, N, order).astype(wide)
        assert np.array_equal(got, want), what
        assert _padding_untouched(out, C, offC, ldc, M, N, order), what


@pytest.mark.parametrize("seed", [1, 2])
def test_random_trsm_calls_backward_error(gpu, seed):
    rng = np.random.default_rng(100 + seed)
    for case in range(800):
        dt = DT[int(rng.integers(0, 4))]
        cplx = np.dtype(dt).kind == "c"
        wide = np.complex128 if cplx else np.float64
        u = np.finfo(dt).eps
        order = int(rng.integers(0, 2))
        side, uplo, tA, diag = (int(rng.integers(0, 2)), int(rng.integers(0, 2)), int(rng.integers(0, 3)),
                                int(rng.integers(0, 2)))
        M, N = _dim(rng, 1500), _dim(rng, 1500)
        n = M if side == 0 else N
        alpha = [1.0, -0.5, 2.0, 0.75][int(rng.integers(0, 4))] + (0.5j if cplx else 0)
        T = (rng.random((n, n)) * 2 - 1) / n
        if cplx:
            T = T + 1j * (rng.random((n, n)) * 2 - 1) / n
        T = T.astype(dt)
        d = (rng.random(n) + 1).astype(dt)
        lower = uplo == 1
        strict = np.tril(np.ones((n, n), bool), -1) if lower else np.triu(np.ones((n, n), bool), 1)
        full = np.where(strict, T, 0).astype(dt) + np.diag(np.ones(n, dtype=dt) if diag == 0 else d)
        stored = np.full((n, n), np.nan, dtype=dt)   # other triangle and a unit diagonal: never read
        stored[strict] = T[strict]
        if diag == 1:
            stored[np.arange(n), np.arange(n)] = d
        Bl = (rng.standard_normal((M, N)) + (1j * rng.standard_normal((M, N)) if cplx else 0)).astype(dt)
        A, offA, lda = _store(rng, stored, order, dt, np.nan)
        B, offB, ldb = _store(rng, Bl, order, dt, 55)
        what = "seed %d case %d: %s order %d side %d uplo %d trans %d diag %d  %d x %d alpha %s" % (
            seed, case, np.dtype(dt).name, order, side, uplo, tA, diag, M, N, alpha)
        st, out = gpu.trsm(order, side, uplo, tA, diag, M, N, alpha, A, offA, lda, B, offB, ldb)
        assert st == 0, what
        X = _view(out, offB, ldb, M, N, order).astype(wide)
        assert np.isfinite(X).all(), what
        opA = _op(full.astype(wide), tA)
        resid = (opA @ X if side == 0 else X @ opA) - alpha * Bl.astype(wide)
        scale = (np.abs(opA) @ np.abs(X) if side == 0 else np.abs(X) @ np.abs(opA)) + abs(alpha) * np.abs(Bl)
        assert np.all(np.abs(resid) <= (n + 2) * u * scale), what + " worst %.3g" % float(
            (np.abs(resid) / ((n + 2) * u * scale)).max())
        assert _padding_untouched(out, B, offB, ldb, M, N, order), what
