"""Input builders and exact expectations shared by the SYRK / TRMM / SYMM tests (CPU oracle
pinning and GPU parity)."""
import numpy as np

import oracle
from helpers import COL, ROW, NOTRANS, TRANS, CONJ, UPPER, LOWER, UNIT, NONUNIT, LEFT, RIGHT, logical_view, mem_dims

REAL = [np.float32, np.float64]
CPLX = [np.complex64, np.complex128]
ALL = REAL + CPLX


def is_cplx(dtype):
    return np.dtype(dtype).kind == "c"


def nan_of(dtype):
    return dtype(complex(np.nan, np.nan)) if is_cplx(dtype) else dtype(np.nan)


def scalars(dtype):
    """Exactly representable alpha, beta (Gaussian integers for the complex types)."""
    return ((2 - 1j), (-1 + 2j)) if is_cplx(dtype) else (2.0, -3.0)


def real_scalars(dtype):
    return ((0.7 - 0.3j), (-1.3 + 0.5j)) if is_cplx(dtype) else (0.7, -1.3)


def matrix(order, rows, cols, off, pad, seed, dtype, integer, limit=8):
    """1-D buffer (+ld) holding a rows x cols matrix in `order` with `pad` extra leading
    elements per stride and `off` leading elements."""
    inner, outer = mem_dims(order, NOTRANS, rows, cols)
    ld = inner + pad
    n = off + outer * ld
    buf = oracle.integers(n, seed, limit, dtype) if integer else oracle.uniform(n, seed, dtype)
    return buf, ld


def tri_mask(n, lower):
    i, j = np.indices((n, n))
    return i >= j if lower else i <= j


def poison_triangle(buf, order, n, off, ld, uplo, unit=False):
    """NaN everywhere in the n x n square except the `uplo` triangle (and, with unit, NaN on the
    diagonal too): anything that reads the wrong element shows up as NaN."""
    v = logical_view(buf, order, NOTRANS, n, n, off, ld)
    keep = tri_mask(n, uplo == LOWER)
    if unit:
        keep = keep & ~np.eye(n, dtype=bool)
    v[~keep] = nan_of(buf.dtype.type)


def tri_dense(buf, order, n, off, ld, uplo, unit):
    """The triangular matrix the routines see: zeros outside the triangle, ones on a unit diagonal."""
    v = logical_view(buf, order, NOTRANS, n, n, off, ld)
    t = np.where(tri_mask(n, uplo == LOWER), v, 0).astype(np.complex128 if is_cplx(buf.dtype) else np.float64)
    if unit:
        np.fill_diagonal(t, 1)
    return t


def sym_dense(buf, order, n, off, ld, uplo):
    v = logical_view(buf, order, NOTRANS, n, n, off, ld)
    wide = np.complex128 if is_cplx(buf.dtype) else np.float64
    t = np.where(tri_mask(n, uplo == LOWER), v, 0).astype(wide)
    return t + t.T - np.diag(np.diag(t))


def op(x, trans):
    return x if trans == NOTRANS else (x.T if trans == TRANS else x.conj().T)


def abs1(x):
    """|re| + |im| (plain |x| for real data)."""
    return np.abs(x.real) + np.abs(x.imag) if np.iscomplexobj(x) else np.abs(x)


def bound(K, mag, dtype, c=2.0):
    """c (2K+6) u mag for complex, c (K+2) u mag for real data (see helpers.gemm_bound)."""
    from helpers import cgemm_bound, gemm_bound
    return cgemm_bound(K, mag, dtype, c) if is_cplx(dtype) else gemm_bound(K, mag, dtype, c)


def err(got, want):
    d = got - want
    return np.maximum(np.abs(d.real), np.abs(d.imag)) if np.iscomplexobj(d) else np.abs(d)


# ---- complex triangular systems (CTRSM / ZTRSM) -------------------------------------------

def ctrsm_inputs(order, side, uplo, diag, M, N, dtype, seed, offA=5, offB=7):
    """Conditioned complex triangular A (real part from the real generator - strict triangle
    uniform/n, diagonal in [1,2) - plus an imaginary part of the same size; NaN outside the
    triangle and on a unit diagonal) and a uniform complex B, with offsets and padded leading
    dimensions."""
    real = np.float32 if np.dtype(dtype) == np.dtype(np.complex64) else np.float64
    n = M if side == LEFT else N
    lda = n + 3
    lower_in_memory = (uplo == LOWER) == (order == COL)
    re = oracle.triangular(n, lda, lower_in_memory, seed, real, poison_diag=(diag == UNIT))
    im = oracle.triangular(n, lda, lower_in_memory, seed + 100, real, poison_diag=(diag == UNIT))
    sq = im[:n * lda].reshape(n, lda)[:, :n]
    sq[np.eye(n, dtype=bool)] -= real(1.5)  # diagonal imaginary parts in [-0.5, 0.5)
    A = np.concatenate([np.full(offA, nan_of(dtype), dtype=dtype), (re + 1j * im).astype(dtype)])
    ib, ob = (M, N) if order == COL else (N, M)
    ldb = ib + 2
    B = oracle.uniform(offB + ob * ldb, seed + 1, dtype)
    return A, lda, B, ldb


def trsm_backward_error(order, side, uplo, tA, diag, M, N, alpha, A, offA, lda, B0, X, offB, ldb):
    """Normwise backward error ||op(A) X - alpha B|| / (||op(A)|| ||X|| + |alpha| ||B||) (infinity
    norms; X op(A) for side == right), evaluated with numpy in complex128."""
    n = M if side == LEFT else N
    Am = op(tri_dense(A, order, n, offA, lda, uplo, diag == UNIT), tA)
    Xm = logical_view(X, order, NOTRANS, M, N, offB, ldb).astype(np.complex128)
    Bm = logical_view(B0, order, NOTRANS, M, N, offB, ldb).astype(np.complex128)
    R = (Am @ Xm if side == LEFT else Xm @ Am) - alpha * Bm
    nrm = lambda Z: np.abs(Z).sum(axis=1).max()
    return nrm(R) / (nrm(Am) * nrm(Xm) + abs(alpha) * nrm(Bm))


# ---- SYR2K / HERK / HER2K / HEMM -----------------------------------------------------------

def herm_dense(buf, order, n, off, ld, uplo):
    """The Hermitian matrix the routines see: the stored triangle, its conjugate mirror, and the
    real parts of the stored diagonal."""
    v = logical_view(buf, order, NOTRANS, n, n, off, ld)
    t = np.where(tri_mask(n, uplo == LOWER), v, 0).astype(np.complex128)
    d = np.diag(t).real.copy()
    np.fill_diagonal(t, 0)
    return t + t.conj().T + np.diag(d)


def rank2k_want(kind, order, uplo, trans, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C0, offC, ldc):
    """Expected stored triangle (N x N, wide precision; entries outside it are meaningless) and the
    magnitude sum |alpha|(|A||B|^T ...) + |beta||C| for error bounds, for kind in
    {"syr2k", "herk", "her2k"}, evaluated with numpy."""
    wide = np.complex128 if is_cplx(C0.dtype) else np.float64
    rows, cols = (N, K) if trans == NOTRANS else (K, N)
    Av = logical_view(A, order, NOTRANS, rows, cols, offA, lda).astype(wide)
    Aop = op(Av, trans)
    Cv = logical_view(C0, order, NOTRANS, N, N, offC, ldc).astype(wide)
    if kind == "herk":
        want = alpha * (Aop @ Aop.conj().T)
        mag = abs(alpha) * (abs1(Aop) @ abs1(Aop).T)
    else:
        Bop = op(logical_view(B, order, NOTRANS, rows, cols, offB, ldb).astype(wide), trans)
        if kind == "syr2k":
            want = alpha * (Aop @ Bop.T + Bop @ Aop.T)
        else:
            want = alpha * (Aop @ Bop.conj().T) + np.conj(alpha) * (Bop @ Aop.conj().T)
        mag = 2 * abs1(np.asarray(alpha)) * (abs1(Aop) @ abs1(Bop).T + abs1(Bop) @ abs1(Aop).T)
    if beta != 0:
        Cin = Cv.copy()
        if kind != "syr2k":
            Cin[np.eye(N, dtype=bool)] = Cin[np.eye(N, dtype=bool)].real
        want = want + beta * Cin
        mag = mag + abs1(np.asarray(beta)) * abs1(np.nan_to_num(Cin))
    if kind != "syr2k":
        want[np.eye(N, dtype=bool)] = want[np.eye(N, dtype=bool)].real
    return want, mag
