"""Pins the CPU oracle's SYR2K (all four types), HERK, HER2K and HEMM (complex types) - oracle/level3.inc:
the reference samples' fixed inputs against exact expected values, exact-integer inputs against
products evaluated with numpy over every order / triangle / transpose (/ side) combination with the
unused triangle NaN-poisoned and junk imaginary parts on Hermitian diagonals, the reference's own
naive syr2k (oracle/_ref), identities that tie the Hermitian routines to the oracle's complex GEMM,
and the argument checks.  CPU only."""
import itertools

import numpy as np
import pytest

import oracle
from helpers import (COL, ROW, NOTRANS, TRANS, CONJ, UPPER, LOWER, LEFT, RIGHT, golden_array, golden_cases,
                     golden_scalar, logical_view)
from l3_util import ALL, CPLX, herm_dense, is_cplx, matrix, nan_of, poison_triangle, rank2k_want, real_scalars, scalars, tri_mask

needs_ref = pytest.mark.skipif(oracle.ref_lib() is None, reason="oracle/_ref not built (no reference tree)")
WIDE = lambda dt: np.complex128 if is_cplx(dt) else np.float64
DT = {"f32": np.float32, "f64": np.float64, "c64": np.complex64, "c128": np.complex128}


def run_golden(mod, c):
    """Runs fixture c through `mod` (the oracle module or the GPU helper module); returns (status, C)."""
    dt = DT[c["dtype"]]
    A, C = golden_array(c["A"], dt), golden_array(c["C"], dt)
    al, be = golden_scalar(c["alpha"]), golden_scalar(c["beta"])
    if c["kind"] == "herk":
        r = mod.herk(c["order"], c["uplo"], c["transA"], c["N"], c["K"], al, A, c["offA"], c["lda"], be, C, c["offC"],
                     c["ldc"])
    elif c["kind"] == "hemm":
        B = golden_array(c["B"], dt)
        r = mod.hemm(c["order"], c["side"], c["uplo"], c["M"], c["N"], al, A, c["offA"], c["lda"], B, c["offB"],
                     c["ldb"], be, C, c["offC"], c["ldc"])
    else:
        B = golden_array(c["B"], dt)
        fn = mod.syr2k if c["kind"] == "syr2k" else mod.her2k
        r = fn(c["order"], c["uplo"], c["transA"], c["N"], c["K"], al, A, c["offA"], c["lda"], B, c["offB"], c["ldb"],
               be, C, c["offC"], c["ldc"])
    return (r, C) if isinstance(r, int) else r


GOLDEN = ["sample_ssyr2k_offsets", "sample_cherk", "sample_cher2k", "sample_chemm"]


@pytest.mark.parametrize("name", GOLDEN)
def test_golden(name):
    c = golden_cases()[name]
    st, out = run_golden(oracle, c)
    assert st == 0
    np.testing.assert_array_equal(out, golden_array(c["expected"], DT[c["dtype"]]))  # small integers: exact


def rank2k_case(kind, dtype, order, uplo, trans, N, K, seed, integer):
    rows, cols = (N, K) if trans == NOTRANS else (K, N)
    A, lda = matrix(order, rows, cols, 5, 3, seed, dtype, integer)
    B, ldb = matrix(order, rows, cols, 3, 1, seed + 1, dtype, integer)
    C, ldc = matrix(order, N, N, 7, 2, seed + 2, dtype, integer)
    keep = tri_mask(N, uplo == LOWER)
    logical_view(C, order, NOTRANS, N, N, 7, ldc)[~keep] = nan_of(dtype)  # must stay untouched
    return A, lda, B, ldb, C, ldc, keep


def rank2k_scalars(kind, dtype, integer):
    al, be = scalars(dtype) if integer else real_scalars(dtype)
    if kind == "herk":
        return (2.0, -3.0) if integer else (0.7, -1.3)
    if kind == "her2k":
        return al, (-3.0 if integer else -1.3)
    return al, be


def call_rank2k(mod, kind, order, uplo, trans, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc):
    if kind == "herk":
        return mod.herk(order, uplo, trans, N, K, alpha, A, offA, lda, beta, C, offC, ldc)
    fn = mod.syr2k if kind == "syr2k" else mod.her2k
    return fn(order, uplo, trans, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc)


def rank2k_variants():
    out = []
    for dtype in ALL:
        for order, uplo in itertools.product([ROW, COL], [UPPER, LOWER]):
            tr = [NOTRANS, TRANS] if is_cplx(dtype) else [NOTRANS, TRANS, CONJ]
            out += [("syr2k", dtype, order, uplo, t) for t in tr]
            if is_cplx(dtype):
                out += [(k, dtype, order, uplo, t) for k in ("herk", "her2k") for t in (NOTRANS, CONJ)]
    return out


RANK2K_SIZES = [(1, 1), (5, 3), (17, 33), (64, 20), (70, 129)]


@pytest.mark.parametrize("kind,dtype,order,uplo,trans", rank2k_variants())
def test_rank2k_integer_exact(kind, dtype, order, uplo, trans):
    alpha, beta = rank2k_scalars(kind, dtype, True)
    for si, (N, K) in enumerate(RANK2K_SIZES):
        A, lda, B, ldb, C, ldc, keep = rank2k_case(kind, dtype, order, uplo, trans, N, K, 10 + 3 * si, True)
        C0 = C.copy()
        assert call_rank2k(oracle, kind, order, uplo, trans, N, K, alpha, A, 5, lda, B, 3, ldb, beta, C, 7, ldc) == 0
        want, _ = rank2k_want(kind, order, uplo, trans, N, K, alpha, A, 5, lda, B, 3, ldb, beta, C0, 7, ldc)
        got = logical_view(C, order, NOTRANS, N, N, 7, ldc)
        np.testing.assert_array_equal(got[keep].astype(WIDE(dtype)), want[keep])
        idx = logical_view(np.arange(C.size), order, NOTRANS, N, N, 7, ldc)[keep]
        rest = np.ones(C.size, dtype=bool)
        rest[idx] = False
        np.testing.assert_array_equal(C[rest].view(np.uint8), C0[rest].view(np.uint8))


@pytest.mark.parametrize("dtype", CPLX)
@pytest.mark.parametrize("kind", ["herk", "her2k"])
def test_hermitian_diagonal_and_beta_zero(kind, dtype):
    """beta == 0 never reads C; the diagonal comes out exactly real."""
    N, K = 9, 4
    A, lda = matrix(COL, N, K, 0, 0, 1, dtype, False)
    B, ldb = matrix(COL, N, K, 0, 0, 2, dtype, False)
    C = np.full(N * N, nan_of(dtype), dtype=dtype)
    alpha = 0.5 if kind == "herk" else (0.5 - 0.25j)
    assert call_rank2k(oracle, kind, COL, LOWER, NOTRANS, N, K, alpha, A, 0, lda, B, 0, ldb, 0.0, C, 0, N) == 0
    Cv = C.reshape(N, N, order="F")
    assert (np.diag(Cv).imag == 0).all() and not np.isnan(Cv[tri_mask(N, True)]).any()
    assert np.isnan(Cv[~tri_mask(N, True)].real).all()
    # her2k with B == A and real alpha is herk with 2 alpha
    if kind == "her2k":
        C1 = np.zeros(N * N, dtype=dtype)
        C2 = np.zeros(N * N, dtype=dtype)
        assert oracle.her2k(COL, LOWER, NOTRANS, N, K, 0.5, A, 0, lda, A, 0, lda, 0.0, C1, 0, N) == 0
        assert oracle.herk(COL, LOWER, NOTRANS, N, K, 1.0, A, 0, lda, 0.0, C2, 0, N) == 0
        np.testing.assert_allclose(C1, C2, rtol=0, atol=8 * K * np.finfo(dtype).eps)


@pytest.mark.parametrize("dtype", CPLX)
def test_rank2k_checks(dtype):
    N, K = 9, 4
    A = np.zeros(N * K, dtype=dtype)
    C = np.zeros(N * N, dtype=dtype)
    for kind in ("syr2k", "herk", "her2k"):
        al = 1.0
        f = lambda **kw: call_rank2k(oracle, kind, COL, LOWER, kw.get("trans", NOTRANS), N, kw.get("K", K), al,
                                     kw.get("A", A), 0, kw.get("lda", N), kw.get("B", A), 0, kw.get("ldb", N), 0.0,
                                     kw.get("C", C), 0, kw.get("ldc", N))
        assert f() == 0
        assert f(A=None) == -1022
        assert f(C=None) == -1020
        assert f(K=0) == -1017
        assert f(lda=N - 1) == -1016
        assert f(ldc=N - 1) == -1014
        if kind != "herk":
            assert f(B=None) == -1021
            assert f(ldb=N - 1) == -1015
        # complex SYR2K has no conjugate transpose; the Hermitian updates have no plain transpose
        assert f(trans=CONJ if kind == "syr2k" else TRANS, lda=K, ldb=K) == -30


@needs_ref
@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("order,uplo,trans", list(itertools.product([ROW, COL], [UPPER, LOWER], [NOTRANS, TRANS])))
def test_syr2k_vs_reference_naive(dtype, order, uplo, trans):
    N, K = 37, 45
    rows, cols = (N, K) if trans == NOTRANS else (K, N)
    for integer in (True, False):
        alpha, beta = scalars(dtype) if integer else real_scalars(dtype)
        A, lda = matrix(order, rows, cols, 0, 2, 1, dtype, integer)
        B, ldb = matrix(order, rows, cols, 0, 3, 3, dtype, integer)
        C, ldc = matrix(order, N, N, 0, 1, 2, dtype, integer)
        Cr = C.copy()
        oracle.ref_syr2k(order, uplo, trans, N, K, alpha, A, lda, B, ldb, beta, Cr, ldc)
        assert oracle.syr2k(order, uplo, trans, N, K, alpha, A, 0, lda, B, 0, ldb, beta, C, 0, ldc) == 0
        if integer:
            np.testing.assert_array_equal(C, Cr)
        else:
            np.testing.assert_allclose(C, Cr, rtol=0, atol=16 * K * np.finfo(dtype).eps * 4)


# ------------------------------------------------------------------------------- HEMM
def hemm_case(dtype, order, side, uplo, M, N, seed, integer):
    n = M if side == LEFT else N
    A, lda = matrix(order, n, n, 5, 3, seed, dtype, integer, limit=4)
    poison_triangle(A, order, n, 5, lda, uplo)  # the other triangle is never read
    B, ldb = matrix(order, M, N, 7, 2, seed + 1, dtype, integer, limit=4)
    C, ldc = matrix(order, M, N, 11, 1, seed + 2, dtype, integer, limit=4)
    return A, lda, B, ldb, C, ldc


def hemm_want(order, side, uplo, M, N, alpha, A, lda, B, ldb, beta, C0, ldc):
    n = M if side == LEFT else N
    H = herm_dense(A, order, n, 5, lda, uplo)
    Bv = logical_view(B, order, NOTRANS, M, N, 7, ldb).astype(np.complex128)
    Cv = logical_view(C0, order, NOTRANS, M, N, 11, ldc).astype(np.complex128)
    return alpha * (H @ Bv if side == LEFT else Bv @ H) + beta * Cv


@pytest.mark.parametrize("dtype", CPLX)
@pytest.mark.parametrize("order,side,uplo", list(itertools.product([ROW, COL], [LEFT, RIGHT], [UPPER, LOWER])))
def test_hemm_integer_exact(dtype, order, side, uplo):
    alpha, beta = scalars(dtype)
    for si, (M, N) in enumerate([(1, 1), (3, 7), (16, 17), (33, 20), (70, 45)]):
        A, lda, B, ldb, C, ldc = hemm_case(dtype, order, side, uplo, M, N, 50 + 3 * si, True)
        C0 = C.copy()
        assert oracle.hemm(order, side, uplo, M, N, alpha, A, 5, lda, B, 7, ldb, beta, C, 11, ldc) == 0
        want = hemm_want(order, side, uplo, M, N, alpha, A, lda, B, ldb, beta, C0, ldc)
        got = logical_view(C, order, NOTRANS, M, N, 11, ldc)
        np.testing.assert_array_equal(got.astype(np.complex128), want)
        mask = np.ones(C.size, dtype=bool)
        logical_view(mask, order, NOTRANS, M, N, 11, ldc)[:] = False
        np.testing.assert_array_equal(C[mask].view(np.uint8), C0[mask].view(np.uint8))


@pytest.mark.parametrize("dtype", CPLX)
def test_hemm_is_gemm_on_the_full_matrix(dtype):
    """HEMM equals the (pinned) complex GEMM oracle applied to the explicitly formed Hermitian matrix."""
    M, N = 23, 31
    for side, uplo in itertools.product([LEFT, RIGHT], [UPPER, LOWER]):
        A, lda, B, ldb, C, ldc = hemm_case(dtype, COL, side, uplo, M, N, 77, False)
        n = M if side == LEFT else N
        H = herm_dense(A, COL, n, 5, lda, uplo).astype(dtype).ravel(order="F").copy()
        Cg = C.copy()
        assert oracle.hemm(COL, side, uplo, M, N, 0.7 - 0.3j, A, 5, lda, B, 7, ldb, -1.3 + 0.5j, C, 11, ldc) == 0
        if side == LEFT:
            st = oracle.gemm(COL, NOTRANS, NOTRANS, M, N, M, 0.7 - 0.3j, H, 0, n, B, 7, ldb, -1.3 + 0.5j, Cg, 11, ldc)
        else:
            st = oracle.gemm(COL, NOTRANS, NOTRANS, M, N, N, 0.7 - 0.3j, B, 7, ldb, H, 0, n, -1.3 + 0.5j, Cg, 11, ldc)
        assert st == 0
        np.testing.assert_allclose(C, Cg, rtol=0, atol=64 * n * np.finfo(dtype).eps)


def test_hemm_checks():
    M, N = 6, 4
    A = np.zeros(36, dtype=np.complex64)
    B = np.zeros(24, dtype=np.complex64)
    C = np.zeros(24, dtype=np.complex64)
    f = lambda **kw: oracle.hemm(COL, kw.get("side", LEFT), LOWER, M, N, 1.0, kw.get("A", A), 0, kw.get("lda", 6),
                                 kw.get("B", B), 0, kw.get("ldb", M), 0.0, kw.get("C", C), 0, kw.get("ldc", M))
    assert f() == 0
    assert f(A=None) == -1022 and f(B=None) == -1021 and f(C=None) == -1020
    assert f(lda=5) == -1016 and f(ldb=5) == -1015 and f(ldc=5) == -1014
    assert f(side=RIGHT, lda=3) == -1016
