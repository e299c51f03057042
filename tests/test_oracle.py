"""Pins the CPU oracle (oracle/oracle.c) before anything is measured against it:
golden fixtures from the reference's own files, exact-integer inputs (the reference tests'
own method), closed forms, identities, and the reference's naive BLAS compiled from the
reference tree (oracle/_ref) where that is present.  CPU only."""
import itertools

import numpy as np
import pytest

import oracle
from helpers import (COL, ROW, NOTRANS, TRANS, CONJ, UPPER, LOWER, UNIT, NONUNIT, LEFT, RIGHT, buf_len,
                     exact_int_limits, gemm_bound, golden_cases, logical_view)

DT = {"f32": np.float32, "f64": np.float64}


# ---------------------------------------------------------------- golden fixtures
@pytest.mark.parametrize("name", ["readme_sgemm", "sample_sgemm_offsets"])
def test_gemm_golden(name):
    c = golden_cases()[name]
    dt = DT[c["dtype"]]
    A, B, C = (np.array(c[k], dtype=dt) for k in "ABC")
    st = oracle.gemm(c["order"], c["transA"], c["transB"], c["M"], c["N"], c["K"], c["alpha"], A, c["offA"],
                     c["lda"], B, c["offB"], c["ldb"], c["beta"], C, c["offC"], c["ldc"])
    assert st == 0
    np.testing.assert_array_equal(C, np.array(c["expected"], dtype=dt))  # integers: exact


@pytest.mark.parametrize("solver", ["naive", "blocked"])
@pytest.mark.parametrize("name", ["sample_strsm_offsets", "extratest_f32", "extratest_f64"])
def test_trsm_golden(name, solver):
    c = golden_cases()[name]
    dt = DT[c["dtype"]]
    A, B = np.array(c["A"], dtype=dt), np.array(c["B"], dtype=dt)
    fn = oracle.trsm_naive if solver == "naive" else oracle.trsm_blocked
    st = fn(c["order"], c["side"], c["uplo"], c["transA"], c["diag"], c["M"], c["N"], c["alpha"], A, c["offA"],
            c["lda"], B, c["offB"], c["ldb"])
    assert st == 0
    exp = np.array(c["expected"], dtype=np.float64)
    tol = c.get("tol", 16 * np.finfo(dt).eps)
    np.testing.assert_allclose(B.astype(np.float64), exp, rtol=tol, atol=tol)


# ---------------------------------------------------------------- exact-integer GEMM
SHAPES = [(1, 1, 1), (2, 1, 3), (8, 16, 17), (17, 32, 62), (64, 33, 128), (65, 67, 5)]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("order", [ROW, COL])
@pytest.mark.parametrize("tA,tB", list(itertools.product([NOTRANS, TRANS, CONJ], [NOTRANS, TRANS])))
def test_gemm_integer_exact(dtype, order, tA, tB):
    for si, (M, N, K) in enumerate(SHAPES):
        alpha, beta = 3.0, -2.0
        la, lc = exact_int_limits(K, alpha, beta, dtype)
        offA, offB, offC = 5, 7, 11
        ia, oa = (M, K) if (order == COL) == (tA == NOTRANS) else (K, M)
        ib, ob = (K, N) if (order == COL) == (tB == NOTRANS) else (N, K)
        ic, oc = (M, N) if order == COL else (N, M)
        lda, ldb, ldc = ia + 3, ib + 2, ic + 1
        A = oracle.integers(offA + oa * lda, 100 + si, la, dtype)
        B = oracle.integers(offB + ob * ldb, 200 + si, la, dtype)
        C = oracle.integers(offC + oc * ldc, 300 + si, lc, dtype)
        C0 = C.copy()
        st = oracle.gemm(order, tA, tB, M, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc)
        assert st == 0
        Av = logical_view(A, order, tA, M, K, offA, lda).astype(np.int64)
        Bv = logical_view(B, order, tB, K, N, offB, ldb).astype(np.int64)
        Cv0 = logical_view(C0, order, NOTRANS, M, N, offC, ldc).astype(np.int64)
        want = int(alpha) * (Av @ Bv) + int(beta) * Cv0
        got = logical_view(C, order, NOTRANS, M, N, offC, ldc)
        np.testing.assert_array_equal(got.astype(np.int64), want)
        # nothing outside the M x N window may change
        mask = np.ones(C.size, dtype=bool)
        idx = logical_view(np.arange(C.size), order, NOTRANS, M, N, offC, ldc)
        mask[idx.ravel()] = False
        np.testing.assert_array_equal(C[mask], C0[mask])
        # the high-precision evaluator must reproduce exact data exactly
        if order == COL:
            rows, cols = np.meshgrid(np.arange(M), np.arange(N), indexing="ij")
            ex, mag = oracle.gemm_exact(tA != NOTRANS, tB != NOTRANS, K, alpha, A[offA:], lda, B[offB:], ldb, beta,
                                        C0[offC:], ldc, rows.ravel(), cols.ravel())
            np.testing.assert_array_equal(ex.reshape(M, N), want.astype(np.float64))
            assert np.all(mag.reshape(M, N) >= np.abs(want))


# ---------------------------------------------------------------- closed forms
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_gemm_closed_forms(dtype):
    n = 37
    X = oracle.uniform(n * n, 1, dtype)
    I = np.eye(n, dtype=dtype).ravel(order="F").copy()
    C = np.full(n * n, np.nan, dtype=dtype)
    # X * I with beta = 0: C is never read, so the NaNs must vanish and C == X bit for bit
    assert oracle.gemm(COL, NOTRANS, NOTRANS, n, n, n, 1.0, X, 0, n, I, 0, n, 0.0, C, 0, n) == 0
    np.testing.assert_array_equal(C, X)
    # alpha = 0, beta = 1 leaves C unchanged
    C1 = X.copy()
    assert oracle.gemm(COL, TRANS, NOTRANS, n, n, n, 0.0, X, 0, n, X, 0, n, 1.0, C1, 0, n) == 0
    np.testing.assert_array_equal(C1, X)
    # rank-1 with powers of two: u * v^T, every product exact, K = 1
    u = (2.0 ** np.arange(n)).astype(dtype)
    v = (2.0 ** -np.arange(n)).astype(dtype)
    C2 = np.zeros(n * n, dtype=dtype)
    assert oracle.gemm(COL, NOTRANS, NOTRANS, n, n, 1, 1.0, u, 0, n, v, 0, 1, 0.0, C2, 0, n) == 0
    np.testing.assert_array_equal(C2.reshape(n, n, order="F"), np.outer(u, v))
    # K == 0 with valid C: the checks pass (A, B not checked) -- xgemm.cc:691
    assert oracle.check_gemm(COL, NOTRANS, NOTRANS, 4, 4, 0, 1, 0, 1, 0, 1, 0, 1, 0, 1, 0, 4, 0) == 0


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_gemm_transpose_and_order_identities(dtype):
    M, N, K = 23, 19, 31
    A = oracle.uniform(M * K, 3, dtype).reshape(M, K)
    B = oracle.uniform(K * N, 4, dtype).reshape(K, N)
    C0 = oracle.uniform(M * N, 5, dtype).reshape(M, N)
    alpha, beta = 0.7, -1.3
    results = []
    for order, tA, tB in itertools.product([ROW, COL], [NOTRANS, TRANS], [NOTRANS, TRANS]):
        a = A if tA == NOTRANS else A.T
        b = B if tB == NOTRANS else B.T
        lay = "C" if order == ROW else "F"
        abuf, bbuf, cbuf = (x.ravel(order=lay).copy() for x in (a, b, C0))  # copies: C is updated in place
        lda = a.shape[1] if order == ROW else a.shape[0]
        ldb = b.shape[1] if order == ROW else b.shape[0]
        ldc = N if order == ROW else M
        assert oracle.gemm(order, tA, tB, M, N, K, alpha, abuf, 0, lda, bbuf, 0, ldb, beta, cbuf, 0, ldc) == 0
        results.append(cbuf.reshape(M, N, order=lay))
    # same logical problem, same k order per element: identical bits in all 8 layouts
    for r in results[1:]:
        np.testing.assert_array_equal(r, results[0])
    want = alpha * (A.astype(np.float64) @ B.astype(np.float64)) + beta * C0.astype(np.float64)
    mag = abs(alpha) * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64)) + abs(beta) * np.abs(C0)
    assert np.all(np.abs(results[0] - want) <= gemm_bound(K, mag, dtype, c=1.0))


# ---------------------------------------------------------------- against the reference's naive BLAS
needs_ref = pytest.mark.skipif(oracle.ref_lib() is None, reason="oracle/_ref not built (no reference tree)")


@needs_ref
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("order", [ROW, COL])
@pytest.mark.parametrize("tA,tB", list(itertools.product([NOTRANS, TRANS], [NOTRANS, TRANS])))
def test_gemm_vs_reference_naive(dtype, order, tA, tB):
    M, N, K = 45, 37, 53
    ia, oa = (M, K) if (order == COL) == (tA == NOTRANS) else (K, M)
    ib, ob = (K, N) if (order == COL) == (tB == NOTRANS) else (N, K)
    ic, oc = (M, N) if order == COL else (N, M)
    lda, ldb, ldc = ia + 2, ib + 1, ic + 3
    for exact in (True, False):
        if exact:
            la, lc = exact_int_limits(K, 2.0, 3.0, dtype)
            A, B, C = (oracle.integers(oa * lda, 1, la, dtype), oracle.integers(ob * ldb, 2, la, dtype),
                       oracle.integers(oc * ldc, 3, lc, dtype))
            alpha, beta = 2.0, 3.0
        else:
            A, B, C = (oracle.uniform(oa * lda, 1, dtype), oracle.uniform(ob * ldb, 2, dtype),
                       oracle.uniform(oc * ldc, 3, dtype))
            alpha, beta = 0.7, -1.3
        Cr = C.copy()
        oracle.ref_gemm(order, tA, tB, M, N, K, alpha, A, lda, B, ldb, beta, Cr, ldc)
        assert oracle.gemm(order, tA, tB, M, N, K, alpha, A, 0, lda, B, 0, ldb, beta, C, 0, ldc) == 0
        if exact:
            np.testing.assert_array_equal(C, Cr)
        else:
            Av = logical_view(A, order, tA, M, K, 0, lda).astype(np.float64)
            Bv = logical_view(B, order, tB, K, N, 0, ldb).astype(np.float64)
            C0 = logical_view(oracle.uniform(oc * ldc, 3, dtype), order, NOTRANS, M, N, 0, ldc).astype(np.float64)
            mag = abs(alpha) * (np.abs(Av) @ np.abs(Bv)) + abs(beta) * np.abs(C0)
            got = logical_view(C, order, NOTRANS, M, N, 0, ldc)
            ref = logical_view(Cr, order, NOTRANS, M, N, 0, ldc)
            assert np.all(np.abs(got.astype(np.float64) - ref) <= gemm_bound(K, mag, dtype))


def _trsm_inputs(order, side, uplo, diag, M, N, dtype, seed, poison=True):
    n = M if side == LEFT else N
    lda = n + 3
    # The generator writes a column-major triangle; in row-major memory the same bytes are
    # its transpose, so ask for the other triangle there.
    lower_in_memory = (uplo == LOWER) == (order == COL)
    A = oracle.triangular(n, lda, lower_in_memory, seed, dtype, poison_diag=(diag == UNIT and poison))
    if not poison:
        A = np.nan_to_num(A, nan=0.0)
    ib = M if order == COL else N
    ob = N if order == COL else M
    ldb = ib + 2
    B = oracle.uniform(ob * ldb, seed + 1, dtype)
    return A, lda, B, ldb


TRSM_VARIANTS = list(itertools.product([LEFT, RIGHT], [UPPER, LOWER], [NOTRANS, TRANS], [UNIT, NONUNIT]))


@needs_ref
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("order", [ROW, COL])
@pytest.mark.parametrize("side,uplo,tA,diag", TRSM_VARIANTS)
def test_trsm_naive_vs_reference_naive(dtype, order, side, uplo, tA, diag):
    M, N = 29, 21
    A, lda, B, ldb = _trsm_inputs(order, side, uplo, diag, M, N, dtype, 7)
    Br = B.copy()
    oracle.ref_trsm(order, side, uplo, tA, diag, M, N, 1.5, A, lda, Br, ldb)
    assert oracle.trsm_naive(order, side, uplo, tA, diag, M, N, 1.5, A, 0, lda, B, 0, ldb) == 0
    assert not np.isnan(logical_view(B, order, NOTRANS, M, N, 0, ldb)).any()
    # same operation sequence; only fma contraction may differ between the two builds
    np.testing.assert_allclose(B, Br, rtol=64 * np.finfo(dtype).eps, atol=64 * np.finfo(dtype).eps)


def _residual(order, side, uplo, tA, diag, M, N, alpha, A, lda, B0, X, ldb):
    """Normwise backward error  ||op(A) X - alpha B|| / (||A|| ||X|| + |alpha| ||B||)  (inf-norms)."""
    n = M if side == LEFT else N
    Am = logical_view(A, order, NOTRANS, n, n, 0, lda).astype(np.float64)
    Am = np.triu(np.nan_to_num(Am)) if uplo == UPPER else np.tril(np.nan_to_num(Am))
    if diag == UNIT:
        np.fill_diagonal(Am, 1.0)
    if tA != NOTRANS:
        Am = Am.T
    Xm = logical_view(X, order, NOTRANS, M, N, 0, ldb).astype(np.float64)
    Bm = logical_view(B0, order, NOTRANS, M, N, 0, ldb).astype(np.float64)
    R = (Am @ Xm if side == LEFT else Xm @ Am) - alpha * Bm
    nrm = lambda Z: np.abs(Z).sum(axis=1).max()
    return nrm(R) / (nrm(Am) * nrm(Xm) + abs(alpha) * nrm(Bm))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("order", [ROW, COL])
@pytest.mark.parametrize("side,uplo,tA,diag", TRSM_VARIANTS)
def test_trsm_blocked_all_variants(dtype, order, side, uplo, tA, diag):
    # sizes straddle the 16 / 128 blocking of the reference algorithm
    for (M, N) in [(5, 3), (37, 29), (130, 17), (23, 300)]:
        A, lda, B, ldb = _trsm_inputs(order, side, uplo, diag, M, N, dtype, 11)
        B0 = B.copy()
        Bn = B.copy()
        assert oracle.trsm_blocked(order, side, uplo, tA, diag, M, N, 0.75, A, 0, lda, B, 0, ldb) == 0
        assert oracle.trsm_naive(order, side, uplo, tA, diag, M, N, 0.75, A, 0, lda, Bn, 0, ldb) == 0
        Xb = logical_view(B, order, NOTRANS, M, N, 0, ldb)
        assert not np.isnan(Xb).any(), "poisoned triangle or unit diagonal was read"
        n = M if side == LEFT else N
        eps = np.finfo(dtype).eps
        assert _residual(order, side, uplo, tA, diag, M, N, 0.75, A, lda, B0, B, ldb) <= 4 * n * eps
        assert _residual(order, side, uplo, tA, diag, M, N, 0.75, A, lda, B0, Bn, ldb) <= 4 * n * eps
        np.testing.assert_allclose(Xb, logical_view(Bn, order, NOTRANS, M, N, 0, ldb), rtol=64 * n * eps,
                                   atol=64 * n * eps)
        # padding of B untouched
        mask = np.ones(B.size, dtype=bool)
        mask[logical_view(np.arange(B.size), order, NOTRANS, M, N, 0, ldb).ravel()] = False
        np.testing.assert_array_equal(B[mask], B0[mask])


def test_trsm_blocked_zero_diagonal_becomes_one():
    # trtri/diag_dtrtri_lower_128_16.cpp:93-96: a zero diagonal entry is inverted as 1
    n = 4
    A = np.array([[2, 0, 0, 0], [1, 0, 0, 0], [1, 1, 4, 0], [1, 1, 1, 8]], dtype=np.float64)
    A1 = A.copy()
    A1[1, 1] = 1.0
    B = np.arange(1, n * 2 + 1, dtype=np.float64)
    Ba, Bb = B.copy(), B.copy()
    assert oracle.trsm_blocked(COL, LEFT, LOWER, NOTRANS, NONUNIT, n, 2, 1.0, A.ravel(order="F").copy(), 0, n, Ba, 0,
                               n) == 0
    assert oracle.trsm_blocked(COL, LEFT, LOWER, NOTRANS, NONUNIT, n, 2, 1.0, A1.ravel(order="F").copy(), 0, n, Bb,
                               0, n) == 0
    np.testing.assert_array_equal(Ba, Bb)
    assert np.isfinite(Ba).all()


# ---------------------------------------------------------------- argument checks
def test_check_tables():
    ok = dict(haveA=1, offA=0, lda=8, memA=0, haveB=1, offB=0, ldb=8, memB=0, haveC=1, offC=0, ldc=8, memC=0)
    def g(order=COL, tA=NOTRANS, tB=NOTRANS, M=8, N=8, K=8, **kw):
        a = dict(ok); a.update(kw)
        return oracle.check_gemm(order, tA, tB, M, N, K, a["haveA"], a["offA"], a["lda"], a["memA"], a["haveB"],
                                 a["offB"], a["ldb"], a["memB"], a["haveC"], a["offC"], a["ldc"], a["memC"])
    assert g() == 0
    # func-error.cpp:58-104: invalid objects in A, B, C order
    assert g(haveA=0, haveB=0, haveC=0) == -1022
    assert g(haveB=0, haveC=0) == -1021
    assert g(haveC=0) == -1020
    assert g(M=0) == -1017 and g(N=0) == -1017
    assert g(K=0, lda=1, ldb=1) == 0          # A, B not checked when K == 0 (xgemm.cc:691)
    assert g(lda=7) == -1016 and g(ldb=7) == -1015 and g(ldc=7) == -1014
    assert g(lda=7, ldb=7, ldc=7) == -1016    # first failing check wins
    assert g(tA=TRANS, M=4, lda=7) == -1016   # transposed A is K x M in memory: lda >= K
    assert g(tA=TRANS, M=4, K=4, lda=4) == 0
    assert g(order=ROW, M=4, lda=8, ldc=8) == 0 and g(order=ROW, K=9, lda=8) == -1016
    # too-small buffers (func-error.cpp: clblasInsufficientMemMatA ...)
    assert g(memA=63) == -1011 and g(memA=64) == 0 and g(offA=1, memA=64) == -1011
    assert g(memB=10) == -1010 and g(memC=10) == -1009
    def t(order=COL, side=LEFT, tA=NOTRANS, M=8, N=4, haveA=1, offA=0, lda=8, memA=0, haveB=1, offB=0, ldb=8,
          memB=0):
        return oracle.check_trsm(order, side, tA, M, N, haveA, offA, lda, memA, haveB, offB, ldb, memB)
    assert t() == 0
    assert t(haveA=0, haveB=0) == -1022 and t(haveB=0) == -1021
    assert t(M=0) == -1017
    assert t(lda=7) == -1016 and t(ldb=7) == -1015
    assert t(side=RIGHT, lda=4) == 0 and t(side=RIGHT, lda=3) == -1016   # A is N x N on the right
    assert t(order=ROW, ldb=4) == 0 and t(order=ROW, ldb=3) == -1015
    assert t(memA=63) == -1011 and t(memB=31) == -1010


def test_generators_are_reproducible():
    a = oracle.uniform(1000, 42, np.float32)
    b = oracle.uniform(1000, 42, np.float32)
    np.testing.assert_array_equal(a, b)
    assert a.min() >= -1.0 and a.max() < 1.0 and abs(a.mean()) < 0.1
    g = oracle.normal(20000, 9, np.float64)
    assert abs(g.mean()) < 0.05 and abs(g.std() - 1.0) < 0.05
    # a prefix of a longer draw is the shorter draw (counter-based generator)
    np.testing.assert_array_equal(oracle.uniform(4, 1, np.float64), oracle.uniform(8, 1, np.float64)[:4])
    t = oracle.triangular(6, 8, True, 3, np.float64)
    T = t.reshape(6, 8).T[:6, :6]
    assert np.isnan(np.triu(T, 1)[np.triu_indices(6, 1)]).all()
    assert (np.diag(T) >= 1).all() and (np.diag(T) < 2).all()
    assert (np.abs(np.tril(T, -1)) <= 1 / 6).all()


def test_generators_match_the_committed_fixtures():
    """First / last values and a hash of the bytes of every seeded generator, as committed in
    tests/golden/generator_fixtures.json (written by tests/golden/make_generator_fixtures.py): the
    inputs of every seeded parity test are pinned to what they were when the tests were written."""
    import importlib.util
    import json
    import os
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    spec = importlib.util.spec_from_file_location("make_generator_fixtures", os.path.join(here, "make_generator_fixtures.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    fixtures = json.load(open(os.path.join(here, "generator_fixtures.json")))
    assert len(fixtures) == len(mod.CASES)
    for fx in fixtures:
        got = mod.describe(mod.generate(fx["generator"], fx["args"]))
        for key in ("count", "first8", "last8", "sha256"):
            assert got[key] == fx[key], (fx["generator"], fx["args"], key)
