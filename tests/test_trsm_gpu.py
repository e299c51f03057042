"""GPU parity tests for clblasStrsm / clblasDtrsm through the C ABI.

The reference solves with explicit inverses of 128x128 diagonal blocks; this library solves
the diagonal blocks by substitution.  The two are not bit-comparable, so parity is judged as
the task states: normwise backward error
    ||op(A) X - alpha B|| / (||A|| ||X|| + |alpha| ||B||) <= 2 n eps        (inf-norms)
plus elementwise agreement with the oracle's restatement of the reference algorithm within
a forward bound for these well-conditioned inputs, plus the reference tests' own devices:
NaN-poisoned unused triangle / unit diagonal, closed-form Extratest, untouched padding."""
import itertools

import numpy as np
import pytest

import oracle
from helpers import (COL, ROW, NOTRANS, TRANS, CONJ, UPPER, LOWER, UNIT, NONUNIT, LEFT, RIGHT, golden_cases,
                     logical_view)

pytestmark = pytest.mark.gpu

DT = {"f32": np.float32, "f64": np.float64}


@pytest.fixture(scope="module")
def gpu():
    import gpu_util
    import torch
    assert torch.cuda.is_available()
    return gpu_util


@pytest.mark.parametrize("name", ["sample_strsm_offsets", "extratest_f32", "extratest_f64"])
def test_golden(gpu, name):
    c = golden_cases()[name]
    dt = DT[c["dtype"]]
    A, B = np.array(c["A"], dtype=dt), np.array(c["B"], dtype=dt)
    st, out = gpu.trsm(c["order"], c["side"], c["uplo"], c["transA"], c["diag"], c["M"], c["N"], c["alpha"], A,
                       c["offA"], c["lda"], B, c["offB"], c["ldb"])
    assert st == 0
    tol = c.get("tol", 16 * np.finfo(dt).eps)   # Extratest: the reference's own 1e-5
    np.testing.assert_allclose(out.astype(np.float64), np.array(c["expected"]), rtol=tol, atol=tol)


def make_inputs(order, side, uplo, diag, M, N, dtype, seed, offA=5, offB=7):
    n = M if side == LEFT else N
    lda = n + 3
    lower_in_memory = (uplo == LOWER) == (order == COL)
    A = oracle.triangular(n, lda, lower_in_memory, seed, dtype, poison_diag=(diag == UNIT))
    A = np.concatenate([np.full(offA, np.nan, dtype=dtype), A])
    ib, ob = (M, N) if order == COL else (N, M)
    ldb = ib + 2
    B = oracle.uniform(offB + ob * ldb, seed + 1, dtype)
    return A, lda, B, ldb


def backward_error(order, side, uplo, tA, diag, M, N, alpha, A, offA, lda, B0, X, offB, ldb):
    n = M if side == LEFT else N
    Am = np.nan_to_num(logical_view(A, order, NOTRANS, n, n, offA, lda).astype(np.float64))
    Am = np.triu(Am) if uplo == UPPER else np.tril(Am)
    if diag == UNIT:
        np.fill_diagonal(Am, 1.0)
    if tA != NOTRANS:
        Am = Am.T
    Xm = logical_view(X, order, NOTRANS, M, N, offB, ldb).astype(np.float64)
    Bm = logical_view(B0, order, NOTRANS, M, N, offB, ldb).astype(np.float64)
    R = (Am @ Xm if side == LEFT else Xm @ Am) - alpha * Bm
    nrm = lambda Z: np.abs(Z).sum(axis=1).max()
    return nrm(R) / (nrm(Am) * nrm(Xm) + abs(alpha) * nrm(Bm))


VARIANTS = list(itertools.product([LEFT, RIGHT], [UPPER, LOWER], [NOTRANS, TRANS], [UNIT, NONUNIT]))
SIZES = [(1, 1), (5, 3), (37, 29), (130, 17), (23, 300), (257, 64), (300, 520), (512, 33), (513, 40), (48, 1030),
         (3000, 1), (1, 3000), (2049, 2), (2, 2049),
         # more than 4096 right-hand sides: the leaf takes 32 of them per workgroup
         (37, 4130), (4130, 29), (530, 4100)]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("order", [ROW, COL])
@pytest.mark.parametrize("side,uplo,tA,diag", VARIANTS)
def test_all_variants(gpu, dtype, order, side, uplo, tA, diag):
    eps = np.finfo(dtype).eps
    for (M, N) in SIZES:
        alpha = 0.75
        A, lda, B, ldb = make_inputs(order, side, uplo, diag, M, N, dtype, 11)
        want = B.copy()
        assert oracle.trsm_blocked(order, side, uplo, tA, diag, M, N, alpha, A, 5, lda, want, 7, ldb) == 0
        st, got = gpu.trsm(order, side, uplo, tA, diag, M, N, alpha, A, 5, lda, B, 7, ldb)
        assert st == 0
        n = M if side == LEFT else N
        Xg = logical_view(got, order, NOTRANS, M, N, 7, ldb)
        assert not np.isnan(Xg).any(), "poisoned triangle or unit diagonal was read (%d,%d)" % (M, N)
        be = backward_error(order, side, uplo, tA, diag, M, N, alpha, A, 5, lda, B, got, 7, ldb)
        assert be <= 2 * n * eps, ((M, N), be)
        Xw = logical_view(want, order, NOTRANS, M, N, 7, ldb)
        scale = np.abs(Xw).max()
        assert np.abs(Xg - Xw).max() <= 32 * n * eps * scale, (M, N)
        mask = np.ones(B.size, dtype=bool)
        logical_view(mask, order, NOTRANS, M, N, 7, ldb)[:] = False
        np.testing.assert_array_equal(got[mask], B[mask])


def test_conjtrans_is_trans_and_alpha_zero(gpu):
    M, N = 70, 33
    A, lda, B, ldb = make_inputs(COL, LEFT, LOWER, NONUNIT, M, N, np.float64, 3)
    st, x1 = gpu.trsm(COL, LEFT, LOWER, TRANS, NONUNIT, M, N, 1.0, A, 5, lda, B, 7, ldb)
    st2, x2 = gpu.trsm(COL, LEFT, LOWER, CONJ, NONUNIT, M, N, 1.0, A, 5, lda, B, 7, ldb)
    assert st == 0 and st2 == 0
    np.testing.assert_array_equal(x1, x2)
    st, x0 = gpu.trsm(COL, LEFT, LOWER, NOTRANS, NONUNIT, M, N, 0.0, A, 5, lda, B, 7, ldb)
    assert st == 0
    assert (logical_view(x0, COL, NOTRANS, M, N, 7, ldb) == 0).all()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_repeated_calls_give_the_same_bits(gpu, dtype):
    """The leaf's wavefronts run at their own pace (flags, no barriers), and which X a wavefront finds
    published first differs from run to run: the order of summation must not."""
    for (side, uplo, tA, M, N) in [(LEFT, LOWER, NOTRANS, 1100, 530), (LEFT, UPPER, TRANS, 520, 4200),
                                   (RIGHT, UPPER, NOTRANS, 300, 1500), (RIGHT, LOWER, TRANS, 4200, 600)]:
        A, lda, B, ldb = make_inputs(COL, side, uplo, NONUNIT, M, N, dtype, 5)
        st, first = gpu.trsm(COL, side, uplo, tA, NONUNIT, M, N, 1.0, A, 5, lda, B, 7, ldb)
        assert st == 0
        for _ in range(3):
            st, again = gpu.trsm(COL, side, uplo, tA, NONUNIT, M, N, 1.0, A, 5, lda, B, 7, ldb)
            assert st == 0
            np.testing.assert_array_equal(again, first, err_msg=str((side, uplo, tA, M, N)))


def test_config5_dtrsm_8192(gpu):
    """BASELINE config 5 at full size: Left/Lower/NoTrans/NonUnit, M=N=8192, alpha=1.
    (a) backward error on sampled right-hand sides, computed in fp64 on the host;
    (b) size-independent: the leading 1024 rows of X solve the leading 1024x1024 system, so
        they must agree with the oracle's solve of that sub-problem."""
    import torch
    import clblas_amd
    n = 8192
    A = oracle.triangular(n, n, True, 21, np.float64)
    B = oracle.normal(n * n, 22, np.float64)
    dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    st = clblas_amd.dtrsm(COL, LEFT, LOWER, NOTRANS, NONUNIT, n, n, 1.0, dA, 0, n, dB, 0, n)
    torch.cuda.synchronize()
    assert st == 0
    X = dB.cpu().numpy().reshape(n, n).T        # X[r, c]
    assert np.isfinite(X).all()
    L = np.tril(np.nan_to_num(A.reshape(n, n).T))
    B0 = B.reshape(n, n).T
    cols = np.r_[0, 1, 63, 64, 4095, 4096, 8190, 8191, np.random.default_rng(0).integers(0, n, 24)]
    R = L @ X[:, cols] - B0[:, cols]
    nrm_L = np.abs(L).sum(axis=1).max()
    be = np.abs(R).max(axis=0) / (nrm_L * np.abs(X[:, cols]).max(axis=0) + np.abs(B0[:, cols]).max(axis=0))
    assert be.max() <= 2 * n * np.finfo(np.float64).eps, be.max()
    k, nc = 1024, 96
    sub = np.ascontiguousarray(B0[:k, :nc].T).ravel()            # column-major k x nc
    Asub = np.ascontiguousarray(A.reshape(n, n)[:k, :k]).ravel()  # columns 0..k-1, rows 0..k-1, ld k
    assert oracle.trsm_blocked(COL, LEFT, LOWER, NOTRANS, NONUNIT, k, nc, 1.0, Asub, 0, k, sub, 0, k) == 0
    want = sub.reshape(nc, k).T
    assert np.abs(X[:k, :nc] - want).max() <= 32 * k * np.finfo(np.float64).eps * np.abs(want).max()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_several_rounds_of_leaf_workgroups(gpu, dtype):
    """More right-hand sides than one round of leaf workgroups takes, in the ranges where the launch is priced
    for 16 per workgroup (8193 .. 12288: three rounds) and for 32 (12289 .. 16384: two rounds), both sides,
    a diagonal block and a half; and each width forced on the other's range (CLBLAS_AMD_TRSM_WIDE).  Same
    bars as test_all_variants."""
    eps = np.finfo(dtype).eps
    cases = [(LEFT, 40, 8300), (LEFT, 530, 8300), (RIGHT, 8300, 40), (RIGHT, 8300, 530), (LEFT, 40, 12500),
             (RIGHT, 12500, 40)]
    for ci, (side, M, N) in enumerate(cases):
        uplo, tA, diag = [(LOWER, NOTRANS, NONUNIT), (UPPER, TRANS, NONUNIT), (UPPER, NOTRANS, UNIT)][ci % 3]
        order = COL if ci % 2 == 0 else ROW
        alpha = 0.75
        A, lda, B, ldb = make_inputs(order, side, uplo, diag, M, N, dtype, 17)
        want = B.copy()
        assert oracle.trsm_blocked(order, side, uplo, tA, diag, M, N, alpha, A, 5, lda, want, 7, ldb) == 0
        n = M if side == LEFT else N
        Xw = logical_view(want, order, NOTRANS, M, N, 7, ldb)
        for forced in (None, 0, 1):
            env = {} if forced is None else {"CLBLAS_AMD_TRSM_WIDE": forced}
            with gpu.debug_env(**env):
                st, got = gpu.trsm(order, side, uplo, tA, diag, M, N, alpha, A, 5, lda, B, 7, ldb)
            assert st == 0
            Xg = logical_view(got, order, NOTRANS, M, N, 7, ldb)
            assert not np.isnan(Xg).any(), "poisoned triangle or unit diagonal was read (%d,%d)" % (M, N)
            be = backward_error(order, side, uplo, tA, diag, M, N, alpha, A, 5, lda, B, got, 7, ldb)
            assert be <= 2 * n * eps, ((M, N), forced, be)
            assert np.abs(Xg - Xw).max() <= 32 * n * eps * np.abs(Xw).max(), (M, N, forced)
            mask = np.ones(B.size, dtype=bool)
            logical_view(mask, order, NOTRANS, M, N, 7, ldb)[:] = False
            np.testing.assert_array_equal(got[mask], B[mask])


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("order", [ROW, COL])
def test_inverted_triangle_leaf_behind_its_switch(gpu, dtype, order):
    """The other way of solving a diagonal block (real types): 64 x 64 triangles inverted by doubling in the
    packing pass - as the reference inverts its 128 x 128 ones - and a leaf of eight steps between barriers
    (CLBLAS_AMD_TRSM_LEAF=1).  Same bars as test_all_variants, nothing widened, on a spread of the variants
    and sizes (short last blocks, 16 and 32 right-hand sides per workgroup, both sides); bit-identical
    when repeated."""
    eps = np.finfo(dtype).eps
    sizes = [(5, 3), (130, 17), (257, 64), (513, 40), (48, 1030), (1100, 530), (37, 4130), (4130, 29)]
    with gpu.debug_env(CLBLAS_AMD_TRSM_LEAF=1):
        for vi, (side, uplo, tA, diag) in enumerate(VARIANTS):
            for (M, N) in sizes[vi % 2::2]:
                alpha = 0.75
                A, lda, B, ldb = make_inputs(order, side, uplo, diag, M, N, dtype, 13)
                want = B.copy()
                assert oracle.trsm_blocked(order, side, uplo, tA, diag, M, N, alpha, A, 5, lda, want, 7, ldb) == 0
                st, got = gpu.trsm(order, side, uplo, tA, diag, M, N, alpha, A, 5, lda, B, 7, ldb)
                assert st == 0
                n = M if side == LEFT else N
                Xg = logical_view(got, order, NOTRANS, M, N, 7, ldb)
                assert not np.isnan(Xg).any(), "poisoned triangle or unit diagonal was read (%d,%d)" % (M, N)
                be = backward_error(order, side, uplo, tA, diag, M, N, alpha, A, 5, lda, B, got, 7, ldb)
                assert be <= 2 * n * eps, ((M, N), be)
                Xw = logical_view(want, order, NOTRANS, M, N, 7, ldb)
                assert np.abs(Xg - Xw).max() <= 32 * n * eps * np.abs(Xw).max(), (M, N)
                mask = np.ones(B.size, dtype=bool)
                logical_view(mask, order, NOTRANS, M, N, 7, ldb)[:] = False
                np.testing.assert_array_equal(got[mask], B[mask])
                if vi % 5 == 0:
                    st, again = gpu.trsm(order, side, uplo, tA, diag, M, N, alpha, A, 5, lda, B, 7, ldb)
                    assert st == 0
                    np.testing.assert_array_equal(again, got)
