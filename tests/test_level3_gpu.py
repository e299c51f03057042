"""GPU parity tests for clblas{S,D,C,Z}{syrk,trmm,symm} through the C ABI, against the CPU
oracle.

Bars: exact equality on exact-integer inputs (every tile of the table forced in turn, unused
triangles NaN-poisoned, everything outside the result untouched bit for bit); for real-valued
data the K*eps bound of the GEMM tests with K = the summation depth; at 4096 the routines are
checked against this library's own (separately pinned) GEMM on explicitly masked / symmetrised
operands."""
import itertools

import numpy as np
import pytest

import oracle
from helpers import COL, ROW, NOTRANS, TRANS, CONJ, UPPER, LOWER, UNIT, NONUNIT, LEFT, RIGHT, logical_view
from l3_util import (ALL, REAL, CPLX, abs1, bound, err, is_cplx, matrix, nan_of, op, poison_triangle, real_scalars,
                     scalars, sym_dense, tri_dense, tri_mask)

pytestmark = pytest.mark.gpu
N_TILES = {np.dtype(np.float32): 7, np.dtype(np.float64): 4, np.dtype(np.complex64): 4, np.dtype(np.complex128): 4}
WIDE = lambda dt: np.complex128 if is_cplx(dt) else np.float64


@pytest.fixture(scope="module")
def gpu():
    import gpu_util
    import torch
    assert torch.cuda.is_available()
    import clblas_amd
    assert clblas_amd.setup() == 0
    return gpu_util


def tiles(dtype):
    return [None] + list(range(N_TILES[np.dtype(dtype)]))


# ------------------------------------------------------------------------------- SYRK
@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("order,uplo,trans", list(itertools.product([ROW, COL], [UPPER, LOWER], [NOTRANS, TRANS])))
def test_syrk_integer_exact_all_tiles(gpu, dtype, order, uplo, trans):
    alpha, beta = scalars(dtype)
    for si, (N, K) in enumerate([(1, 1), (5, 3), (64, 20), (70, 129), (257, 33), (300, 130), (513, 17)]):
        rows, cols = (N, K) if trans == NOTRANS else (K, N)
        A, lda = matrix(order, rows, cols, 5, 3, 10 + si, dtype, True)
        C, ldc = matrix(order, N, N, 7, 2, 20 + si, dtype, True)
        keep = tri_mask(N, uplo == LOWER)
        logical_view(C, order, NOTRANS, N, N, 7, ldc)[~keep] = nan_of(dtype)
        want = C.copy()
        assert oracle.syrk(order, uplo, trans, N, K, alpha, A, 5, lda, beta, want, 7, ldc) == 0
        for tile in tiles(dtype):
            st, got = gpu.syrk(order, uplo, trans, N, K, alpha, A, 5, lda, beta, C, 7, ldc, tile=tile)
            assert st == 0
            np.testing.assert_array_equal(got.view(np.uint8), want.view(np.uint8),
                                          err_msg="N=%d K=%d tile %s" % (N, K, tile))


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("order,uplo,trans", list(itertools.product([ROW, COL], [UPPER, LOWER], [NOTRANS, TRANS])))
def test_syrk_small_c_deep_k_integer_exact(gpu, dtype, order, uplo, trans):
    """A small C from operands thousands deep runs as a plain product with a K split into a scratch
    square and a pass that folds the wanted triangle into C: the other triangle of C (NaN here) and
    everything around it stay untouched."""
    alpha, beta = scalars(dtype)
    for si, (N, K) in enumerate([(64, 5000), (300, 4100), (704, 4096)] if not is_cplx(dtype) else [(64, 5000), (200, 4100)]):
        rows, cols = (N, K) if trans == NOTRANS else (K, N)
        A, lda = matrix(order, rows, cols, 5, 3, 60 + si, dtype, True, limit=4)
        C, ldc = matrix(order, N, N, 7, 2, 70 + si, dtype, True)
        keep = tri_mask(N, uplo == LOWER)
        logical_view(C, order, NOTRANS, N, N, 7, ldc)[~keep] = nan_of(dtype)
        want = C.copy()
        assert oracle.syrk(order, uplo, trans, N, K, alpha, A, 5, lda, beta, want, 7, ldc) == 0
        st, got = gpu.syrk(order, uplo, trans, N, K, alpha, A, 5, lda, beta, C, 7, ldc)
        assert st == 0
        np.testing.assert_array_equal(got.view(np.uint8), want.view(np.uint8), err_msg="N=%d K=%d" % (N, K))


@pytest.mark.parametrize("dtype", ALL)
def test_syrk_uniform_data(gpu, dtype):
    alpha, beta = real_scalars(dtype)
    for uplo, trans, (N, K) in [(LOWER, NOTRANS, (700, 513)), (UPPER, TRANS, (1031, 300)), (LOWER, TRANS, (129, 2048))]:
        rows, cols = (N, K) if trans == NOTRANS else (K, N)
        A, lda = matrix(COL, rows, cols, 0, 1, 1, dtype, False)
        C, ldc = matrix(COL, N, N, 0, 3, 2, dtype, False)
        st, got = gpu.syrk(COL, uplo, trans, N, K, alpha, A, 0, lda, beta, C, 0, ldc)
        assert st == 0
        Aop = op(logical_view(A, COL, NOTRANS, rows, cols, 0, lda).astype(WIDE(dtype)), trans if trans != CONJ else TRANS)
        C0 = logical_view(C, COL, NOTRANS, N, N, 0, ldc).astype(WIDE(dtype))
        al, be = (complex(dtype(alpha)), complex(dtype(beta))) if is_cplx(dtype) else (float(dtype(alpha)), float(dtype(beta)))
        want = al * (Aop @ Aop.T) + be * C0
        mag = abs1(np.asarray(al)) * (abs1(Aop) @ abs1(Aop).T) + abs1(np.asarray(be)) * abs1(C0)
        keep = tri_mask(N, uplo == LOWER)
        gv = logical_view(got, COL, NOTRANS, N, N, 0, ldc)
        assert np.all(err(gv.astype(WIDE(dtype)), want)[keep] <= bound(K, mag, dtype)[keep])
        np.testing.assert_array_equal(gv[~keep], logical_view(C, COL, NOTRANS, N, N, 0, ldc)[~keep])
        # beta == 0 with a NaN-filled C: the triangle comes out finite, the rest stays NaN
        Cn = np.full(C.size, nan_of(dtype), dtype=dtype)
        st, got = gpu.syrk(COL, uplo, trans, N, K, alpha, A, 0, lda, 0, Cn, 0, ldc)
        gv = logical_view(got, COL, NOTRANS, N, N, 0, ldc)
        assert st == 0 and np.isfinite(gv[keep].real).all() and np.isnan(gv[~keep].real).all()


# ------------------------------------------------------------------------------- TRMM
TRMM_CASES = list(itertools.product([LEFT, RIGHT], [UPPER, LOWER], [NOTRANS, TRANS, CONJ], [UNIT, NONUNIT]))


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("order", [ROW, COL])
@pytest.mark.parametrize("side,uplo,trans,diag", TRMM_CASES)
def test_trmm_integer_exact_all_tiles(gpu, dtype, order, side, uplo, trans, diag):
    alpha, _ = scalars(dtype)
    for si, (M, N) in enumerate([(1, 1), (3, 7), (33, 20), (70, 45), (257, 130), (140, 300)]):
        n = M if side == LEFT else N
        A, lda = matrix(order, n, n, 5, 3, 30 + si, dtype, True, limit=4)
        poison_triangle(A, order, n, 5, lda, uplo, unit=diag == UNIT)
        B, ldb = matrix(order, M, N, 7, 2, 40 + si, dtype, True, limit=4)
        want = B.copy()
        assert oracle.trmm(order, side, uplo, trans, diag, M, N, alpha, A, 5, lda, want, 7, ldb) == 0
        for tile in tiles(dtype):
            st, got = gpu.trmm(order, side, uplo, trans, diag, M, N, alpha, A, 5, lda, B, 7, ldb, tile=tile)
            assert st == 0
            np.testing.assert_array_equal(got, want, err_msg="M=%d N=%d tile %s" % (M, N, tile))


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("side,uplo,trans,diag", TRMM_CASES)
def test_trmm_uniform_data(gpu, dtype, side, uplo, trans, diag):
    alpha, _ = real_scalars(dtype)
    M, N = (700, 300) if side == LEFT else (300, 700)
    n = M if side == LEFT else N
    A, lda = matrix(COL, n, n, 0, 1, 3, dtype, False)
    poison_triangle(A, COL, n, 0, lda, uplo, unit=diag == UNIT)
    B, ldb = matrix(COL, M, N, 0, 2, 4, dtype, False)
    st, got = gpu.trmm(COL, side, uplo, trans, diag, M, N, alpha, A, 0, lda, B, 0, ldb)
    assert st == 0
    T = op(tri_dense(A, COL, n, 0, lda, uplo, diag == UNIT), trans)
    Bv = logical_view(B, COL, NOTRANS, M, N, 0, ldb).astype(T.dtype)
    al = complex(dtype(alpha)) if is_cplx(dtype) else float(dtype(alpha))
    want = al * (T @ Bv if side == LEFT else Bv @ T)
    mag = abs1(np.asarray(al)) * (abs1(T) @ abs1(Bv) if side == LEFT else abs1(Bv) @ abs1(T))
    gv = logical_view(got, COL, NOTRANS, M, N, 0, ldb).astype(T.dtype)
    assert np.all(err(gv, want) <= bound(n, mag, dtype))
    pad = np.arange(B.size).reshape(-1, ldb)[:, M:].ravel()
    np.testing.assert_array_equal(got[pad], B[pad])


@pytest.mark.parametrize("dtype", REAL)
def test_trmm_then_trsm_round_trip_4096(gpu, dtype):
    """B -> op(A) B -> op(A)^-1 (op(A) B) == B at the size class of the headline runs."""
    import clblas_amd
    import torch
    n = 4096
    A = oracle.triangular(n, n, True, 3, dtype)
    B0 = oracle.uniform(n * n, 4, dtype)
    dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B0).cuda()
    p = "S" if dtype == np.float32 else "D"
    trsm = clblas_amd.strsm if dtype == np.float32 else clblas_amd.dtrsm
    for side, trans in ((LEFT, NOTRANS), (RIGHT, TRANS)):
        dB.copy_(torch.from_numpy(B0))
        assert clblas_amd.trmm(p, COL, side, LOWER, trans, NONUNIT, n, n, 1.0, dA, 0, n, dB, 0, n) == 0
        assert trsm(COL, side, LOWER, trans, NONUNIT, n, n, 1.0, dA, 0, n, dB, 0, n) == 0
        torch.cuda.synchronize()
        back = dB.cpu().numpy()
        assert np.abs(back - B0).max() <= 256 * n * np.finfo(dtype).eps


# ------------------------------------------------------------------------------- SYMM
@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("order,side,uplo", list(itertools.product([ROW, COL], [LEFT, RIGHT], [UPPER, LOWER])))
def test_symm_integer_exact_all_tiles(gpu, dtype, order, side, uplo):
    alpha, beta = scalars(dtype)
    for si, (M, N) in enumerate([(1, 1), (3, 7), (33, 20), (70, 45), (257, 130), (140, 300)]):
        n = M if side == LEFT else N
        A, lda = matrix(order, n, n, 5, 3, 50 + si, dtype, True)
        poison_triangle(A, order, n, 5, lda, uplo)
        B, ldb = matrix(order, M, N, 7, 2, 60 + si, dtype, True)
        C, ldc = matrix(order, M, N, 11, 1, 70 + si, dtype, True)
        want = C.copy()
        assert oracle.symm(order, side, uplo, M, N, alpha, A, 5, lda, B, 7, ldb, beta, want, 11, ldc) == 0
        for tile in tiles(dtype):
            st, got = gpu.symm(order, side, uplo, M, N, alpha, A, 5, lda, B, 7, ldb, beta, C, 11, ldc, tile=tile)
            assert st == 0
            np.testing.assert_array_equal(got, want, err_msg="M=%d N=%d tile %s" % (M, N, tile))


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("side,uplo", list(itertools.product([LEFT, RIGHT], [UPPER, LOWER])))
def test_symm_uniform_data(gpu, dtype, side, uplo):
    alpha, beta = real_scalars(dtype)
    M, N = (700, 300) if side == LEFT else (300, 700)
    n = M if side == LEFT else N
    A, lda = matrix(COL, n, n, 0, 1, 5, dtype, False)
    poison_triangle(A, COL, n, 0, lda, uplo)
    B, ldb = matrix(COL, M, N, 0, 2, 6, dtype, False)
    C, ldc = matrix(COL, M, N, 0, 3, 7, dtype, False)
    st, got = gpu.symm(COL, side, uplo, M, N, alpha, A, 0, lda, B, 0, ldb, beta, C, 0, ldc)
    assert st == 0
    S = sym_dense(A, COL, n, 0, lda, uplo)
    Bv = logical_view(B, COL, NOTRANS, M, N, 0, ldb).astype(S.dtype)
    C0 = logical_view(C, COL, NOTRANS, M, N, 0, ldc).astype(S.dtype)
    al, be = (complex(dtype(alpha)), complex(dtype(beta))) if is_cplx(dtype) else (float(dtype(alpha)), float(dtype(beta)))
    want = al * (S @ Bv if side == LEFT else Bv @ S) + be * C0
    mag = abs1(np.asarray(al)) * (abs1(S) @ abs1(Bv) if side == LEFT else abs1(Bv) @ abs1(S)) + abs1(np.asarray(be)) * abs1(C0)
    gv = logical_view(got, COL, NOTRANS, M, N, 0, ldc).astype(S.dtype)
    assert np.all(err(gv, want) <= bound(n, mag, dtype))
    Cn = np.full(C.size, nan_of(dtype), dtype=dtype)
    st, got = gpu.symm(COL, side, uplo, M, N, alpha, A, 0, lda, B, 0, ldb, 0, Cn, 0, ldc)
    assert st == 0 and np.isfinite(logical_view(got, COL, NOTRANS, M, N, 0, ldc).real).all()


# ------------------------------------------------------------------- 4096: against the pinned GEMM
@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.complex64])
def test_level3_matches_gemm_on_explicit_operands_4096(gpu, dtype):
    import clblas_amd
    import torch
    n = 4096
    p = {np.float32: "S", np.float64: "D", np.complex64: "C"}[dtype]
    gemm = {np.float32: clblas_amd.sgemm, np.float64: clblas_amd.dgemm, np.complex64: clblas_amd.cgemm}[dtype]
    alpha, beta = real_scalars(dtype)
    A = torch.from_numpy(oracle.uniform(n * n, 1, dtype)).cuda()
    B = torch.from_numpy(oracle.uniform(n * n, 2, dtype)).cuda()
    C0 = torch.from_numpy(oracle.uniform(n * n, 3, dtype)).cuda()
    Am = A.view(n, n).T  # Am[i, j] = element (i, j) of the column-major matrix
    tol = 64 * n * np.finfo(dtype).eps
    lower = torch.ones(n, n, dtype=torch.bool, device="cuda").tril()

    def colmajor(x):  # logical matrix -> flat column-major buffer
        return x.T.contiguous().view(-1)

    # SYRK lower == GEMM(A, A^T) on the lower triangle; the upper triangle is untouched
    C = C0.clone()
    Cg = C0.clone()
    assert clblas_amd.syrk(p, COL, LOWER, NOTRANS, n, n, alpha, A, 0, n, beta, C, 0, n) == 0
    assert gemm(COL, NOTRANS, TRANS, n, n, n, alpha, A, 0, n, A, 0, n, beta, Cg, 0, n) == 0
    d = (C.view(n, n).T - Cg.view(n, n).T).abs()
    assert d[lower].max().item() <= tol
    assert torch.equal(C.view(n, n).T[~lower], C0.view(n, n).T[~lower])
    # TRMM left/upper/trans/unit == GEMM with the explicit unit-upper matrix
    Tm = torch.where(lower.T, Am, torch.zeros_like(Am))
    Tm.diagonal().fill_(1)
    Bt = B.clone()
    Cg = torch.zeros_like(B)
    assert clblas_amd.trmm(p, COL, LEFT, UPPER, TRANS, UNIT, n, n, alpha, A, 0, n, Bt, 0, n) == 0
    assert gemm(COL, TRANS, NOTRANS, n, n, n, alpha, colmajor(Tm), 0, n, B, 0, n, 0, Cg, 0, n) == 0
    assert (Bt - Cg).abs().max().item() <= tol
    # SYMM right/lower == GEMM with the explicitly symmetrised matrix
    Lm = torch.where(lower, Am, torch.zeros_like(Am))
    Sm = Lm + Lm.T - torch.diag(torch.diagonal(Lm))
    C = C0.clone()
    Cg = C0.clone()
    assert clblas_amd.symm(p, COL, RIGHT, LOWER, n, n, alpha, A, 0, n, B, 0, n, beta, C, 0, n) == 0
    assert gemm(COL, NOTRANS, NOTRANS, n, n, n, alpha, B, 0, n, colmajor(Sm), 0, n, beta, Cg, 0, n) == 0
    torch.cuda.synchronize()
    assert (C - Cg).abs().max().item() <= tol


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("order", [ROW, COL])
def test_long_thin_shapes_integer_exact(gpu, dtype, order):
    """Triangles of a few thousand rows against one to three columns (and the reverse): SYRK with
    K = 1 and N = 1, TRMM and SYMM with a single right-hand side on either side.  Exact-integer
    data, poisoned triangles, default tile choice."""
    alpha, beta = scalars(dtype)
    for si, (N, K) in enumerate([(3000, 1), (1, 3000), (2049, 3)]):
        for uplo, trans in itertools.product([UPPER, LOWER], [NOTRANS, TRANS]):
            rows, cols = (N, K) if trans == NOTRANS else (K, N)
            A, lda = matrix(order, rows, cols, 5, 3, 110 + si, dtype, True, limit=4)
            C, ldc = matrix(order, N, N, 7, 2, 120 + si, dtype, True)
            logical_view(C, order, NOTRANS, N, N, 7, ldc)[~tri_mask(N, uplo == LOWER)] = nan_of(dtype)
            want = C.copy()
            assert oracle.syrk(order, uplo, trans, N, K, alpha, A, 5, lda, beta, want, 7, ldc) == 0
            st, got = gpu.syrk(order, uplo, trans, N, K, alpha, A, 5, lda, beta, C, 7, ldc)
            assert st == 0
            np.testing.assert_array_equal(got.view(np.uint8), want.view(np.uint8), err_msg="syrk N=%d K=%d" % (N, K))
    for si, (M, N) in enumerate([(3000, 1), (1, 3000), (2049, 2), (2, 2049)]):
        for side, uplo in itertools.product([LEFT, RIGHT], [UPPER, LOWER]):
            n = M if side == LEFT else N
            A0, lda = matrix(order, n, n, 5, 3, 130 + si, dtype, True, limit=2)
            B, ldb = matrix(order, M, N, 7, 2, 140 + si, dtype, True, limit=2)
            C, ldc = matrix(order, M, N, 11, 1, 150 + si, dtype, True)
            A = A0.copy()
            poison_triangle(A, order, n, 5, lda, uplo)
            want = C.copy()
            assert oracle.symm(order, side, uplo, M, N, alpha, A, 5, lda, B, 7, ldb, beta, want, 11, ldc) == 0
            st, got = gpu.symm(order, side, uplo, M, N, alpha, A, 5, lda, B, 7, ldb, beta, C, 11, ldc)
            assert st == 0
            np.testing.assert_array_equal(got, want, err_msg="symm M=%d N=%d" % (M, N))
            for trans, diag in itertools.product([NOTRANS, CONJ], [UNIT, NONUNIT]):
                A = A0.copy()
                poison_triangle(A, order, n, 5, lda, uplo, unit=diag == UNIT)
                want = B.copy()
                assert oracle.trmm(order, side, uplo, trans, diag, M, N, alpha, A, 5, lda, want, 7, ldb) == 0
                st, got = gpu.trmm(order, side, uplo, trans, diag, M, N, alpha, A, 5, lda, B, 7, ldb)
                assert st == 0
                assert not np.isnan(got[7:]).any()
                np.testing.assert_array_equal(got, want, err_msg="trmm M=%d N=%d" % (M, N))


def test_validation_codes(gpu):
    import clblas_amd
    import torch
    S = clblas_amd.Status
    x = torch.zeros(64, dtype=torch.float32, device="cuda")
    z = torch.zeros(64, dtype=torch.complex64, device="cuda")
    assert clblas_amd.syrk("S", COL, LOWER, NOTRANS, 4, 4, 1, None, 0, 4, 0, x, 0, 4) == S.InvalidMatA
    assert clblas_amd.syrk("S", COL, LOWER, NOTRANS, 4, 4, 1, x, 0, 4, 0, None, 0, 4) == S.InvalidMatC
    assert clblas_amd.syrk("S", COL, LOWER, NOTRANS, 4, 0, 1, x, 0, 4, 0, x, 0, 4) == S.InvalidDim
    assert clblas_amd.syrk("S", COL, LOWER, NOTRANS, 4, 4, 1, x, 0, 3, 0, x, 0, 4) == S.InvalidLeadDimA
    assert clblas_amd.syrk("S", COL, LOWER, NOTRANS, 4, 4, 1, x, 0, 4, 0, x, 0, 3) == S.InvalidLeadDimC
    assert clblas_amd.syrk("C", COL, LOWER, CONJ, 4, 4, 1, z, 0, 4, 0, z, 0, 4) == S.InvalidValue
    assert clblas_amd.syrk("S", COL, LOWER, CONJ, 4, 4, 1, x, 0, 4, 0, x, 0, 4) == S.Success
    assert clblas_amd.trmm("S", COL, LEFT, UPPER, NOTRANS, NONUNIT, 4, 4, 1, None, 0, 4, x, 0, 4) == S.InvalidMatA
    assert clblas_amd.trmm("S", COL, LEFT, UPPER, NOTRANS, NONUNIT, 4, 4, 1, x, 0, 4, None, 0, 4) == S.InvalidMatB
    assert clblas_amd.trmm("S", COL, LEFT, UPPER, NOTRANS, NONUNIT, 4, 4, 1, x, 0, 3, x, 0, 4) == S.InvalidLeadDimA
    assert clblas_amd.trmm("S", COL, RIGHT, UPPER, NOTRANS, NONUNIT, 2, 4, 1, x, 0, 3, x, 0, 4) == S.InvalidLeadDimA
    assert clblas_amd.trmm("S", COL, LEFT, UPPER, NOTRANS, NONUNIT, 4, 4, 1, x, 0, 4, x, 0, 3) == S.InvalidLeadDimB
    assert clblas_amd.trmm("S", COL, LEFT, 5, NOTRANS, NONUNIT, 4, 4, 1, x, 0, 4, x, 0, 4) == S.InvalidValue
    assert clblas_amd.symm("S", COL, LEFT, UPPER, 4, 4, 1, None, 0, 4, x, 0, 4, 0, x, 0, 4) == S.InvalidMatA
    assert clblas_amd.symm("S", COL, LEFT, UPPER, 4, 4, 1, x, 0, 4, None, 0, 4, 0, x, 0, 4) == S.InvalidMatB
    assert clblas_amd.symm("S", COL, LEFT, UPPER, 4, 4, 1, x, 0, 4, x, 0, 4, 0, None, 0, 4) == S.InvalidMatC
    assert clblas_amd.symm("S", COL, LEFT, UPPER, 4, 0, 1, x, 0, 4, x, 0, 4, 0, x, 0, 4) == S.InvalidDim
    assert clblas_amd.symm("S", COL, RIGHT, UPPER, 2, 4, 1, x, 0, 3, x, 0, 4, 0, x, 0, 4) == S.InvalidLeadDimA
    assert clblas_amd.symm("S", COL, LEFT, UPPER, 4, 4, 1, x, 0, 4, x, 0, 3, 0, x, 0, 4) == S.InvalidLeadDimB
    assert clblas_amd.symm("S", COL, LEFT, UPPER, 4, 4, 1, x, 0, 4, x, 0, 4, 0, x, 0, 3) == S.InvalidLeadDimC


def test_workspaces_per_stream_growth_and_teardown(gpu):
    """TRMM (copy of B) and TRSM (packed diagonal blocks) keep their workspaces per stream: two
    streams run different problems at once, a later larger problem makes the workspaces grow,
    and everything still works after clblasTeardown released them."""
    import clblas_amd
    import torch
    dtype = np.float64
    for rep, (M, N) in enumerate([(300, 200), (700, 520)]):
        s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
        A1, lda1 = matrix(COL, M, M, 0, 0, 1 + rep, dtype, True, limit=4)
        A2, lda2 = matrix(COL, N, N, 0, 0, 2 + rep, dtype, True, limit=4)
        B1, ldb = matrix(COL, M, N, 0, 0, 3 + rep, dtype, True, limit=4)
        B2 = oracle.integers(B1.size, 4 + rep, 4, dtype)
        w1, w2 = B1.copy(), B2.copy()
        assert oracle.trmm(COL, LEFT, LOWER, NOTRANS, NONUNIT, M, N, 2.0, A1, 0, lda1, w1, 0, ldb) == 0
        assert oracle.trmm(COL, RIGHT, UPPER, TRANS, UNIT, M, N, 2.0, A2, 0, lda2, w2, 0, ldb) == 0
        T1 = oracle.triangular(M, M, True, 5 + rep, dtype)
        X = oracle.uniform(M * N, 6 + rep, dtype)
        x_want = X.copy()
        assert oracle.trsm_blocked(COL, LEFT, LOWER, NOTRANS, NONUNIT, M, N, 1.0, T1, 0, M, x_want, 0, M) == 0
        d = [torch.from_numpy(x).cuda() for x in (A1, B1, A2, B2, T1, X)]
        torch.cuda.synchronize()
        assert clblas_amd.trmm("D", COL, LEFT, LOWER, NOTRANS, NONUNIT, M, N, 2.0, d[0], 0, lda1, d[1], 0, ldb, stream=s1) == 0
        assert clblas_amd.trmm("D", COL, RIGHT, UPPER, TRANS, UNIT, M, N, 2.0, d[2], 0, lda2, d[3], 0, ldb, stream=s2) == 0
        assert clblas_amd.dtrsm(COL, LEFT, LOWER, NOTRANS, NONUNIT, M, N, 1.0, d[4], 0, M, d[5], 0, M, stream=s1) == 0
        torch.cuda.synchronize()
        np.testing.assert_array_equal(d[1].cpu().numpy(), w1)
        np.testing.assert_array_equal(d[3].cpu().numpy(), w2)
        got = d[5].cpu().numpy()
        assert np.abs(got - x_want).max() <= 64 * M * np.finfo(dtype).eps * np.abs(x_want).max()
        if rep == 0:
            clblas_amd.teardown()
    assert clblas_amd.setup() == 0


@pytest.mark.parametrize("name", ["sample_ssymm", "sample_ssyrk_offsets", "sample_strmm_offsets"])
def test_level3_golden(gpu, name):
    """Fixed inputs of src/samples/example_ssymm.c, example_ssyrk.c, example_strmm.c with expected
    values computed in exact arithmetic (integers: the results are exact)."""
    from helpers import golden_cases
    c = golden_cases()[name]
    dt = np.float32
    A = np.array(c["A"], dtype=dt)
    if c["kind"] == "syrk":
        st, out = gpu.syrk(c["order"], c["uplo"], c["transA"], c["N"], c["K"], c["alpha"], A, c["offA"], c["lda"],
                           c["beta"], np.array(c["C"], dtype=dt), c["offC"], c["ldc"])
    elif c["kind"] == "trmm":
        st, out = gpu.trmm(c["order"], c["side"], c["uplo"], c["transA"], c["diag"], c["M"], c["N"], c["alpha"], A,
                           c["offA"], c["lda"], np.array(c["B"], dtype=dt), c["offB"], c["ldb"])
    else:
        st, out = gpu.symm(c["order"], c["side"], c["uplo"], c["M"], c["N"], c["alpha"], A, c["offA"], c["lda"],
                           np.array(c["B"], dtype=dt), c["offB"], c["ldb"], c["beta"], np.array(c["C"], dtype=dt),
                           c["offC"], c["ldc"])
    assert st == 0
    np.testing.assert_array_equal(out, np.array(c["expected"], dtype=dt))
