"""GPU parity tests for clblas{S,D,C,Z}syr2k and clblas{C,Z}{herk,her2k,hemm} through the C ABI,
against the CPU oracle.

Bars: exact equality with the oracle on exact-integer inputs (every tile of the table forced in
turn, unused triangles NaN-poisoned, junk imaginary parts on Hermitian diagonals, everything
outside the result untouched); the reference samples' fixed inputs; for real-valued
data the K*eps bound of the GEMM tests; at 2048 agreement with this library's own (separately
pinned) complex GEMM on the explicitly formed Hermitian operands."""
import itertools

import numpy as np
import pytest

import oracle
from helpers import COL, ROW, NOTRANS, TRANS, CONJ, UPPER, LOWER, LEFT, RIGHT, golden_array, golden_cases, logical_view
from l3_util import (CPLX, abs1, bound, err, herm_dense, is_cplx, matrix, nan_of, rank2k_want, real_scalars, scalars,
                     tri_mask)
from test_oracle_rank2k_hermitian import (DT, GOLDEN, call_rank2k, hemm_case, rank2k_case, rank2k_scalars,
                                          rank2k_variants, run_golden)

pytestmark = pytest.mark.gpu
N_TILES = {np.dtype(np.float32): 7, np.dtype(np.float64): 4, np.dtype(np.complex64): 4, np.dtype(np.complex128): 4}
WIDE = lambda dt: np.complex128 if is_cplx(dt) else np.float64


@pytest.fixture(scope="module")
def gpu():
    import gpu_util
    import torch
    assert torch.cuda.is_available()
    return gpu_util


def tiles(dtype):
    return [None] + list(range(N_TILES[np.dtype(dtype)]))


@pytest.mark.parametrize("name", GOLDEN)
def test_golden(gpu, name):
    c = golden_cases()[name]
    st, out = run_golden(gpu, c)
    assert st == 0
    np.testing.assert_array_equal(out, golden_array(c["expected"], DT[c["dtype"]]))


@pytest.mark.parametrize("kind,dtype,order,uplo,trans", rank2k_variants())
def test_rank2k_integer_exact_all_tiles(gpu, kind, dtype, order, uplo, trans):
    alpha, beta = rank2k_scalars(kind, dtype, True)
    for si, (N, K) in enumerate([(1, 1), (5, 3), (64, 20), (70, 129), (257, 33), (300, 130), (513, 17)]):
        A, lda, B, ldb, C, ldc, keep = rank2k_case(kind, dtype, order, uplo, trans, N, K, 10 + 3 * si, True)
        want = C.copy()
        assert call_rank2k(oracle, kind, order, uplo, trans, N, K, alpha, A, 5, lda, B, 3, ldb, beta, want, 7, ldc) == 0
        for tile in tiles(dtype):
            st, got = getattr(gpu, kind)(*((order, uplo, trans, N, K, alpha, A, 5, lda) +
                                           (() if kind == "herk" else (B, 3, ldb)) + (beta, C, 7, ldc)), tile=tile)
            assert st == 0
            # values, not bits: conjugation makes zeros whose sign depends on the order of the sum
            np.testing.assert_array_equal(got, want, err_msg="%s N=%d K=%d tile %s" % (kind, N, K, tile))


@pytest.mark.parametrize("kind,dtype", [("syr2k", np.float32), ("syr2k", np.float64), ("syr2k", np.complex64),
                                        ("syr2k", np.complex128), ("herk", np.complex64), ("herk", np.complex128),
                                        ("her2k", np.complex64), ("her2k", np.complex128)])
def test_rank2k_uniform_data(gpu, kind, dtype):
    alpha, beta = rank2k_scalars(kind, dtype, False)
    tr2 = TRANS if kind == "syr2k" else CONJ
    for uplo, trans, (N, K) in [(LOWER, NOTRANS, (700, 513)), (UPPER, tr2, (1031, 300)), (LOWER, tr2, (129, 2048))]:
        rows, cols = (N, K) if trans == NOTRANS else (K, N)
        A, lda = matrix(COL, rows, cols, 0, 1, 1, dtype, False)
        B, ldb = matrix(COL, rows, cols, 0, 2, 5, dtype, False)
        C, ldc = matrix(COL, N, N, 0, 3, 2, dtype, False)
        st, got = getattr(gpu, kind)(*((COL, uplo, trans, N, K, alpha, A, 0, lda) +
                                       (() if kind == "herk" else (B, 0, ldb)) + (beta, C, 0, ldc)))
        assert st == 0
        real = np.float32 if np.dtype(dtype) in (np.dtype(np.float32), np.dtype(np.complex64)) else np.float64
        al = complex(dtype(alpha)) if (is_cplx(dtype) and kind != "herk") else float(real(alpha))
        be = complex(dtype(beta)) if (is_cplx(dtype) and kind == "syr2k") else float(real(beta))
        want, mag = rank2k_want(kind, COL, uplo, trans, N, K, al, A, 0, lda, B, 0, ldb, be, C, 0, ldc)
        keep = tri_mask(N, uplo == LOWER)
        gv = logical_view(got, COL, NOTRANS, N, N, 0, ldc)
        depth = K if kind == "herk" else 2 * K
        assert np.all(err(gv.astype(WIDE(dtype)), want)[keep] <= bound(depth, mag, dtype)[keep])
        if kind != "syr2k":
            assert (np.diag(gv).imag == 0).all()
        np.testing.assert_array_equal(gv[~keep], logical_view(C, COL, NOTRANS, N, N, 0, ldc)[~keep])
        # beta == 0 with a NaN-filled C: the triangle comes out finite, the rest stays NaN
        Cn = np.full(C.size, nan_of(dtype), dtype=dtype)
        st, got = getattr(gpu, kind)(*((COL, uplo, trans, N, K, alpha, A, 0, lda) +
                                       (() if kind == "herk" else (B, 0, ldb)) + (0.0, Cn, 0, ldc)))
        gv = logical_view(got, COL, NOTRANS, N, N, 0, ldc)
        assert st == 0 and np.isfinite(gv[keep].real).all() and np.isnan(gv[~keep].real).all()


@pytest.mark.parametrize("dtype", CPLX)
@pytest.mark.parametrize("order,side,uplo", list(itertools.product([ROW, COL], [LEFT, RIGHT], [UPPER, LOWER])))
def test_hemm_integer_exact_all_tiles(gpu, dtype, order, side, uplo):
    alpha, beta = scalars(dtype)
    for si, (M, N) in enumerate([(1, 1), (3, 7), (33, 20), (70, 45), (257, 130), (140, 300)]):
        A, lda, B, ldb, C, ldc = hemm_case(dtype, order, side, uplo, M, N, 50 + 3 * si, True)
        want = C.copy()
        assert oracle.hemm(order, side, uplo, M, N, alpha, A, 5, lda, B, 7, ldb, beta, want, 11, ldc) == 0
        for tile in tiles(dtype):
            st, got = gpu.hemm(order, side, uplo, M, N, alpha, A, 5, lda, B, 7, ldb, beta, C, 11, ldc, tile=tile)
            assert st == 0
            np.testing.assert_array_equal(got, want, err_msg="M=%d N=%d tile %s" % (M, N, tile))


@pytest.mark.parametrize("kind,dtype,order,uplo,trans", rank2k_variants())
def test_rank2k_long_thin_integer_exact(gpu, kind, dtype, order, uplo, trans):
    """Rank-1 / rank-3 updates of a triangle of a few thousand rows, a 1 x 1 result from
    operands 3000 deep, and small results from operands thousands deep (those run as a plain
    product with a K split into a scratch square, folded into the triangle by a second pass):
    exact-integer data, default tile choice."""
    alpha, beta = rank2k_scalars(kind, dtype, True)
    for si, (N, K) in enumerate([(3000, 1), (1, 3000), (2049, 3), (64, 5000), (300, 4100)]):
        A, lda, B, ldb, C, ldc, keep = rank2k_case(kind, dtype, order, uplo, trans, N, K, 210 + 3 * si, True)
        want = C.copy()
        assert call_rank2k(oracle, kind, order, uplo, trans, N, K, alpha, A, 5, lda, B, 3, ldb, beta, want, 7, ldc) == 0
        st, got = getattr(gpu, kind)(*((order, uplo, trans, N, K, alpha, A, 5, lda) +
                                       (() if kind == "herk" else (B, 3, ldb)) + (beta, C, 7, ldc)))
        assert st == 0
        np.testing.assert_array_equal(got, want, err_msg="%s N=%d K=%d" % (kind, N, K))


@pytest.mark.parametrize("dtype", CPLX)
@pytest.mark.parametrize("order,side,uplo", list(itertools.product([ROW, COL], [LEFT, RIGHT], [UPPER, LOWER])))
def test_hemm_long_thin_integer_exact(gpu, dtype, order, side, uplo):
    alpha, beta = scalars(dtype)
    for si, (M, N) in enumerate([(3000, 1), (1, 3000), (2049, 2), (2, 2049)]):
        A, lda, B, ldb, C, ldc = hemm_case(dtype, order, side, uplo, M, N, 250 + 3 * si, True)
        want = C.copy()
        assert oracle.hemm(order, side, uplo, M, N, alpha, A, 5, lda, B, 7, ldb, beta, want, 11, ldc) == 0
        st, got = gpu.hemm(order, side, uplo, M, N, alpha, A, 5, lda, B, 7, ldb, beta, C, 11, ldc)
        assert st == 0
        np.testing.assert_array_equal(got, want, err_msg="M=%d N=%d" % (M, N))


@pytest.mark.parametrize("dtype", CPLX)
@pytest.mark.parametrize("side,uplo", list(itertools.product([LEFT, RIGHT], [UPPER, LOWER])))
def test_hemm_uniform_data(gpu, dtype, side, uplo):
    alpha, beta = real_scalars(dtype)
    M, N = (700, 300) if side == LEFT else (300, 700)
    n = M if side == LEFT else N
    A, lda, B, ldb, C, ldc = hemm_case(dtype, COL, side, uplo, M, N, 91, False)
    st, got = gpu.hemm(COL, side, uplo, M, N, alpha, A, 5, lda, B, 7, ldb, beta, C, 11, ldc)
    assert st == 0
    H = herm_dense(A, COL, n, 5, lda, uplo)
    Bv = logical_view(B, COL, NOTRANS, M, N, 7, ldb).astype(np.complex128)
    Cv = logical_view(C, COL, NOTRANS, M, N, 11, ldc).astype(np.complex128)
    al, be = complex(dtype(alpha)), complex(dtype(beta))
    want = al * (H @ Bv if side == LEFT else Bv @ H) + be * Cv
    mag = abs1(np.asarray(al)) * (abs1(H) @ abs1(Bv) if side == LEFT else abs1(Bv) @ abs1(H)) + \
        abs1(np.asarray(be)) * abs1(Cv)
    gv = logical_view(got, COL, NOTRANS, M, N, 11, ldc).astype(np.complex128)
    assert np.all(err(gv, want) <= bound(n, mag, dtype))


@pytest.mark.parametrize("dtype", CPLX)
def test_hermitian_routines_vs_gemm_2048(gpu, dtype):
    """At a size the CPU oracle does not reach: HERK / HER2K / HEMM against this library's complex
    GEMM on explicitly formed operands (same data, same device)."""
    import torch
    import clblas_amd
    n, k = 2048, 1536
    pre = "C" if dtype == np.complex64 else "Z"
    tdt = torch.complex64 if dtype == np.complex64 else torch.complex128
    eps = np.finfo(dtype).eps
    g = torch.Generator(device="cuda").manual_seed(5)
    rnd = lambda *s: (torch.rand(*s, 2, device="cuda", generator=g, dtype=torch.float64) - 0.5)
    cplx = lambda t: torch.view_as_complex(t.contiguous()).to(tdt)
    Ad, Bd = cplx(rnd(n * k)), cplx(rnd(n * k))          # n x k column-major buffers (ld = n)
    gemm = clblas_amd.cgemm if dtype == np.complex64 else clblas_amd.zgemm
    lower = torch.tril(torch.ones(n, n, device="cuda", dtype=torch.bool))
    # HERK: lower triangle of 0.5 A A^H
    C1 = torch.zeros(n * n, device="cuda", dtype=tdt)
    C2 = torch.zeros(n * n, device="cuda", dtype=tdt)
    assert clblas_amd.herk(pre, COL, LOWER, NOTRANS, n, k, 0.5, Ad, 0, n, 0.0, C1, 0, n) == 0
    assert gemm(COL, NOTRANS, CONJ, n, n, k, 0.5, Ad, 0, n, Ad, 0, n, 0.0, C2, 0, n) == 0
    torch.cuda.synchronize()
    m1, m2 = C1.view(n, n).T, C2.view(n, n).T            # element (i, j) of the column-major result
    d = (m1 - m2)[lower].abs().max().item()
    assert d <= 8 * k * eps, d
    assert (torch.diagonal(m1).imag == 0).all()
    assert (m1[~lower] == 0).all()
    # HER2K: lower triangle of al A B^H + conj(al) B A^H
    al = 0.5 - 0.25j
    C1.zero_()
    assert clblas_amd.her2k(pre, COL, LOWER, NOTRANS, n, k, al, Ad, 0, n, Bd, 0, n, 0.0, C1, 0, n) == 0
    assert gemm(COL, NOTRANS, CONJ, n, n, k, al, Ad, 0, n, Bd, 0, n, 0.0, C2, 0, n) == 0
    assert gemm(COL, NOTRANS, CONJ, n, n, k, np.conj(al), Bd, 0, n, Ad, 0, n, 1.0, C2, 0, n) == 0
    torch.cuda.synchronize()
    d = (m1 - m2)[lower & ~torch.eye(n, device="cuda", dtype=torch.bool)].abs().max().item()
    assert d <= 16 * k * eps, d
    assert (torch.diagonal(m1).imag == 0).all()
    assert (torch.diagonal(m1).real - torch.diagonal(m2).real).abs().max().item() <= 16 * k * eps
    # HEMM: Hermitian H (upper triangle stored, junk below and in the diagonal's imaginary parts)
    H = cplx(rnd(n, n))
    H = H + H.conj().T                                   # H[i][j], real diagonal
    stored = torch.triu(H) + torch.tril(torch.full_like(H, float("nan")), -1)
    stored = stored + 1j * torch.eye(n, device="cuda", dtype=tdt)
    Hs = stored.T.contiguous().view(-1)                  # column-major buffers: element (i, j) at i + j n
    Hf = H.T.contiguous().view(-1)
    Bm = cplx(rnd(n * n))
    C1 = torch.zeros(n * n, device="cuda", dtype=tdt)
    C2 = torch.zeros(n * n, device="cuda", dtype=tdt)
    assert clblas_amd.hemm(pre, COL, LEFT, UPPER, n, n, 1.0, Hs, 0, n, Bm, 0, n, 0.0, C1, 0, n) == 0
    assert gemm(COL, NOTRANS, NOTRANS, n, n, n, 1.0, Hf, 0, n, Bm, 0, n, 0.0, C2, 0, n) == 0
    torch.cuda.synchronize()
    d = (C1 - C2).abs().max().item()
    assert d <= 16 * n * eps, d
