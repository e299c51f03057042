"""GPU parity tests for clblasCgemm / clblasZgemm through the C ABI, against the CPU oracle.

Bars: exact equality on Gaussian-integer inputs (every partial sum is exactly representable,
so any order of the multiply-adds gives the same bits); for real-valued data, on the real and
on the imaginary part separately,
    |C - C_exact| <= 2 (2K+6) u (|alpha|_1 |A|_1 |B|_1 + |beta|_1 |C|_1),   |z|_1 = |re| + |im|,
u = unit roundoff: the K*eps bound of the real routines applied to the 2K products that make
up each part."""
import itertools

import numpy as np
import pytest

import oracle
from helpers import COL, ROW, NOTRANS, TRANS, CONJ, cgemm_bound, mem_dims

pytestmark = pytest.mark.gpu

CDT = [np.complex64, np.complex128]
ALL_T = [NOTRANS, TRANS, CONJ]
N_TILES = {np.complex64: 4, np.complex128: 4}


@pytest.fixture(scope="module")
def gpu():
    import gpu_util
    import torch
    assert torch.cuda.is_available()
    import clblas_amd
    assert clblas_amd.setup() == 0
    return gpu_util


def _layout(order, tA, tB, M, N, K, pad, offs):
    ia, oa = mem_dims(order, tA, M, K)
    ib, ob = mem_dims(order, tB, K, N)
    ic, oc = mem_dims(order, NOTRANS, M, N)
    lda, ldb, ldc = ia + pad, ib + pad, ic + pad
    return lda, ldb, ldc, offs[0] + oa * lda, offs[1] + ob * ldb, offs[2] + oc * ldc


INT_SHAPES = [(1, 1, 1), (2, 1, 3), (8, 16, 17), (17, 32, 62), (64, 64, 64), (62, 144, 128), (128, 128, 8),
              (129, 65, 33), (300, 260, 100), (130, 70, 1031)]


@pytest.mark.parametrize("dtype", CDT)
@pytest.mark.parametrize("order", [ROW, COL])
@pytest.mark.parametrize("tA,tB", list(itertools.product(ALL_T, ALL_T)))
def test_gaussian_integer_exact_all_tiles(gpu, dtype, order, tA, tB):
    """The reference's correctness method (exact-integer inputs, assert-equal) on complex data,
    every tile of the table forced in turn plus the default choice; odd offsets, padded leading
    dimensions, and nothing outside the M x N window of C may change."""
    alpha, beta = 2 - 1j, -1 + 2j
    for si, (M, N, K) in enumerate(INT_SHAPES):
        offs = (5, 7, 11)
        lda, ldb, ldc, na, nb, nc = _layout(order, tA, tB, M, N, K, 3, offs)
        A = oracle.integers(na, 100 + si, 8, dtype)
        B = oracle.integers(nb, 200 + si, 8, dtype)
        C = oracle.integers(nc, 300 + si, 8, dtype)
        want = C.copy()
        assert oracle.gemm(order, tA, tB, M, N, K, alpha, A, offs[0], lda, B, offs[1], ldb, beta, want, offs[2],
                           ldc) == 0
        for tile in [None] + list(range(N_TILES[dtype])):
            st, got = gpu.gemm(order, tA, tB, M, N, K, alpha, A, offs[0], lda, B, offs[1], ldb, beta, C, offs[2], ldc,
                               tile=tile)
            assert st == 0
            np.testing.assert_array_equal(got, want, err_msg="shape %s tile %s" % ((M, N, K), tile))


def _check_sampled(dtype, tA, tB, M, N, K, alpha, beta, A, lda, B, ldb, C0, got, ldc, nsamp=2000, seed=0):
    """Column-major buffers starting at element (0,0); sampled elements incl. all four borders."""
    rng = np.random.default_rng(seed)
    rows = [rng.integers(0, M, nsamp), np.full(200, M - 1), np.zeros(200, dtype=np.int64), rng.integers(0, M, 400)]
    cols = [rng.integers(0, N, nsamp), rng.integers(0, N, 200), rng.integers(0, N, 200),
            np.concatenate([np.full(200, N - 1), np.zeros(200, dtype=np.int64)])]
    rows, cols = np.concatenate(rows), np.concatenate(cols)
    exact, mag = oracle.gemm_exact(tA, tB, K, alpha, A, lda, B, ldb, beta, C0, ldc, rows, cols)
    vals = got[rows + cols * ldc].astype(np.complex128)
    err = np.maximum(np.abs(vals.real - exact.real), np.abs(vals.imag - exact.imag))
    bound = cgemm_bound(K, mag, dtype)
    worst = np.argmax(err / bound)
    assert np.all(err <= bound), "element (%d,%d): err %.3e bound %.3e" % (rows[worst], cols[worst], err[worst],
                                                                          bound[worst])
    return float((err / bound).max())


REAL_SHAPES = [(1024, 1024, 1024), (1000, 777, 513), (4097, 255, 1031), (127, 129, 4096), (64, 8192, 512)]


@pytest.mark.parametrize("dtype", CDT)
@pytest.mark.parametrize("tA,tB", list(itertools.product(ALL_T, ALL_T)))
def test_uniform_data_against_exact(gpu, dtype, tA, tB):
    alpha, beta = 0.7 - 0.3j, -1.3 + 0.5j
    for si, (M, N, K) in enumerate(REAL_SHAPES):
        lda, ldb, ldc, na, nb, nc = _layout(COL, tA, tB, M, N, K, 1, (0, 0, 0))
        A, B, C = oracle.uniform(na, 10 + si, dtype), oracle.uniform(nb, 20 + si, dtype), oracle.uniform(nc, 30 + si, dtype)
        st, got = gpu.gemm(COL, tA, tB, M, N, K, alpha, A, 0, lda, B, 0, ldb, beta, C, 0, ldc)
        assert st == 0
        _check_sampled(dtype, tA, tB, M, N, K, alpha, beta, A, lda, B, ldb, C, got, ldc, seed=si)
        # padding rows of C stay as they were
        pad = np.arange(nc).reshape(-1, ldc)[:, M:].ravel()
        np.testing.assert_array_equal(got[pad], C[pad])


@pytest.mark.parametrize("dtype", CDT)
def test_against_oracle_elementwise(gpu, dtype):
    """Every element of a mid-size product against the oracle's restatement of the reference
    arithmetic: both sit within the bound of the exact result, hence within twice the bound of
    each other."""
    M, N, K = 384, 320, 448
    alpha, beta = 1.1 + 0.4j, 0.3 - 0.9j
    for tA, tB in ((NOTRANS, NOTRANS), (CONJ, TRANS), (TRANS, CONJ)):
        lda, ldb, ldc, na, nb, nc = _layout(COL, tA, tB, M, N, K, 0, (0, 0, 0))
        A, B, C = oracle.uniform(na, 1, dtype), oracle.uniform(nb, 2, dtype), oracle.uniform(nc, 3, dtype)
        want = C.copy()
        assert oracle.gemm(COL, tA, tB, M, N, K, alpha, A, 0, lda, B, 0, ldb, beta, want, 0, ldc) == 0
        st, got = gpu.gemm(COL, tA, tB, M, N, K, alpha, A, 0, lda, B, 0, ldb, beta, C, 0, ldc)
        assert st == 0
        rows, cols = np.meshgrid(np.arange(M), np.arange(N), indexing="ij")
        _, mag = oracle.gemm_exact(tA, tB, K, alpha, A, lda, B, ldb, beta, C, ldc, rows.ravel(), cols.ravel())
        bound = cgemm_bound(K, mag.reshape(M, N).ravel(order="F"), dtype)
        d = got.astype(np.complex128) - want
        assert np.all(np.maximum(np.abs(d.real), np.abs(d.imag)) <= 2 * bound)


def test_beta_zero_alpha_zero_k_zero(gpu):
    for dtype in CDT:
        M, N, K = 70, 90, 50
        A, B = oracle.uniform(M * K, 1, dtype), oracle.uniform(K * N, 2, dtype)
        nan = np.full(M * N, np.nan + 1j * np.nan, dtype=dtype)
        want = nan.copy()
        oracle.gemm(COL, NOTRANS, NOTRANS, M, N, K, 1, A, 0, M, B, 0, K, 0, want, 0, M)
        st, got = gpu.gemm(COL, NOTRANS, NOTRANS, M, N, K, 1, A, 0, M, B, 0, K, 0, nan, 0, M)
        assert st == 0 and np.isfinite(got.real).all() and np.isfinite(got.imag).all()
        np.testing.assert_allclose(got, want, rtol=0, atol=8 * K * np.finfo(dtype).eps)
        # beta with only an imaginary part is not zero: C is read
        st, got = gpu.gemm(COL, NOTRANS, NOTRANS, M, N, K, 1, A, 0, M, B, 0, K, 1e-30j, nan, 0, M)
        assert st == 0 and np.isnan(got.real).all()
        # alpha == 0, beta == 1 leaves C as it was; beta == i rotates it exactly
        C1 = oracle.uniform(M * N, 3, dtype)
        st, got = gpu.gemm(COL, NOTRANS, CONJ, M, N, K, 0, A, 0, M, B, 0, N, 1, C1, 0, M)
        assert st == 0
        np.testing.assert_array_equal(got, C1)
        st, got = gpu.gemm(COL, NOTRANS, NOTRANS, M, N, K, 0, A, 0, M, B, 0, K, 1j, C1, 0, M)
        assert st == 0
        np.testing.assert_array_equal(got.real, -C1.imag)
        np.testing.assert_array_equal(got.imag, C1.real)
        # K == 0: C <- beta * C; beta == 0 clears NaNs
        st, got = gpu.gemm(COL, NOTRANS, NOTRANS, M, N, 0, 1, A, 0, M, B, 0, 1, 0.5, C1, 0, M)
        assert st == 0
        np.testing.assert_array_equal(got, (0.5 * C1).astype(dtype))
        st, got = gpu.gemm(COL, NOTRANS, NOTRANS, M, N, 0, 1, A, 0, M, B, 0, 1, 0, nan, 0, M)
        assert st == 0 and (got == 0).all()


def test_validation_codes_match_real_routines(gpu):
    import clblas_amd
    import torch
    x = torch.zeros(64, dtype=torch.complex64, device="cuda")
    assert clblas_amd.cgemm(COL, 0, 0, 4, 4, 4, 1, None, 0, 4, x, 0, 4, 0, x, 0, 4) == clblas_amd.Status.InvalidMatA
    assert clblas_amd.cgemm(COL, 0, 0, 4, 4, 4, 1, x, 0, 3, x, 0, 4, 0, x, 0, 4) == clblas_amd.Status.InvalidLeadDimA
    assert clblas_amd.cgemm(COL, 0, 2, 4, 4, 4, 1, x, 0, 4, x, 0, 3, 0, x, 0, 4) == clblas_amd.Status.InvalidLeadDimB
    assert clblas_amd.cgemm(COL, 0, 0, 4, 4, 4, 1, x, 0, 4, x, 0, 4, 0, x, 0, 3) == clblas_amd.Status.InvalidLeadDimC
    assert clblas_amd.cgemm(COL, 0, 0, 0, 4, 4, 1, x, 0, 4, x, 0, 4, 0, x, 0, 4) == clblas_amd.Status.InvalidDim
    assert clblas_amd.cgemm(COL, 0, 3, 4, 4, 4, 1, x, 0, 4, x, 0, 4, 0, x, 0, 4) == clblas_amd.Status.InvalidValue
    z = torch.zeros(64, dtype=torch.complex128, device="cuda")
    assert clblas_amd.zgemm(COL, 0, 0, 4, 4, 4, 1, z, 0, 4, z, 0, 4, 0, None, 0, 4) == clblas_amd.Status.InvalidMatC


@pytest.mark.parametrize("dtype", CDT)
def test_large_square(gpu, dtype):
    """4096^3 (the size class of the headline configurations), conjugate-transposed A."""
    n = 4096
    alpha, beta = 1.0 - 0.5j, 0.25 + 0.75j
    A, B, C = oracle.uniform(n * n, 1, dtype), oracle.uniform(n * n, 2, dtype), oracle.uniform(n * n, 3, dtype)
    st, got = gpu.gemm(COL, CONJ, NOTRANS, n, n, n, alpha, A, 0, n, B, 0, n, beta, C, 0, n)
    assert st == 0
    _check_sampled(dtype, CONJ, NOTRANS, n, n, n, alpha, beta, A, n, B, n, C, got, n)
    # linearity in the right-hand operand: C(B v) summed over columns == (alpha A^H B + beta C0) v
    v = np.random.default_rng(5).uniform(-1, 1, n)
    lhs = got.reshape(n, n, order="F").astype(np.complex128) @ v
    Bv = B.reshape(n, n, order="F").astype(np.complex128) @ v
    rhs = complex(dtype(alpha)) * (A.reshape(n, n, order="F").astype(np.complex128).conj().T @ Bv) + \
        complex(dtype(beta)) * (C.reshape(n, n, order="F").astype(np.complex128) @ v)
    scale = np.abs(rhs).max()
    assert np.abs(lhs - rhs).max() <= 64 * n * np.finfo(dtype).eps * scale
