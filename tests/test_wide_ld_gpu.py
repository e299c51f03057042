"""Leading dimensions beyond the reach of one buffer descriptor per panel (256 * ld * sizeof(T) >= 2^31):
the library switches to the wide-ld form of its smallest tile (one descriptor per panel row), for
GEMM and for every GEMM-shaped routine.  The reference indexes with 32-bit element offsets and so
serves any such leading dimension whose matrix fits 2^32 elements
(src/library/blas/AutoGemm/KernelOpenCL.py:68-81).

Two kinds of cases, all on exact-integer data (equality, not a tolerance):
  * the wide-ld kernels forced (CLBLAS_AMD_GEMM_WIDE_LD=1) on ordinary small problems: every
    transpose pair and type, K splits, sliced tails, and the routines with triangular structure;
  * really large leading dimensions: DGEMM TN 64 x 64 x 2^21 (lda = ldb = 2^21), ZGEMM with
    ld = 600 000, DSYRK Trans with K = 2^21, STRMM with lda = 2 200 000."""
import itertools

import numpy as np
import pytest
import torch

import clblas_amd
import oracle
from helpers import COL, ROW, NOTRANS, TRANS, CONJ, LEFT, RIGHT, UPPER, LOWER, UNIT, NONUNIT, exact_int_limits, logical_view

pytestmark = pytest.mark.gpu

TYPES = [np.float32, np.float64, np.complex64, np.complex128]


@pytest.fixture(scope="module")
def gpu():
    import gpu_util
    assert clblas_amd.setup() == 0
    return gpu_util


@pytest.mark.parametrize("dtype", TYPES)
def test_forced_wide_ld_kernels_integer_exact(gpu, dtype):
    cplx = np.dtype(dtype).kind == "c"
    alpha, beta = ((2 - 1j), (-1 + 2j)) if cplx else (3.0, -2.0)
    transes = [NOTRANS, TRANS, CONJ] if cplx else [NOTRANS, TRANS]
    shapes = [(1, 1, 1), (17, 32, 62), (64, 64, 64), (257, 129, 33), (300, 520, 200), (130, 70, 1031),
              (100, 90, 4096),      # K split
              (1100, 1000, 520)]    # more than 256 tiles: sliced tail
    with gpu.debug_env(CLBLAS_AMD_GEMM_WIDE_LD=1):
        for si, (M, N, K) in enumerate(shapes):
            for tA, tB in itertools.product(transes, transes):
                if si >= 6 and (tA, tB) not in ((NOTRANS, NOTRANS), (TRANS, TRANS)):
                    continue
                lim = 8 if cplx else exact_int_limits(K, alpha, beta, dtype)[0]
                ra, ca = (M, K) if tA == NOTRANS else (K, M)
                rb, cb = (K, N) if tB == NOTRANS else (N, K)
                lda, ldb, ldc = ra + 3, rb + 1, M + 2
                A = oracle.integers(5 + lda * ca, 10 + si, lim, dtype)
                B = oracle.integers(7 + ldb * cb, 20 + si, lim, dtype)
                C = oracle.integers(11 + ldc * N, 30 + si, 8, dtype)
                want = C.copy()
                assert oracle.gemm(COL, tA, tB, M, N, K, alpha, A, 5, lda, B, 7, ldb, beta, want, 11, ldc) == 0
                st, got = gpu.gemm(COL, tA, tB, M, N, K, alpha, A, 5, lda, B, 7, ldb, beta, C, 11, ldc)
                what = clblas_amd.last_dispatch()[0]
                assert st == 0 and "wide ld" in what, what
                np.testing.assert_array_equal(got, want, err_msg="%s %s" % ((M, N, K, tA, tB), what))
        # triangular structure through the same kernels
        n, k = 200, 150
        lim = 8 if cplx else 30
        A = oracle.integers(n * n, 41, lim, dtype)
        B = oracle.integers(n * k, 42, lim, dtype)
        C = oracle.integers(n * n, 43, 8, dtype)
        for uplo, tr in itertools.product([UPPER, LOWER], [NOTRANS, TRANS]):
            want = C.copy()
            Ak = oracle.integers(n * k, 44, lim, dtype)
            assert oracle.syrk(COL, uplo, tr, n, k, alpha, Ak, 0, n if tr == NOTRANS else k, beta, want, 0, n) == 0
            st, got = gpu.syrk(COL, uplo, tr, n, k, alpha, Ak, 0, n if tr == NOTRANS else k, beta, C, 0, n)
            assert st == 0
            np.testing.assert_array_equal(got, want)
        for side, uplo, tr, diag in itertools.product([LEFT, RIGHT], [UPPER, LOWER], [NOTRANS, TRANS], [UNIT, NONUNIT]):
            Bm = oracle.integers(n * n, 45, lim, dtype)
            want = Bm.copy()
            assert oracle.trmm(COL, side, uplo, tr, diag, n, n, alpha, A, 0, n, want, 0, n) == 0
            st, got = gpu.trmm(COL, side, uplo, tr, diag, n, n, alpha, A, 0, n, Bm, 0, n)
            assert st == 0
            np.testing.assert_array_equal(got, want)
            want = C.copy()
            assert oracle.symm(COL, side, uplo, n, n, alpha, A, 0, n, B[:n * n] if B.size >= n * n else Bm, 0, n, beta, want, 0, n) == 0
            st, got = gpu.symm(COL, side, uplo, n, n, alpha, A, 0, n, B[:n * n] if B.size >= n * n else Bm, 0, n, beta, C, 0, n)
            assert st == 0
            np.testing.assert_array_equal(got, want)


def _int_tensor(shape, lim, dtype, gen):
    x = torch.randint(-lim, lim + 1, shape, device="cuda", generator=gen).to(dtype)
    return x


def test_dgemm_tn_with_k_of_two_million():
    """C (64 x 64) = A^T B with K = 2^21: A and B are K x 64 column-major, lda = ldb = 2^21, so
    consecutive rows of the k-contiguous panels lie 16 MiB apart."""
    M = N = 64
    K = 1 << 21
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1)
    A = _int_tensor((M, K), 3, torch.float64, gen)     # A[m, :] is column m of the stored K x M matrix
    B = _int_tensor((N, K), 3, torch.float64, gen)
    C = torch.full((N, M), float("nan"), device="cuda", dtype=torch.float64)
    st = clblas_amd.dgemm(COL, TRANS, NOTRANS, M, N, K, 1.0, A, 0, K, B, 0, K, 0.0, C, 0, M)
    torch.cuda.synchronize()
    assert st == 0 and "wide ld" in clblas_amd.last_dispatch()[0], clblas_amd.last_dispatch()[0]
    want = B @ A.T          # want[n, m] = sum_k B[n, k] A[m, k] = C(m, n), exact in double precision
    assert torch.equal(C, want)


def test_zgemm_with_leading_dimensions_of_600000():
    M, N, K = 64, 48, 300
    ld = 600_000
    gen = torch.Generator(device="cuda")
    gen.manual_seed(2)
    # Every operand has max(rows, columns) = K columns of ld elements, so that it is large enough both as
    # it lies and transposed (op(B) = B^T reads K columns of the N x K matrix).
    A = torch.view_as_complex(_int_tensor((K, ld, 2), 4, torch.float64, gen))     # A[c, r] = stored element (r, c)
    B = torch.view_as_complex(_int_tensor((K, ld, 2), 4, torch.float64, gen))
    C = torch.view_as_complex(_int_tensor((N, ld, 2), 4, torch.float64, gen))
    C0 = C.clone()
    alpha, beta = 2 - 1j, -1 + 2j
    for tA, tB in ((NOTRANS, NOTRANS), (CONJ, TRANS)):
        C.copy_(C0)
        st = clblas_amd.zgemm(COL, tA, tB, M, N, K, alpha, A, 0, ld, B, 0, ld, beta, C, 0, ld)
        torch.cuda.synchronize()
        assert st == 0 and "wide ld" in clblas_amd.last_dispatch()[0]
        # operands as matrices: stored(r, c) = X[c, r]
        opA = A[:K, :M].T if tA == NOTRANS else A[:M, :K].conj()                   # M x K
        opB = B[:N, :K].T if tB == NOTRANS else B[:K, :N]                           # K x N
        want = alpha * (opA @ opB) + beta * C0[:N, :M].T
        assert torch.equal(C[:N, :M].T, want)
        assert torch.equal(C[:, M:], C0[:, M:])                                     # padding rows untouched


def test_dsyrk_trans_with_k_of_two_million():
    N = 64
    K = 1 << 21
    gen = torch.Generator(device="cuda")
    gen.manual_seed(3)
    A = _int_tensor((N, K), 3, torch.float64, gen)       # stored K x N column-major, lda = K
    C = _int_tensor((N, N), 5, torch.float64, gen)
    C0 = C.clone()
    st = clblas_amd.syrk("D", COL, LOWER, TRANS, N, K, 1.0, A, 0, K, 2.0, C, 0, N)
    torch.cuda.synchronize()
    assert st == 0
    full = A @ A.T + 2.0 * C0.T                            # C(m, n) for all m, n
    got = C.T                                              # got[m, n] = C(m, n)
    low = torch.tril(torch.ones(N, N, device="cuda", dtype=torch.bool))
    assert torch.equal(got[low], full[low])
    assert torch.equal(got[~low], C0.T[~low])              # the other triangle is not touched


def test_strmm_with_lda_of_2200000():
    M, N = 300, 70
    lda = 2_200_000
    gen = torch.Generator(device="cuda")
    gen.manual_seed(4)
    A = _int_tensor((M, lda), 3, torch.float32, gen)      # column c of the triangle is A[c, :M]
    B = _int_tensor((N, M), 3, torch.float32, gen)
    B0 = B.clone()
    st = clblas_amd.trmm("S", COL, LEFT, UPPER, TRANS, NONUNIT, M, N, 2.0, A, 0, lda, B, 0, M)
    torch.cuda.synchronize()
    assert st == 0
    T = torch.triu(A[:, :M].T.double())                   # M x M upper triangle
    want = 2.0 * (T.T @ B0.T.double())                    # op(A) = T^T
    assert torch.equal(B.T.double(), want)
