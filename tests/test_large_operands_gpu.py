"""Operands beyond 2^31 elements: the header accepts dimensions up to 2^31 - 513 and every offset in
the kernels is 64-bit; these two cases put element indices past 2^31 (and past 2^32 bytes many times
over) through SGEMM and DTRSM.

SGEMM 47000 x 47000 x 64 (C: 2.2e9 elements, 8.8 GB): integer-valued A and B, C pre-filled with NaN
and beta = 0, so (i) every element must have been written, (ii) sampled elements - among them the last
rows / columns and indices past 2^31 - must equal the exact integer product, (iii) C v = A (B v) for
the whole matrix.  DTRSM with a 300 x 7 200 000 right-hand side (2.16e9 elements, 17 GB): sampled
columns, the first and the last among them, against the long double substitution."""
import numpy as np
import pytest
import torch

import clblas_amd
import oracle
from helpers import COL, NOTRANS, LEFT, LOWER, NONUNIT

pytestmark = pytest.mark.gpu


def test_sgemm_c_beyond_2_31_elements():
    M = N = 47000
    K = 64
    assert M * N > 2 ** 31
    A = oracle.integers(M * K, 1, 8, np.float32)      # column-major M x K
    B = oracle.integers(K * N, 2, 8, np.float32)      # column-major K x N
    dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    dC = torch.full((M * N,), float("nan"), device="cuda", dtype=torch.float32)
    st = clblas_amd.sgemm(COL, NOTRANS, NOTRANS, M, N, K, 2.0, dA, 0, M, dB, 0, K, 0.0, dC, 0, M)
    torch.cuda.synchronize()
    assert st == 0, st
    assert not bool(torch.isnan(dC).any())
    # sampled elements, exact (|sum| <= 2 * 64 * 49 fits fp32 exactly)
    rng = np.random.default_rng(3)
    rows = np.concatenate([[0, M - 1, 0, M - 1, 255, 256], rng.integers(0, M, 3000), rng.integers(M - 300, M, 300)])
    cols = np.concatenate([[0, 0, N - 1, N - 1, N - 1, N - 2], rng.integers(0, N, 3000), rng.integers(N - 300, N, 300)])
    idx = torch.from_numpy(rows.astype(np.int64) + cols.astype(np.int64) * M).cuda()
    assert int(idx.max()) > 2 ** 31
    got = dC[idx].cpu().numpy()
    Am, Bm = A.reshape(K, M).T.astype(np.float64), B.reshape(N, K).T.astype(np.float64)   # M x K, K x N
    want = 2.0 * np.einsum("ik,ki->i", Am[rows], Bm[:, cols])
    assert np.array_equal(got.astype(np.float64), want)
    # the whole matrix through a vector: C v = 2 A (B v), exact in double precision for integer data
    v = torch.randint(-3, 4, (N,), device="cuda", dtype=torch.float64)
    Cv = torch.zeros(M, device="cuda", dtype=torch.float64)
    Cm = dC.view(N, M)                                   # Cm[n, m] = C(m, n)
    step = 4000
    for n0 in range(0, N, step):                         # in slabs, to keep the double precision copy small
        Cv += Cm[n0:n0 + step].double().T @ v[n0:n0 + step]
    want_v = 2.0 * (dA.view(K, M).T.double() @ (dB.view(N, K).T.double() @ v))
    assert torch.equal(Cv, want_v)


def test_dtrsm_b_beyond_2_31_elements():
    M, N = 300, 7_200_000
    assert M * N > 2 ** 31
    A = oracle.triangular(M, M, True, 5, np.float64)
    dA = torch.from_numpy(A).cuda()
    gen = torch.Generator(device="cuda")
    gen.manual_seed(77)
    dB = torch.randn(M * N, device="cuda", dtype=torch.float64, generator=gen)
    rng = np.random.default_rng(4)
    cols = np.unique(np.concatenate([[0, 1, 15, 16, N - 17, N - 16, N - 2, N - 1], rng.integers(0, N, 40),
                                     rng.integers(N - 100000, N, 16)]))
    cidx = torch.from_numpy(cols.astype(np.int64)).cuda()
    B0 = dB.view(N, M).index_select(0, cidx).cpu().numpy()        # (ncols, M): the sampled right-hand sides
    st = clblas_amd.dtrsm(COL, LEFT, LOWER, NOTRANS, NONUNIT, M, N, 1.5, dA, 0, M, dB, 0, M)
    torch.cuda.synchronize()
    assert st == 0, st
    assert bool(torch.isfinite(dB).all())
    X = dB.view(N, M).index_select(0, cidx).cpu().numpy()
    Bs = np.ascontiguousarray(B0).ravel()                          # column-major M x ncols
    want = oracle.trsm_hp(COL, LEFT, LOWER, NOTRANS, NONUNIT, M, len(cols), 1.5, A, 0, M, Bs, 0, M, list(range(len(cols))))
    assert np.abs(X - want).max() <= 32 * M * np.finfo(np.float64).eps * np.abs(want).max()
