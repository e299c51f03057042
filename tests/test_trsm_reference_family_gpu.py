"""clblas{S,D,C,Z}trsm on the reference's OWN test inputs, judged by the reference's own bound.

Inputs: the family of randomTrsmMatrices (src/tests/include/blas-random.h:205-372, restated in
oracle/trsm_reftest.inc): integer entries, non-unit diagonals spread over a factor 100 with
|a_ii| up to 2^7 (fp32) / 2^5 (fp64), off-diagonal entries that use up each row's diagonal
dominance budget, right-hand sides up to 2^16 / 2^47 times the diagonal, NaN in everything
that must not be read.  Shapes: the reference's smallRange and its big shapes
(src/tests/correctness/test-correctness.cpp:146-160, 910-1011), all side / triangle /
transpose / diagonal variants, both orders, all four types.

Bars:
  * the per-element bound trsmDelta of src/tests/correctness/trsm-delta.h:44-240 (restated in
    helpers.trsm_ref_delta), applied to |X - X_hp| where X_hp is the substitution solution in
    long double (the reference applies it to the difference from a CPU BLAS result in the
    working precision, so this is the stricter use of the same bound);
  * normwise backward error <= 2 n eps, evaluated in double precision;
  * no NaN in the result (nothing outside the referenced triangle was read) and nothing
    outside the M x N result written.
Also pins what a zero on a non-unit diagonal does here (Inf/NaN from that equation on; the
reference's inversion kernel reads it as 1, trtri/diag_dtrtri_lower_128_16.cpp:93-96)."""
import itertools

import numpy as np
import pytest
import torch

import clblas_amd
import oracle
from helpers import (COL, ROW, NOTRANS, TRANS, CONJ, UPPER, LOWER, UNIT, NONUNIT, LEFT, RIGHT, logical_view,
                     trsm_ref_delta)

pytestmark = pytest.mark.gpu

TYPES = {"s": np.float32, "d": np.float64, "c": np.complex64, "z": np.complex128}
FN = {"s": clblas_amd.strsm, "d": clblas_amd.dtrsm, "c": clblas_amd.ctrsm, "z": clblas_amd.ztrsm}
SMALL_RANGE = [8, 16, 17, 32, 62, 64, 128, 144, 256]      # test-correctness.cpp:157-158
TRANSES = [NOTRANS, TRANS, CONJ]                            # transSet
ALPHAS = {"s": [1.0, 2.0, -3.0], "d": [1.0, 2.0, -3.0], "c": [1.0, 2.0 - 1.0j, -3.0], "z": [1.0, 2.0 - 1.0j, -3.0]}


def _unit_roundoff(dtype):
    return np.finfo(np.dtype(dtype)).eps / 2


def _check_against_hp(t, order, side, uplo, tA, diag, M, N, alpha, A, offA, lda, B0, offB, ldb, rhs, Xsel):
    """Xsel: (len(rhs), n) the library's solutions of the right-hand sides `rhs`."""
    dtype = np.dtype(TYPES[t])
    n = M if side == LEFT else N
    Xhp = oracle.trsm_hp(order, side, uplo, tA, diag, M, N, alpha, A, offA, lda, B0, offB, ldb, rhs)
    Av = logical_view(A, order, NOTRANS, n, n, offA, lda)
    Bv = logical_view(B0, order, NOTRANS, M, N, offB, ldb)
    absd = np.abs(np.diagonal(Av)).astype(np.float64) if diag == NONUNIT else np.ones(n)
    absb = np.abs(Bv[:, rhs].T if side == LEFT else Bv[rhs, :]).astype(np.float64)
    delta = trsm_ref_delta(dtype, side, uplo, tA, diag, alpha, absd, absb)
    diff = Xsel.astype(np.complex128 if dtype.kind == "c" else np.float64) - Xhp
    worst = np.maximum(np.abs(diff.real), np.abs(diff.imag)) if dtype.kind == "c" else np.abs(diff)
    # an element with a zero bound (b and everything before it zero) must be reproduced exactly
    ratio = np.where(delta > 0, worst / np.where(delta > 0, delta, 1), np.where(worst > 0, np.inf, 0))
    return float(ratio.max()), Xhp


def _backward_error_host(order, side, uplo, tA, diag, M, N, alpha, A, offA, lda, B0, X, offB, ldb):
    n = M if side == LEFT else N
    wide = np.complex128 if np.dtype(X.dtype).kind == "c" else np.float64
    Am = np.nan_to_num(logical_view(A, order, NOTRANS, n, n, offA, lda).astype(wide))
    Am = np.triu(Am) if uplo == UPPER else np.tril(Am)
    if diag == UNIT:
        np.fill_diagonal(Am, 1.0)
    if tA != NOTRANS:
        Am = Am.T
    if tA == CONJ:
        Am = Am.conj()
    Xm = logical_view(X, order, NOTRANS, M, N, offB, ldb).astype(wide)
    Bm = logical_view(B0, order, NOTRANS, M, N, offB, ldb).astype(wide)
    R = (Am @ Xm if side == LEFT else Xm @ Am) - alpha * Bm
    nrm = lambda Z: np.abs(Z).sum(axis=1).max()
    return nrm(R) / (nrm(Am) * nrm(Xm) + abs(alpha) * nrm(Bm))


@pytest.mark.parametrize("order", [ROW, COL], ids=["row", "col"])
@pytest.mark.parametrize("t", list(TYPES))
def test_small_range(t, order):
    """smallRange x smallRange (the square sizes and, for every M, three of the nine N), every
    variant, tight / padded leading dimensions (500 / 501) and offsets as the reference's
    SmallRange, SmallRange_BigLDA and SmallRangeEx instantiations."""
    dtype = TYPES[t]
    u = _unit_roundoff(dtype)
    worst_ratio, worst_be, cases = 0.0, 0.0, 0
    for mi, M in enumerate(SMALL_RANGE):
        for N in sorted({M, SMALL_RANGE[(mi + 3) % 9], SMALL_RANGE[(mi + 7) % 9]}):
            for side, uplo, diag in itertools.product([LEFT, RIGHT], [UPPER, LOWER], [UNIT, NONUNIT]):
                n = M if side == LEFT else N
                inner_b = M if order == COL else N
                cases += 1
                style = cases % 3   # 0: tight, 1: big leading dimensions, 2: offsets
                lda, ldb = (500, 501) if style == 1 else (n, inner_b)
                offA, offB = (500, 501) if style == 2 else (0, 0)
                alpha = ALPHAS[t][cases % 3]
                A, B0 = oracle.trsm_ref_inputs(dtype, order, side, uplo, diag, M, N, alpha, offA, lda, offB, ldb,
                                               1000 + cases)
                dA, dB0 = torch.from_numpy(A).cuda(), torch.from_numpy(B0).cuda()
                for tA in TRANSES:
                    dB = dB0.clone()
                    st = FN[t](order, side, uplo, tA, diag, M, N, alpha, dA, offA, lda, dB, offB, ldb)
                    torch.cuda.synchronize()
                    assert st == 0
                    got = dB.cpu().numpy()
                    Xv = logical_view(got, order, NOTRANS, M, N, offB, ldb)
                    tag = (t, order, side, uplo, tA, diag, M, N, style, alpha)
                    assert np.isfinite(Xv).all(), tag
                    mask = np.ones(got.size, dtype=bool)
                    logical_view(mask, order, NOTRANS, M, N, offB, ldb)[:] = False
                    assert np.array_equal(got[mask], B0[mask], equal_nan=True), tag
                    rhs = list(range(N if side == LEFT else M))
                    Xsel = np.ascontiguousarray(Xv.T if side == LEFT else Xv)
                    ratio, _ = _check_against_hp(t, order, side, uplo, tA, diag, M, N, alpha, A, offA, lda, B0, offB, ldb,
                                                 rhs, Xsel)
                    assert ratio <= 1.0, (tag, ratio)
                    be = _backward_error_host(order, side, uplo, tA, diag, M, N, alpha, A, offA, lda, B0, got, offB, ldb)
                    assert be <= 2 * n * 2 * u, (tag, be)
                    worst_ratio, worst_be = max(worst_ratio, ratio), max(worst_be, be / (2 * n * 2 * u))
    print("trsm reference family, small range, %s %s: %d inputs x 3 transposes, worst |X - X_hp| / delta = %.3g, "
          "worst backward error / (2 n eps) = %.3g" % (t, "col" if order == COL else "row", cases, worst_ratio, worst_be))


BIG = [(2801, 2903), (4567, 4321), (6567, 3321)]          # test-correctness.cpp:986-1011
# the variant the reference itself runs at each of these shapes (both orders)
REF_VARIANT = {(2801, 2903): (RIGHT, UPPER, TRANS, NONUNIT), (4567, 4321): (RIGHT, UPPER, TRANS, NONUNIT),
               (6567, 3321): (LEFT, LOWER, TRANS, UNIT)}


def _dev_view(buf, order, rows, cols, off, ld):
    """rows x cols strided view of a matrix inside a flat device buffer."""
    strides = (1, ld) if order == COL else (ld, 1)
    return torch.as_strided(buf, (rows, cols), strides, off)


def _big_case(t, order, side, uplo, diag, M, N, transes, seed):
    dtype = np.dtype(TYPES[t])
    u = _unit_roundoff(dtype)
    n = M if side == LEFT else N
    lda, ldb = n, (M if order == COL else N)
    alpha = ALPHAS[t][seed % 3]
    A, B0 = oracle.trsm_ref_inputs(dtype, order, side, uplo, diag, M, N, alpha, 0, lda, 0, ldb, seed)
    dA, dB0 = torch.from_numpy(A).cuda(), torch.from_numpy(B0).cuda()
    wide = torch.complex128 if dtype.kind == "c" else torch.float64
    Am = torch.nan_to_num(_dev_view(dA, order, n, n, 0, lda).to(wide), nan=0.0)
    Am = torch.triu(Am) if uplo == UPPER else torch.tril(Am)
    if diag == UNIT:
        Am.diagonal().fill_(1.0)
    Bw = _dev_view(dB0, order, M, N, 0, ldb).to(wide)
    nr = N if side == LEFT else M
    rng = np.random.default_rng(seed)
    rhs = sorted(set([0, 1, 15, 16, 31, 32, nr // 2, nr - 2, nr - 1] + list(rng.integers(0, nr, 12))))
    out = []
    for tA in transes:
        dB = dB0.clone()
        st = FN[t](order, side, uplo, tA, diag, M, N, alpha, dA, 0, lda, dB, 0, ldb)
        torch.cuda.synchronize()
        tag = (t, order, side, uplo, tA, diag, M, N, alpha)
        assert st == 0, tag
        Xd = _dev_view(dB, order, M, N, 0, ldb)
        assert bool(torch.isfinite(torch.view_as_real(Xd) if dtype.kind == "c" else Xd).all()), tag
        # normwise backward error over the whole problem, in double precision on the device
        op = Am if tA == NOTRANS else (Am.T.conj() if tA == CONJ else Am.T)
        Xw = Xd.to(wide)
        R = (op @ Xw if side == LEFT else Xw @ op) - alpha * Bw
        nrm = lambda Z: float(Z.abs().sum(dim=1).max())
        be = nrm(R) / (nrm(op) * nrm(Xw) + abs(alpha) * nrm(Bw))
        assert be <= 2 * n * 2 * u, (tag, be)
        # the reference's per-element bound on sampled right-hand sides against the long double solution
        idx = torch.tensor(rhs, device="cuda")
        Xsel = (Xd.index_select(1, idx).T if side == LEFT else Xd.index_select(0, idx)).contiguous().cpu().numpy()
        ratio, _ = _check_against_hp(t, order, side, uplo, tA, diag, M, N, alpha, A, 0, lda, B0, 0, ldb, rhs, Xsel)
        assert ratio <= 1.0, (tag, ratio)
        out.append((ratio, be / (2 * n * 2 * u)))
        del dB, Xw, R
    return out


@pytest.mark.parametrize("shape", BIG, ids=["%dx%d" % s for s in BIG])
@pytest.mark.parametrize("t", list(TYPES))
def test_big_shapes_all_variants(t, shape):
    """Every side / triangle / transpose / diagonal variant at the reference's big shapes:
    column-major throughout, plus row-major for the smallest of them and for the variant that the
    reference itself runs at each shape."""
    M, N = shape
    seed = 7000
    worst = [0.0, 0.0]
    cases = 0
    for order in ([COL, ROW] if shape == BIG[0] else [COL]):
        for side, uplo, diag in itertools.product([LEFT, RIGHT], [UPPER, LOWER], [UNIT, NONUNIT]):
            seed += 1
            for ratio, be in _big_case(t, order, side, uplo, diag, M, N, TRANSES, seed):
                worst = [max(worst[0], ratio), max(worst[1], be)]
                cases += 1
    if shape != BIG[0]:
        side, uplo, tA, diag = REF_VARIANT[shape]
        for ratio, be in _big_case(t, ROW, side, uplo, diag, M, N, [tA], seed + 1):
            worst = [max(worst[0], ratio), max(worst[1], be)]
            cases += 1
    print("trsm reference family, %d x %d, %s: %d solves, worst |X - X_hp| / delta = %.3g, worst backward error / "
          "(2 n eps) = %.3g" % (M, N, t, cases, worst[0], worst[1]))


@pytest.mark.parametrize("t", list(TYPES))
def test_zero_on_a_non_unit_diagonal(t):
    """A zero diagonal entry: the equations before it (in substitution order) are solved as if the
    system ended there; from that equation on every value is Inf or NaN.  With a unit diagonal
    the stored zero is never read."""
    dtype = np.dtype(TYPES[t])
    M, N = 300, 40
    for uplo, tA, p in ((LOWER, NOTRANS, 137), (UPPER, NOTRANS, 200), (LOWER, TRANS, 20), (UPPER, CONJ, 271)):
        A, B0 = oracle.trsm_ref_inputs(dtype, COL, LEFT, uplo, NONUNIT, M, N, 1.0, 0, M, 0, M, 99)
        Av = logical_view(A, COL, NOTRANS, M, M, 0, M)
        Av[p, p] = 0
        dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B0).cuda()
        assert FN[t](COL, LEFT, uplo, tA, NONUNIT, M, N, 1.0, dA, 0, M, dB, 0, M) == 0
        torch.cuda.synchronize()
        X = logical_view(dB.cpu().numpy(), COL, NOTRANS, M, N, 0, M)
        forward = (uplo == LOWER) == (tA == NOTRANS)      # equations run from row 0 down
        before = slice(0, p) if forward else slice(p + 1, M)
        after = slice(p, M) if forward else slice(0, p + 1)
        assert np.isfinite(X[before]).all(), (t, uplo, tA)
        assert not np.isfinite(X[after]).any(), (t, uplo, tA)
        Xhp = oracle.trsm_hp(COL, LEFT, uplo, tA, NONUNIT, M, N, 1.0, np.nan_to_num(A), 0, M, B0, 0, M, list(range(N)))
        want = Xhp.T[before]
        assert np.abs(X[before] - want).max() <= 64 * M * _unit_roundoff(dtype) * np.abs(want).max(), (t, uplo, tA)
    # unit diagonal: whatever is stored on the diagonal (here zeros) is not part of the matrix
    A, B0 = oracle.trsm_ref_inputs(dtype, COL, LEFT, LOWER, UNIT, M, N, 1.0, 0, M, 0, M, 98)
    Av = logical_view(A, COL, NOTRANS, M, M, 0, M)
    Av[np.tril_indices(M, -1)] = (np.arange(M * (M - 1) // 2) % 3 - 1) / 4.0   # some off-diagonal entries
    np.fill_diagonal(Av, 0)
    dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B0).cuda()
    assert FN[t](COL, LEFT, LOWER, NOTRANS, UNIT, M, N, 1.0, dA, 0, M, dB, 0, M) == 0
    torch.cuda.synchronize()
    X = logical_view(dB.cpu().numpy(), COL, NOTRANS, M, N, 0, M)
    Xhp = oracle.trsm_hp(COL, LEFT, LOWER, NOTRANS, UNIT, M, N, 1.0, A, 0, M, B0, 0, M, list(range(N))).T
    assert np.isfinite(X).all()
    assert np.abs(X - Xhp).max() <= 64 * M * _unit_roundoff(dtype) * np.abs(Xhp).max()


@pytest.mark.parametrize("t", list(TYPES))
def test_dense_triangles_with_graded_diagonals(t):
    """A harder family than the reference's (whose big matrices are mostly zero away from one
    corner): dense triangles, diagonals of both signs spread over a factor 100, every row's
    off-diagonal entries summing to 0.95 of its diagonal in magnitude.  Bar: componentwise
    backward error |op(A) X - alpha B| <= 2 (n + 2) u (|op(A)| |X| + |alpha| |B|), evaluated in
    double precision on the device (the factor 2 leaves room for the evaluation itself in the
    double precision types)."""
    dtype = np.dtype(TYPES[t])
    u = _unit_roundoff(dtype)
    wide = torch.complex128 if dtype.kind == "c" else torch.float64
    gen = torch.Generator(device="cuda")
    worst = 0.0
    case = 0
    for (M, N) in ((700, 333), (2049, 515), (3000, 2900)):
        for side, uplo in itertools.product([LEFT, RIGHT], [UPPER, LOWER]):
            n = M if side == LEFT else N
            gen.manual_seed(100 + case)
            shape = (n, n, 2) if dtype.kind == "c" else (n, n)
            W = torch.rand(shape, device="cuda", dtype=torch.float64, generator=gen) * 2 - 1
            W = torch.view_as_complex(W) if dtype.kind == "c" else W
            W = torch.triu(W, 1) if uplo == UPPER else torch.tril(W, -1)
            d = torch.exp(torch.rand(n, device="cuda", dtype=torch.float64, generator=gen) * np.log(100.0))
            sign = torch.where(torch.rand(n, device="cuda", generator=gen) < 0.5, -1.0, 1.0).to(torch.float64)
            rows = W.abs().sum(dim=1).clamp_min(1e-300)
            W = W * (0.95 * d / rows)[:, None]
            W = W + torch.diag((d * sign).to(W.dtype))
            Alog = W.to(torch.from_numpy(np.empty(0, dtype=dtype)).dtype)          # n x n logical, working precision
            bshape = (M, N, 2) if dtype.kind == "c" else (M, N)
            Blog = torch.rand(bshape, device="cuda", dtype=torch.float64, generator=gen) * 2 - 1
            Blog = (torch.view_as_complex(Blog) if dtype.kind == "c" else Blog).to(Alog.dtype)
            # column-major buffers; NaN in the triangle that must not be read
            poison = torch.full_like(Alog, float("nan"))
            keep = torch.triu(torch.ones(n, n, device="cuda", dtype=torch.bool)) if uplo == UPPER else \
                torch.tril(torch.ones(n, n, device="cuda", dtype=torch.bool))
            dA = torch.where(keep, Alog, poison).T.contiguous().view(-1)
            for tA in TRANSES:
                case += 1
                alpha = ALPHAS[t][case % 3]
                dB = Blog.T.contiguous().view(-1).clone()
                st = FN[t](COL, side, uplo, tA, NONUNIT, M, N, alpha, dA, 0, n, dB, 0, M)
                torch.cuda.synchronize()
                assert st == 0
                X = dB.view(N, M).T.to(wide)
                Aw, Bw = Alog.to(wide), Blog.to(wide)
                op = Aw if tA == NOTRANS else (Aw.T.conj() if tA == CONJ else Aw.T)
                R = ((op @ X if side == LEFT else X @ op) - alpha * Bw).abs()
                D = (op.abs() @ X.abs() if side == LEFT else X.abs() @ op.abs()) + abs(alpha) * Bw.abs()
                ratio = float((R / D).max()) / (2 * (n + 2) * u)
                tag = (t, side, uplo, tA, M, N, alpha)
                assert bool(torch.isfinite(R).all()) and ratio <= 1.0, (tag, ratio)
                worst = max(worst, ratio)
                del X, R, D, dB
            del W, Alog, Blog, dA
    print("trsm dense graded family, %s: %d solves, worst componentwise backward error / (2 (n+2) u) = %.3g"
          % (t, case, worst))
