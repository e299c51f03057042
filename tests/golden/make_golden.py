"""Writes tests/golden/fixed_cases.json: the fixed-input cases the reference's own files hold
for the xGEMM / xTRSM path and its SYMM / SYRK / TRMM neighbours, with expected outputs computed here in exact rational arithmetic
(python Fractions) -- independent of both the oracle and the HIP library.

Sources of the INPUT DATA (data only; no reference code is run or copied):
  * README.md:77-156            row-major SGEMM 4x5 * 5x3, alpha=10, beta=20, zero offsets
  * src/samples/example_sgemm.c:31-73,156-160  same matrices, sub-problem (M-1,N-1,K-1) at
                                offA=K+1, offB=N+1, offC=N+1
  * src/samples/example_strsm.c:30-63,140-142  row-major STRSM left/upper/notrans/nonunit,
                                sub-problem (M-1,N-1) at offA=M+1, offB=N+1, alpha=10
  * src/tests/correctness/corr-trsm.cpp:240-291,313-452  TRSM_extratest: column-major,
                                left/upper/notrans/nonunit, M=5, N=2, lda=ldb=32,
                                a_rr=r+1, a_rc=1 (c>r), b_r = sum(1..M)-sum(1..r+1)+(r+1)^2
                                => x_r = r+1 (closed form)
  * src/samples/example_ctrsm.c:30-63,145-147  the same numbers as FloatComplex with zero imaginary
                                parts, same call (clblasCtrsm)
  * src/samples/example_ssymm.c:30-63,146-148  row-major SSYMM left/lower, M=4, N=3,
                                alpha=10, beta=20, upper triangle of A filled with -1
  * src/samples/example_ssyrk.c:30-63,142-144  row-major SSYRK upper/notrans, sub-problem
                                (N-1, K-1) at offA=K+1, offC=N+1, alpha=10, beta=20
  * src/samples/example_ssyr2k.c:30-73,156-159  row-major SSYR2K upper/notrans, sub-problem (N-1, K-1) at
                                offA=offB=K+1, offC=N+1, alpha=10, beta=20, B == A
  * src/samples/example_cherk.cpp:30-68,152-154  column-major CHERK lower/notrans, N=5, K=4, A all ones
                                (lda=5), alpha=10, beta=1, C lower triangle with non-zero imaginary diagonal
  * src/samples/example_cher2k.c:30-67,153-154  column-major CHER2K lower/notrans, alpha=(10,1), beta=1,
                                the same C
  * src/samples/example_chemm.cpp:30-64,146-148  row-major CHEMM left/lower, M=4, N=3, alpha=(10,10),
                                beta=(20,20), complex diagonal of A, upper triangle filled with (-1,-1)
  * src/samples/example_strmm.c:30-63,140-142  row-major STRMM left/upper/notrans/nonunit,
                                sub-problem (M-1, N-1) at offA=M+1, offB=N+1, alpha=10

Run:  python tests/golden/make_golden.py
"""
import json
import os
from fractions import Fraction as F

HERE = os.path.dirname(os.path.abspath(__file__))

ROW, COL = 0, 1
N_, T_ = 0, 1
UPPER, LOWER = 0, 1
UNIT, NONUNIT = 0, 1
LEFT, RIGHT = 0, 1


def a_index(order, trans, r, c, ld):
    """Buffer index of element (r,c) of op(X) (src/library/blas/AutoGemm/KernelOpenCL.py:68-81)."""
    if (order == COL) == (trans == N_):
        return r + c * ld
    return r * ld + c


def gemm_exact(order, tA, tB, M, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc):
    out = [F(x) for x in C]
    for m in range(M):
        for n in range(N):
            s = F(0)
            for k in range(K):
                s += F(A[offA + a_index(order, tA, m, k, lda)]) * F(B[offB + a_index(order, tB, k, n, ldb)])
            ci = offC + a_index(order, N_, m, n, ldc)
            out[ci] = F(alpha) * s + F(beta) * F(C[ci])
    return out


def trsm_exact(order, side, uplo, tA, diag, M, N, alpha, A, offA, lda, B, offB, ldb):
    """Solves op(A) X = alpha B (left) or X op(A) = alpha B (right) exactly."""
    n = M if side == LEFT else N
    # dense op(A) restricted to its triangle
    opA = [[F(0)] * n for _ in range(n)]
    for r in range(n):
        for c in range(n):
            # (r,c) of op(A) is (c,r) of A when transposed
            rr, cc = (c, r) if tA != N_ else (r, c)
            in_tri = (rr <= cc) if uplo == UPPER else (rr >= cc)
            if not in_tri:
                continue
            if rr == cc and diag == UNIT:
                opA[r][c] = F(1)
            else:
                opA[r][c] = F(A[offA + a_index(order, N_, rr, cc, lda)])
    out = [F(x) for x in B]
    nrhs = N if side == LEFT else M
    for j in range(nrhs):
        # right: x^T solves op(A)^T x^T = alpha b^T
        Tm = opA if side == LEFT else [[opA[c][r] for c in range(n)] for r in range(n)]
        def bidx(i):
            return offB + (a_index(order, N_, i, j, ldb) if side == LEFT else a_index(order, N_, j, i, ldb))
        rhs = [F(alpha) * F(B[bidx(i)]) for i in range(n)]
        # generic exact elimination on a triangular system (forward or backward)
        x = [None] * n
        lower = all(Tm[r][c] == 0 for r in range(n) for c in range(r + 1, n))
        order_rows = range(n) if lower else range(n - 1, -1, -1)
        for r in order_rows:
            s = rhs[r]
            for c in range(n):
                if c != r and x[c] is not None:
                    s -= Tm[r][c] * x[c]
            x[r] = s / Tm[r][r]
        for i in range(n):
            out[bidx(i)] = x[i]
    return out


def tri_dense(order, uplo, tA, diag, n, A, offA, lda):
    """Dense op(A) of a triangular matrix: zeros outside the `uplo` triangle, ones on a unit diagonal."""
    opA = [[F(0)] * n for _ in range(n)]
    for r in range(n):
        for c in range(n):
            rr, cc = (c, r) if tA != N_ else (r, c)
            if not ((rr <= cc) if uplo == UPPER else (rr >= cc)):
                continue
            opA[r][c] = F(1) if (rr == cc and diag == UNIT) else F(A[offA + a_index(order, N_, rr, cc, lda)])
    return opA


def trmm_exact(order, side, uplo, tA, diag, M, N, alpha, A, offA, lda, B, offB, ldb):
    n = M if side == LEFT else N
    T = tri_dense(order, uplo, tA, diag, n, A, offA, lda)
    out = [F(x) for x in B]
    for i in range(M):
        for j in range(N):
            if side == LEFT:
                s = sum(T[i][k] * F(B[offB + a_index(order, N_, k, j, ldb)]) for k in range(n))
            else:
                s = sum(F(B[offB + a_index(order, N_, i, k, ldb)]) * T[k][j] for k in range(n))
            out[offB + a_index(order, N_, i, j, ldb)] = F(alpha) * s
    return out


def syrk_exact(order, uplo, tA, N, K, alpha, A, offA, lda, beta, C, offC, ldc):
    out = [F(x) for x in C]
    for i in range(N):
        for j in range(N):
            if not ((i <= j) if uplo == UPPER else (i >= j)):
                continue
            s = sum(F(A[offA + a_index(order, tA, i, k, lda)]) * F(A[offA + a_index(order, tA, j, k, lda)])
                    for k in range(K))
            ci = offC + a_index(order, N_, i, j, ldc)
            out[ci] = F(alpha) * s + F(beta) * F(C[ci])
    return out


def symm_exact(order, side, uplo, M, N, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc):
    n = M if side == LEFT else N

    def a(r, c):  # symmetric element from the stored triangle
        if not ((r <= c) if uplo == UPPER else (r >= c)):
            r, c = c, r
        return F(A[offA + a_index(order, N_, r, c, lda)])
    out = [F(x) for x in C]
    for i in range(M):
        for j in range(N):
            if side == LEFT:
                s = sum(a(i, k) * F(B[offB + a_index(order, N_, k, j, ldb)]) for k in range(n))
            else:
                s = sum(F(B[offB + a_index(order, N_, i, k, ldb)]) * a(k, j) for k in range(n))
            ci = offC + a_index(order, N_, i, j, ldc)
            out[ci] = F(alpha) * s + F(beta) * F(C[ci])
    return out


class G:
    """Gaussian integer / rational: exact complex arithmetic on Fractions."""

    def __init__(self, re, im=0):
        self.re, self.im = F(re), F(im)

    @staticmethod
    def of(x):
        return x if isinstance(x, G) else (G(x[0], x[1]) if isinstance(x, (list, tuple)) else G(x))

    def __add__(self, o):
        o = G.of(o)
        return G(self.re + o.re, self.im + o.im)

    def __mul__(self, o):
        o = G.of(o)
        return G(self.re * o.re - self.im * o.im, self.re * o.im + self.im * o.re)

    def conj(self):
        return G(self.re, -self.im)

    def pair(self):
        return [float(self.re), float(self.im)]


def gsum(terms):
    s = G(0)
    for t in terms:
        s = s + t
    return s


def syr2k_exact(order, uplo, tAB, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc):
    out = [F(x) for x in C]
    a = lambda i, k: F(A[offA + a_index(order, tAB, i, k, lda)])
    b = lambda i, k: F(B[offB + a_index(order, tAB, i, k, ldb)])
    for i in range(N):
        for j in range(N):
            if not ((i <= j) if uplo == UPPER else (i >= j)):
                continue
            s = sum(a(i, k) * b(j, k) + b(i, k) * a(j, k) for k in range(K))
            ci = offC + a_index(order, N_, i, j, ldc)
            out[ci] = F(alpha) * s + F(beta) * F(C[ci])
    return out


def her2k_exact(order, uplo, trans, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc):
    """C = alpha op(A) op(B)^H + conj(alpha) op(B) op(A)^H + beta C on one triangle, op = identity
    (trans == N_) or conjugate transpose; diagonal real.  B is None: herk, C = alpha op(A) op(A)^H + beta C
    with real alpha."""
    def el(X, off, ld, i, k):   # op(X)(i, k)
        v = G.of(X[off + a_index(order, N_ if trans == N_ else T_, i, k, ld)])
        return v if trans == N_ else v.conj()
    out = [G.of(x) for x in C]
    al = G.of(alpha)
    for i in range(N):
        for j in range(N):
            if not ((i <= j) if uplo == UPPER else (i >= j)):
                continue
            if B is None:
                s = al * gsum(el(A, offA, lda, i, k) * el(A, offA, lda, j, k).conj() for k in range(K))
            else:
                s = al * gsum(el(A, offA, lda, i, k) * el(B, offB, ldb, j, k).conj() for k in range(K)) + \
                    al.conj() * gsum(el(B, offB, ldb, i, k) * el(A, offA, lda, j, k).conj() for k in range(K))
            ci = offC + a_index(order, N_, i, j, ldc)
            c0 = G.of(C[ci])
            if i == j:
                c0 = G(c0.re, 0)
            r = s + G(beta) * c0
            out[ci] = G(r.re, 0) if i == j else r
    return out


def hemm_exact(order, side, uplo, M, N, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc):
    n = M if side == LEFT else N

    def a(r, c):  # Hermitian element from the stored triangle; stored diagonal imaginary parts ignored
        if r == c:
            return G(G.of(A[offA + a_index(order, N_, r, c, lda)]).re, 0)
        if (r <= c) if uplo == UPPER else (r >= c):
            return G.of(A[offA + a_index(order, N_, r, c, lda)])
        return G.of(A[offA + a_index(order, N_, c, r, lda)]).conj()
    out = [G.of(x) for x in C]
    for i in range(M):
        for j in range(N):
            if side == LEFT:
                s = gsum(a(i, k) * G.of(B[offB + a_index(order, N_, k, j, ldb)]) for k in range(n))
            else:
                s = gsum(G.of(B[offB + a_index(order, N_, i, k, ldb)]) * a(k, j) for k in range(n))
            ci = offC + a_index(order, N_, i, j, ldc)
            out[ci] = G.of(alpha) * s + G.of(beta) * G.of(C[ci])
    return out


def as_pairs(v):
    return [G.of(x).pair() for x in v]


def as_floats(v):
    return [float(x) for x in v]


def main():
    cases = {}
    A = [11, 12, 13, 14, 15, 21, 22, 23, 24, 25, 31, 32, 33, 34, 35, 41, 42, 43, 44, 45]
    B = [11, 12, 13, 21, 22, 23, 31, 32, 33, 41, 42, 43, 51, 52, 53]
    C = [11, 12, 13, 21, 22, 23, 31, 32, 33, 41, 42, 43]
    M, N, K = 4, 3, 5
    cases["readme_sgemm"] = dict(
        kind="gemm", dtype="f32", order=ROW, transA=N_, transB=N_, M=M, N=N, K=K, alpha=10, beta=20, A=A, offA=0,
        lda=K, B=B, offB=0, ldb=N, C=C, offC=0, ldc=N,
        expected=as_floats(gemm_exact(ROW, N_, N_, M, N, K, 10, A, 0, K, B, 0, N, 20, C, 0, N)))
    cases["sample_sgemm_offsets"] = dict(
        kind="gemm", dtype="f32", order=ROW, transA=N_, transB=N_, M=M - 1, N=N - 1, K=K - 1, alpha=10, beta=20,
        A=A, offA=K + 1, lda=K, B=B, offB=N + 1, ldb=N, C=C, offC=N + 1, ldc=N,
        expected=as_floats(gemm_exact(ROW, N_, N_, M - 1, N - 1, K - 1, 10, A, K + 1, K, B, N + 1, N, 20, C, N + 1,
                                      N)))
    At = [11, 12, 13, 14, 0, 22, 23, 24, 0, 0, 33, 34, 0, 0, 0, 44]
    Bt = [11, 12, 13, 14, 15, 21, 22, 23, 24, 25, 31, 32, 33, 34, 35, 41, 42, 43, 44, 45]
    cases["sample_strsm_offsets"] = dict(
        kind="trsm", dtype="f32", order=ROW, side=LEFT, uplo=UPPER, transA=N_, diag=NONUNIT, M=3, N=4, alpha=10,
        A=At, offA=5, lda=4, B=Bt, offB=6, ldb=5,
        expected=as_floats(trsm_exact(ROW, LEFT, UPPER, N_, NONUNIT, 3, 4, 10, At, 5, 4, Bt, 6, 5)))
    # TRSM_extratest
    Me, Ne, ld = 5, 2, 32
    Ae = [0.0] * (Me * ld)
    Be = [0.0] * (Ne * ld)
    tri = lambda n: n * (n + 1) // 2
    for i in range(Me):          # column i
        for j in range(Me):      # row j
            Ae[i * ld + j] = float(j + 1) if j == i else (0.0 if j > i else 1.0)
    for i in range(Ne):
        for j in range(Me):
            Be[i * ld + j] = float(tri(Me) - tri(j + 1) + (j + 1) * (j + 1))
    exp = trsm_exact(COL, LEFT, UPPER, N_, NONUNIT, Me, Ne, 1, Ae, 0, ld, Be, 0, ld)
    # closed form from the reference test: X_r = r + 1
    for i in range(Ne):
        for j in range(Me):
            assert exp[i * ld + j] == j + 1
    for dt in ("f32", "f64"):
        cases["extratest_" + dt] = dict(
            kind="trsm", dtype=dt, order=COL, side=LEFT, uplo=UPPER, transA=N_, diag=NONUNIT, M=Me, N=Ne, alpha=1,
            A=Ae, offA=0, lda=ld, B=Be, offB=0, ldb=ld, expected=as_floats(exp), tol=1e-5)
    # SYMM / SYRK / TRMM samples
    As = [11, -1, -1, -1, 21, 22, -1, -1, 31, 32, 33, -1, 41, 42, 43, 44]
    Bs = [11, 12, 13, 21, 22, 23, 31, 32, 33, 41, 42, 43]
    cases["sample_ssymm"] = dict(
        kind="symm", dtype="f32", order=ROW, side=LEFT, uplo=LOWER, M=4, N=3, alpha=10, beta=20, A=As, offA=0, lda=4,
        B=Bs, offB=0, ldb=3, C=list(Bs), offC=0, ldc=3,
        expected=as_floats(symm_exact(ROW, LEFT, LOWER, 4, 3, 10, As, 0, 4, Bs, 0, 3, 20, Bs, 0, 3)))
    Ak = [11, 12, 13, 14, 21, 22, 23, 24, 31, 32, 33, 34, 41, 42, 43, 44, 51, 52, 53, 54]
    Ck = [11, 12, 13, 14, 15, 12, 22, 23, 24, 25, 13, 23, 33, 34, 35, 14, 24, 34, 44, 45, 15, 25, 35, 45, 55]
    cases["sample_ssyrk_offsets"] = dict(
        kind="syrk", dtype="f32", order=ROW, uplo=UPPER, transA=N_, N=4, K=3, alpha=10, beta=20, A=Ak, offA=5, lda=4,
        C=Ck, offC=6, ldc=5,
        expected=as_floats(syrk_exact(ROW, UPPER, N_, 4, 3, 10, Ak, 5, 4, 20, Ck, 6, 5)))
    cases["sample_strmm_offsets"] = dict(
        kind="trmm", dtype="f32", order=ROW, side=LEFT, uplo=UPPER, transA=N_, diag=NONUNIT, M=3, N=4, alpha=10,
        A=At, offA=5, lda=4, B=Bt, offB=6, ldb=5,
        expected=as_floats(trmm_exact(ROW, LEFT, UPPER, N_, NONUNIT, 3, 4, 10, At, 5, 4, Bt, 6, 5)))
    # The CTRSM sample holds the STRSM sample's numbers as complex values with zero imaginary
    # parts, so its exact solution is the real one (imaginary parts stay zero).
    cases["sample_ctrsm_offsets"] = dict(
        kind="trsm", dtype="c64", order=ROW, side=LEFT, uplo=UPPER, transA=N_, diag=NONUNIT, M=3, N=4, alpha=10,
        A=At, offA=5, lda=4, B=Bt, offB=6, ldb=5,
        expected=as_floats(trsm_exact(ROW, LEFT, UPPER, N_, NONUNIT, 3, 4, 10, At, 5, 4, Bt, 6, 5)))
    # SYR2K / HERK / HER2K / HEMM samples.  Complex buffers are lists of [re, im] pairs.
    A2 = [11, 12, 13, 14, 21, 22, 23, 24, 31, 32, 33, 34, 41, 42, 43, 44, 51, 52, 53, 54]
    C2 = [11, 12, 13, 14, 15, 12, 22, 23, 24, 25, 13, 23, 33, 34, 35, 14, 24, 34, 44, 45, 15, 25, 35, 45, 55]
    cases["sample_ssyr2k_offsets"] = dict(
        kind="syr2k", dtype="f32", order=ROW, uplo=UPPER, transA=N_, N=4, K=3, alpha=10, beta=20, A=A2, offA=5,
        lda=4, B=A2, offB=5, ldb=4, C=C2, offC=6, ldc=5,
        expected=as_floats(syr2k_exact(ROW, UPPER, N_, 4, 3, 10, A2, 5, 4, A2, 5, 4, 20, C2, 6, 5)))
    Ch = [[0, 0]] * 25
    for j, (d, im) in enumerate([(11, 1), (22, 2), (33, 4), (44, 5), (55, 6)]):
        Ch[j * 5 + j] = [d, im]
        for i in range(j + 1, 5):
            Ch[j * 5 + i] = [10 * (j + 1) + i + 1, 0]
    Aones = [[1, 0]] * 20
    cases["sample_cherk"] = dict(
        kind="herk", dtype="c64", order=COL, uplo=LOWER, transA=N_, N=5, K=4, alpha=10, beta=1, A=Aones, offA=0,
        lda=5, C=Ch, offC=0, ldc=5,
        expected=as_pairs(her2k_exact(COL, LOWER, N_, 5, 4, 10, Aones, 0, 5, None, 0, 0, 1, Ch, 0, 5)))
    Ah = [[x, 0] for x in A2]
    Bh = [[x, 0] for x in [1, 2, 3, 4, 2, 2, 3, 4, 3, 2, 3, 3, 4, 4, 4, 4, 5, 5, 5, 5]]
    cases["sample_cher2k"] = dict(
        kind="her2k", dtype="c64", order=COL, uplo=LOWER, transA=N_, N=5, K=4, alpha=[10, 1], beta=1, A=Ah, offA=0,
        lda=5, B=Bh, offB=0, ldb=5, C=Ch, offC=0, ldc=5,
        expected=as_pairs(her2k_exact(COL, LOWER, N_, 5, 4, [10, 1], Ah, 0, 5, Bh, 0, 5, 1, Ch, 0, 5)))
    Am = [[11, 12], [-1, -1], [-1, -1], [-1, -1], [21, 22], [22, 23], [-1, -1], [-1, -1],
          [31, 32], [32, 33], [33, 34], [-1, -1], [41, 61], [42, 62], [43, 73], [44, 23]]
    Bm = [[11, -21], [-12, 23], [13, 33], [21, 12], [22, -10], [23, 5], [31, 1], [-32, 65], [33, -1],
          [1, 41], [-33, 42], [12, 43]]
    Cm = [[11, 11], [-12, 12], [13, 33], [21, -32], [22, -1], [23, 0], [31, 13], [-32, 78], [33, 45],
          [41, 14], [0, 42], [43, -1]]
    cases["sample_chemm"] = dict(
        kind="hemm", dtype="c64", order=ROW, side=LEFT, uplo=LOWER, M=4, N=3, alpha=[10, 10], beta=[20, 20], A=Am,
        offA=0, lda=4, B=Bm, offB=0, ldb=3, C=Cm, offC=0, ldc=3,
        expected=as_pairs(hemm_exact(ROW, LEFT, LOWER, 4, 3, [10, 10], Am, 0, 4, Bm, 0, 3, [20, 20], Cm, 0, 3)))
    with open(os.path.join(HERE, "fixed_cases.json"), "w") as f:
        json.dump(cases, f, indent=1)
    print("wrote", len(cases), "cases")


if __name__ == "__main__":
    main()
