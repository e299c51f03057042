"""clblas{S,D,C,Z}gemm on the reference's OWN GEMM test family, by the reference's own method.

The reference's correctness test for GEMM (src/tests/correctness/corr-gemm.cpp:140-200) fills A, B, C
with integers small enough that every partial sum is exactly representable
(src/tests/include/blas-random.h:60-93 with the limits of test-limits.h:20-21) and compares the device
result with a CPU result element by element.  Its instantiations
(src/tests/correctness/test-correctness.cpp:593-700):
  * SmallRange: smallRange^3 = {8, 16, 17, 32, 62, 64, 128, 144, 256}^3 (:157-158), transSet^2 (all nine
    pairs of NoTrans / Trans / ConjTrans), both orders;
  * SmallRange_BigLDA: the same with lda, ldb, ldc = 500, 501, 502;
  * SmallRange_BigLDA_OffSet and SmallRangeEx_0..3: offsets into the buffers (offA = 1 with the big
    leading dimensions; 67 x 135 x 228, 64^3, 128 x 64 x 77, 112 x 86 x 68 with offsets 500 / 501 / 502);
  * SelectedBig_0..3: 2801 x 2903 x 3005 NN, 4777 x 4333 x 5000 NN, 5777 x 5333 x 3000 TN,
    6777 x 3333 x 3000 T/ConjT, both orders.
Here: all four types through the C ABI, compared with assert-equal against the CPU oracle.  The cube
of smallRange is thinned the way the TRSM family test thins its square - every M with three N and
three K, so that every size meets every other in some position - and the three styles (tight, big
leading dimensions, offsets) rotate over the cases so that every transpose pair meets every style in
both orders.  The big shapes run with the library's default tile choice (XCD remapping, row groups,
late start, sliced tail, all together) and are compared in full on the device."""
import itertools

import numpy as np
import pytest
import torch

import clblas_amd
import oracle
from helpers import COL, ROW, NOTRANS, TRANS, CONJ, exact_int_limits, mem_dims

pytestmark = pytest.mark.gpu

TYPES = {"s": np.float32, "d": np.float64, "c": np.complex64, "z": np.complex128}
FN = {"s": clblas_amd.sgemm, "d": clblas_amd.dgemm, "c": clblas_amd.cgemm, "z": clblas_amd.zgemm}
SMALL_RANGE = [8, 16, 17, 32, 62, 64, 128, 144, 256]      # test-correctness.cpp:157-158
TRANSES = [NOTRANS, TRANS, CONJ]                            # transSet
EX_SHAPES = [(67, 135, 228, (500, 0, 0)), (64, 64, 64, (0, 501, 0)), (128, 64, 77, (0, 0, 502)),
             (112, 86, 68, (500, 501, 502))]                # SmallRangeEx_0..3 (:640-665)
BIG = [(NOTRANS, NOTRANS, 2801, 2903, 3005), (NOTRANS, NOTRANS, 4777, 4333, 5000),
       (TRANS, NOTRANS, 5777, 5333, 3000), (TRANS, CONJ, 6777, 3333, 3000)]   # SelectedBig_0..3 (:672-696)


def _scalars(t, case):
    """alpha and beta as the reference draws them: integers (Gaussian integers), alpha not zero
    (blas-random.h:56-60, 78-80); small, so that the exact-integer limits stay useful."""
    rng = np.random.default_rng(7000 + case)
    def one():
        v = int(rng.integers(1, 6)) * (1 if rng.integers(0, 2) else -1)
        if t in "cz":
            return complex(v, int(rng.integers(-3, 4)))
        return float(v)
    return one(), one()


def _limits(t, K, alpha, beta):
    """Largest |entry| of A and B, and of C, that keeps every partial sum exact: the reference's bounds
    (blas-random.h:64-65, 84-88), which helpers.exact_int_limits restates for the real types; a
    complex product has two real products per part and |alpha| a modulus, so the complex limits are
    taken from the real rule with 2 |alpha|_1 and |beta|_1."""
    real = np.float32 if t in "sc" else np.float64
    if t in "cz":
        a1 = 2 * (abs(alpha.real) + abs(alpha.imag))
        b1 = abs(beta.real) + abs(beta.imag)
        return exact_int_limits(2 * K, a1, b1, real)
    return exact_int_limits(K, alpha, beta, real)


def _case(t, order, tA, tB, M, N, K, lds, offs, seed, alpha, beta):
    """Buffers of one call, the oracle's result and the dimensions as passed."""
    dtype = TYPES[t]
    ia, oa = mem_dims(order, tA, M, K)
    ib, ob = mem_dims(order, tB, K, N)
    ic, oc = mem_dims(order, NOTRANS, M, N)
    lda, ldb, ldc = (max(l, i) if l else i for l, i in zip(lds, (ia, ib, ic)))
    la, lc = _limits(t, K, alpha, beta)
    A = oracle.integers(offs[0] + oa * lda, seed, la, dtype)
    B = oracle.integers(offs[1] + ob * ldb, seed + 1, la, dtype)
    C = oracle.integers(offs[2] + oc * ldc, seed + 2, lc, dtype)
    want = C.copy()
    assert oracle.gemm(order, tA, tB, M, N, K, alpha, A, offs[0], lda, B, offs[1], ldb, beta, want, offs[2], ldc) == 0
    return A, B, C, want, lda, ldb, ldc


@pytest.mark.parametrize("order", [ROW, COL], ids=["row", "col"])
@pytest.mark.parametrize("t", list(TYPES))
def test_small_range(t, order):
    assert clblas_amd.setup() == 0
    cases = 0
    for mi, M in enumerate(SMALL_RANGE):
        for N in (M, SMALL_RANGE[(mi + 3) % 9], SMALL_RANGE[(mi + 7) % 9]):
            for K in (SMALL_RANGE[(mi + 1) % 9], SMALL_RANGE[(mi + 4) % 9], SMALL_RANGE[(mi + 8) % 9]):
                for ti, (tA, tB) in enumerate(itertools.product(TRANSES, TRANSES)):
                    cases += 1
                    style = (cases + ti) % 3          # 0: tight, 1: lda/ldb/ldc = 500/501/502, 2: those with offA = 1
                    lds = (500, 501, 502) if style else (0, 0, 0)
                    offs = (1, 0, 0) if style == 2 else (0, 0, 0)
                    alpha, beta = _scalars(t, cases)
                    A, B, C, want, lda, ldb, ldc = _case(t, order, tA, tB, M, N, K, lds, offs, 10 * cases, alpha, beta)
                    dA, dB, dC = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), torch.from_numpy(C).cuda()
                    st = FN[t](order, tA, tB, M, N, K, alpha, dA, offs[0], lda, dB, offs[1], ldb, beta, dC, offs[2], ldc)
                    torch.cuda.synchronize()
                    assert st == 0
                    np.testing.assert_array_equal(dC.cpu().numpy(), want,
                                                  err_msg=str((t, order, tA, tB, M, N, K, style, alpha, beta)))
    print("gemm reference family, small range, %s %s: %d calls, all equal to the oracle" % (
        t, "col" if order == COL else "row", cases))


@pytest.mark.parametrize("order", [ROW, COL], ids=["row", "col"])
@pytest.mark.parametrize("t", list(TYPES))
def test_small_range_ex_offsets(t, order):
    """SmallRangeEx_0..3: single shapes with offsets of 500 / 501 / 502 elements into A / B / C, all nine
    transpose pairs."""
    assert clblas_amd.setup() == 0
    for si, (M, N, K, offs) in enumerate(EX_SHAPES):
        for ti, (tA, tB) in enumerate(itertools.product(TRANSES, TRANSES)):
            alpha, beta = _scalars(t, 500 + 9 * si + ti)
            A, B, C, want, lda, ldb, ldc = _case(t, order, tA, tB, M, N, K, (0, 0, 0), offs, 9000 + 30 * si + 3 * ti, alpha, beta)
            dA, dB, dC = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), torch.from_numpy(C).cuda()
            st = FN[t](order, tA, tB, M, N, K, alpha, dA, offs[0], lda, dB, offs[1], ldb, beta, dC, offs[2], ldc)
            torch.cuda.synchronize()
            assert st == 0
            np.testing.assert_array_equal(dC.cpu().numpy(), want, err_msg=str((t, order, tA, tB, M, N, K, offs)))


# The real types take all four big shapes in both orders; the complex types (eight real multiply-adds per
# element and step, on the CPU oracle too) take SelectedBig_0 in both orders and the T / ConjT shape once.
BIG_CASES = ([(t, order, b) for t in "sd" for order in (COL, ROW) for b in range(4)] +
             [(t, order, 0) for t in "cz" for order in (COL, ROW)] + [("c", COL, 3), ("z", ROW, 3)])


@pytest.mark.parametrize("t,order,b", BIG_CASES,
                         ids=["%s-%s-big%d" % (t, "col" if o == COL else "row", b) for t, o, b in BIG_CASES])
def test_selected_big(t, order, b):
    """Default tile choice, the whole matrix compared on the device with the oracle's result (and what
    lies between the columns of C, none here, would have to be unchanged: the buffers are compared whole)."""
    assert clblas_amd.setup() == 0
    tA, tB, M, N, K = BIG[b]
    alpha, beta = _scalars(t, 900 + b)
    A, B, C, want, lda, ldb, ldc = _case(t, order, tA, tB, M, N, K, (0, 0, 0), (0, 0, 0), 20000 + 10 * b, alpha, beta)
    dA, dB, dC = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), torch.from_numpy(C).cuda()
    st = FN[t](order, tA, tB, M, N, K, alpha, dA, 0, lda, dB, 0, ldb, beta, dC, 0, ldc)
    torch.cuda.synchronize()
    assert st == 0
    what = clblas_amd.last_dispatch()[0]
    dW = torch.from_numpy(want).cuda()
    if not torch.equal(dC, dW):
        bad = torch.nonzero(dC != dW).flatten()
        raise AssertionError("%d of %d elements differ, first at %d (%s)" % (bad.numel(), dW.numel(), int(bad[0]), what))
    assert bool(torch.isfinite(torch.view_as_real(dC) if dC.is_complex() else dC).all())
