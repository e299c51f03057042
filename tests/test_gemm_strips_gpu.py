"""clblas{S,D,C,Z}gemm where a product is made in two or three launches: a dimension that is a few rows or columns
more than a whole number of tiles has its last rows / columns (at most 64) split off as a product of their own
when the tile model prices that lower.  The debug switch CLBLAS_AMD_GEMM_PEEL=2 splits wherever a strip exists,
=0 never does; every result is compared with the CPU oracle on integer data (exact whatever the order of
summation), so the pieces must tile C exactly, with the right operands, offsets and leading dimensions, in both
orders and all transposes.  The default's own choice is exercised on the shapes it was made for."""
import itertools

import numpy as np
import pytest
import torch

import clblas_amd
import oracle
import gpu_util
from helpers import COL, ROW, NOTRANS, TRANS, CONJ, exact_int_limits, mem_dims

pytestmark = pytest.mark.gpu

TYPES = {"s": np.float32, "d": np.float64, "c": np.complex64, "z": np.complex128}
FN = {"s": clblas_amd.sgemm, "d": clblas_amd.dgemm, "c": clblas_amd.cgemm, "z": clblas_amd.zgemm}
# (M, N, K): a strip of rows, of columns, of both, and strips of 32 and of the full 64
SHAPES = [(1030, 1100, 70), (1100, 1027, 130), (1025, 1056, 33), (1056, 1152, 64), (2049, 1025, 40), (1088, 1100, 50)]


def _case(t, order, tA, tB, M, N, K, seed, pad, offs, alpha, beta):
    dtype = TYPES[t]
    real = np.float32 if t in "sc" else np.float64
    ia, oa = mem_dims(order, tA, M, K)
    ib, ob = mem_dims(order, tB, K, N)
    ic, oc = mem_dims(order, NOTRANS, M, N)
    lda, ldb, ldc = ia + pad, ib + pad, ic + pad
    if t in "cz":
        la, lc = exact_int_limits(2 * K, 2 * (abs(alpha.real) + abs(alpha.imag)), abs(beta.real) + abs(beta.imag), real)
    else:
        la, lc = exact_int_limits(K, alpha, beta, real)
    A = oracle.integers(offs[0] + oa * lda, seed, la, dtype)
    B = oracle.integers(offs[1] + ob * ldb, seed + 1, la, dtype)
    C = oracle.integers(offs[2] + oc * ldc, seed + 2, lc, dtype)
    want = C.copy()
    assert oracle.gemm(order, tA, tB, M, N, K, alpha, A, offs[0], lda, B, offs[1], ldb, beta, want, offs[2], ldc) == 0
    return A, B, C, want, lda, ldb, ldc


@pytest.mark.parametrize("order", [ROW, COL], ids=["row", "col"])
@pytest.mark.parametrize("t", list(TYPES))
def test_strips_forced(t, order):
    assert clblas_amd.setup() == 0
    transes = [NOTRANS, TRANS, CONJ] if t in "cz" else [NOTRANS, TRANS]
    case = 0
    for (M, N, K) in SHAPES:
        for tA, tB in itertools.product(transes, transes):
            case += 1
            alpha, beta = (complex(2, -1), complex(-1, 2)) if t in "cz" else (2.0, -3.0)
            if case % 4 == 0:
                beta = beta * 0           # C is then never read
            pad, offs = (0, (0, 0, 0)) if case % 2 else (3, (5, 7, 11))
            A, B, C, want, lda, ldb, ldc = _case(t, order, tA, tB, M, N, K, 100 * case, pad, offs, alpha, beta)
            dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
            launches = {}
            for mode in (2, 0):
                dC = torch.from_numpy(C).cuda()
                with gpu_util.debug_env(CLBLAS_AMD_GEMM_PEEL=mode):
                    n0 = clblas_amd.last_dispatch()[1]
                    st = FN[t](order, tA, tB, M, N, K, alpha, dA, offs[0], lda, dB, offs[1], ldb, beta, dC, offs[2], ldc)
                    torch.cuda.synchronize()
                    launches[mode] = clblas_amd.last_dispatch()[1] - n0
                assert st == 0
                np.testing.assert_array_equal(dC.cpu().numpy(), want, err_msg=str((t, order, tA, tB, M, N, K, mode)))
            assert launches[2] > launches[0], (launches, M, N, K)   # the strips were launches of their own


@pytest.mark.parametrize("t,M,N,K", [("s", 8193, 8193, 1024), ("s", 4097, 4095, 1031), ("d", 4100, 4100, 1000),
                                     ("s", 10000, 2000, 512), ("d", 2050, 8200, 600)])
def test_default_choice_on_shapes_just_over_whole_tiles(t, M, N, K):
    """Whatever the default decides (strips or not), the whole of C is right: compared on the device."""
    assert clblas_amd.setup() == 0
    alpha, beta = 1.0, 1.0
    A, B, C, want, lda, ldb, ldc = _case(t, COL, NOTRANS, NOTRANS, M, N, K, 4242, 0, (0, 0, 0), alpha, beta)
    dA, dB, dC = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), torch.from_numpy(C).cuda()
    st = FN[t](COL, NOTRANS, NOTRANS, M, N, K, alpha, dA, 0, lda, dB, 0, ldb, beta, dC, 0, ldc)
    torch.cuda.synchronize()
    assert st == 0
    assert torch.equal(dC, torch.from_numpy(want).cuda()), clblas_amd.last_dispatch()[0]


def test_no_alloc_entry_point_makes_the_same_pieces():
    """clblasSgemmNoAlloc goes through the same launcher: same pieces, same bits as clblasSgemm."""
    assert clblas_amd.setup() == 0
    M, N, K = 1030, 2049, 300
    A, B, C, want, lda, ldb, ldc = _case("s", COL, NOTRANS, TRANS, M, N, K, 77, 0, (0, 0, 0), 2.0, -3.0)
    dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    with gpu_util.debug_env(CLBLAS_AMD_GEMM_PEEL=2):
        outs = []
        for fn in (clblas_amd.sgemm, clblas_amd.sgemm_noalloc):
            dC = torch.from_numpy(C).cuda()
            assert fn(COL, NOTRANS, TRANS, M, N, K, 2.0, dA, 0, lda, dB, 0, ldb, -3.0, dC, 0, ldc) == 0
            torch.cuda.synchronize()
            outs.append(dC.cpu().numpy())
    np.testing.assert_array_equal(outs[0], want)
    np.testing.assert_array_equal(outs[1], want)
