"""CLBLAS_AMD_CHECK_MEM=1 on a real device: the library looks up the allocation behind every operand
(hipMemGetAddressRange) and applies the reference's rule for clblasInsufficientMemMat{A,B,C}
(src/library/blas/generic/common.c:644-684; expected by src/tests/functional/func-error.cpp:58-104, which
passes matrices larger than their buffers).  torch's allocator hands out pieces of larger blocks, so the
matrices that must be refused are made far larger than any block a 4 KiB tensor can sit in."""
import numpy as np
import pytest
import torch

import clblas_amd
from gpu_util import debug_env
from helpers import COL, ROW, NOTRANS, TRANS, LEFT, LOWER, NONUNIT

pytestmark = pytest.mark.gpu

S = clblas_amd.Status


def test_operands_that_do_not_fit_their_allocations_are_refused():
    assert clblas_amd.setup() == 0
    small = torch.zeros(1024, device="cuda", dtype=torch.float32)
    n = 4096                                                   # 64 MiB per matrix
    big = [torch.zeros(n * n, device="cuda", dtype=torch.float32) for _ in range(3)]
    keep = big[2].clone()
    with debug_env(CLBLAS_AMD_CHECK_MEM=1):
        for order in (COL, ROW):
            for tA in (NOTRANS, TRANS):
                args = lambda A, B, C: (order, tA, NOTRANS, n, n, n, 1.0, A, 0, n, B, 0, n, 0.0, C, 0, n)
                assert clblas_amd.sgemm(*args(small, big[1], big[2])) == S.InsufficientMemMatA
                assert clblas_amd.sgemm(*args(big[0], small, big[2])) == S.InsufficientMemMatB
                assert clblas_amd.sgemm(*args(big[0], big[1], small)) == S.InsufficientMemMatC
        # an offset that pushes the last column out of an otherwise sufficient buffer
        assert clblas_amd.sgemm(COL, NOTRANS, NOTRANS, n, n, n, 1.0, big[0], 0, n, big[1], 0, n, 0.0, big[2], 1 << 26, n) \
            == S.InsufficientMemMatC
        assert clblas_amd.strsm(COL, LEFT, LOWER, NOTRANS, NONUNIT, n, n, 1.0, small, 0, n, big[1], 0, n) == S.InsufficientMemMatA
        assert clblas_amd.strsm(COL, LEFT, LOWER, NOTRANS, NONUNIT, n, n, 1.0, big[0], 0, n, small, 0, n) == S.InsufficientMemMatB
        # an address that no device allocation holds is no matrix (the reference: clGetMemObjectInfo fails)
        assert clblas_amd.sgemm(COL, NOTRANS, NOTRANS, 8, 8, 8, 1.0, 0x1000, 0, 8, small, 0, 8, 0.0, small, 256, 8) == S.InvalidMatA
        torch.cuda.synchronize()
        assert torch.equal(big[2], keep), "a refused call must not have run"
        # what fits runs as usual
        a = torch.from_numpy(np.arange(64, dtype=np.float32)).cuda()
        c = torch.zeros(64, device="cuda", dtype=torch.float32)
        eye = torch.eye(8, device="cuda", dtype=torch.float32).reshape(-1).contiguous()
        assert clblas_amd.sgemm(COL, NOTRANS, NOTRANS, 8, 8, 8, 1.0, a, 0, 8, eye, 0, 8, 0.0, c, 0, 8) == 0
        torch.cuda.synchronize()
        assert torch.equal(a, c)
    # without the switch nothing is looked up: the same oversize call is the caller's business, and is not made here
