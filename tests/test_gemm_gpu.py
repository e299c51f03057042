"""GPU parity tests for clblasSgemm / clblasDgemm through the C ABI, against the CPU oracle.

Bars: exact equality on the reference tests' exact-integer inputs (any summation order gives
the same bits there); for real-valued inputs
    |C - C_exact| <= 2 (K+2) u (|alpha| |A||B| + |beta||C|),   u = unit roundoff,
i.e. the task's c*K*eps bound with c = 2, which both our result and the reference's
one-accumulator result satisfy."""
import itertools

import numpy as np
import pytest

import oracle
from helpers import (COL, ROW, NOTRANS, TRANS, CONJ, LEFT, LOWER, NONUNIT, buf_len, exact_int_limits, gemm_bound, golden_cases,
                     logical_view, mem_dims)

pytestmark = pytest.mark.gpu

DT = {"f32": np.float32, "f64": np.float64}
N_TILES = {np.float32: 7, np.float64: 4}


@pytest.fixture(scope="module")
def gpu():
    import gpu_util
    import torch
    assert torch.cuda.is_available()
    import clblas_amd
    assert clblas_amd.setup() == 0
    return gpu_util


@pytest.mark.parametrize("name", ["readme_sgemm", "sample_sgemm_offsets"])
def test_golden(gpu, name):
    c = golden_cases()[name]
    dt = DT[c["dtype"]]
    A, B, C = (np.array(c[k], dtype=dt) for k in "ABC")
    st, out = gpu.gemm(c["order"], c["transA"], c["transB"], c["M"], c["N"], c["K"], c["alpha"], A, c["offA"],
                       c["lda"], B, c["offB"], c["ldb"], c["beta"], C, c["offC"], c["ldc"])
    assert st == 0
    np.testing.assert_array_equal(out, np.array(c["expected"], dtype=dt))


def _layout(order, tA, tB, M, N, K, pad, offs):
    ia, oa = mem_dims(order, tA, M, K)
    ib, ob = mem_dims(order, tB, K, N)
    ic, oc = mem_dims(order, NOTRANS, M, N)
    lda, ldb, ldc = ia + pad, ib + pad, ic + pad
    offA, offB, offC = offs
    return (lda, ldb, ldc, offA + oa * lda, offB + ob * ldb, offC + oc * ldc)


INT_SHAPES = [(1, 1, 1), (2, 1, 3), (8, 16, 17), (17, 32, 62), (64, 64, 64), (62, 144, 128), (256, 128, 16),
              (257, 129, 33), (300, 520, 200), (130, 70, 1031)]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("order", [ROW, COL])
@pytest.mark.parametrize("tA,tB", list(itertools.product([NOTRANS, TRANS], [NOTRANS, TRANS, CONJ])))
def test_integer_exact_all_tiles(gpu, dtype, order, tA, tB):
    """The reference's own correctness method (corr-gemm.cpp:192, matrix.h:322-327): integer
    data small enough that the result is exact, compared with assert-equal.  Every tile of
    the table is forced in turn, plus the default choice."""
    for si, (M, N, K) in enumerate(INT_SHAPES):
        alpha, beta = 3.0, -2.0
        la, lc = exact_int_limits(K, alpha, beta, dtype)
        offs = (5, 7, 11)
        lda, ldb, ldc, na, nb, nc = _layout(order, tA, tB, M, N, K, 3, offs)
        A = oracle.integers(na, 100 + si, la, dtype)
        B = oracle.integers(nb, 200 + si, la, dtype)
        C = oracle.integers(nc, 300 + si, lc, dtype)
        want = C.copy()
        assert oracle.gemm(order, tA, tB, M, N, K, alpha, A, offs[0], lda, B, offs[1], ldb, beta, want, offs[2],
                           ldc) == 0
        for tile in [None] + list(range(N_TILES[dtype])):
            st, got = gpu.gemm(order, tA, tB, M, N, K, alpha, A, offs[0], lda, B, offs[1], ldb, beta, C, offs[2], ldc,
                               tile=tile)
            assert st == 0
            np.testing.assert_array_equal(got, want, err_msg="shape %s tile %s" % ((M, N, K), tile))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("tA,tB", list(itertools.product([NOTRANS, TRANS], [NOTRANS, TRANS])))
def test_integer_exact_deep_panel_variant(gpu, dtype, tA, tB):
    """The smallest tile has a second form with panels twice as deep, used where a workgroup's K
    range is long.  Here it is switched on for every depth (CLBLAS_AMD_GEMM_DEEP=2), with and without a
    K split, on depths that are and are not multiples of the panel depth."""
    import clblas_amd
    small = N_TILES[dtype] - 1
    shapes = INT_SHAPES + [(200, 150, 1100), (100, 90, 4096), (250, 130, 2050)]
    for si, (M, N, K) in enumerate(shapes):
        alpha, beta = 3.0, -2.0
        la, lc = exact_int_limits(K, alpha, beta, dtype)
        offs = (5, 7, 11)
        lda, ldb, ldc, na, nb, nc = _layout(COL, tA, tB, M, N, K, 3, offs)
        A = oracle.integers(na, 400 + si, la, dtype)
        B = oracle.integers(nb, 500 + si, la, dtype)
        C = oracle.integers(nc, 600 + si, lc, dtype)
        want = C.copy()
        assert oracle.gemm(COL, tA, tB, M, N, K, alpha, A, offs[0], lda, B, offs[1], ldb, beta, want, offs[2], ldc) == 0
        with gpu.debug_env(CLBLAS_AMD_GEMM_DEEP=2, CLBLAS_AMD_GEMM_TILE=small):
            st, got = gpu.gemm(COL, tA, tB, M, N, K, alpha, A, offs[0], lda, B, offs[1], ldb, beta, C, offs[2], ldc)
            what = clblas_amd.last_dispatch()[0]
        assert st == 0
        deep = "64x64x64" if dtype == np.float32 else "64x64x32"
        assert deep in what or "splits=1 " not in what, what   # a K split whose ranges are not multiples of the depth keeps the plain form
        np.testing.assert_array_equal(got, want, err_msg="shape %s: %s" % ((M, N, K), what))


def _check_sampled(dtype, tA, tB, M, N, K, alpha, beta, A, lda, B, ldb, C0, got, ldc, nsamp=3000, seed=0):
    """Column-major buffers starting at element (0,0).  Checks sampled elements (all four
    borders plus random interior points) against the high-precision oracle."""
    rng = np.random.default_rng(seed)
    rows = [rng.integers(0, M, nsamp), np.full(200, M - 1), np.zeros(200, dtype=np.int64), rng.integers(0, M, 400)]
    cols = [rng.integers(0, N, nsamp), rng.integers(0, N, 200), rng.integers(0, N, 200),
            np.concatenate([np.full(200, N - 1), np.zeros(200, dtype=np.int64)])]
    rows, cols = np.concatenate(rows), np.concatenate(cols)
    exact, mag = oracle.gemm_exact(tA, tB, K, alpha, A, lda, B, ldb, beta, C0, ldc, rows, cols)
    vals = got[rows + cols * ldc].astype(np.float64)
    err = np.abs(vals - exact)
    bound = gemm_bound(K, mag, dtype)
    worst = np.argmax(err / bound)
    assert np.all(err <= bound), "element (%d,%d): err %.3e bound %.3e" % (rows[worst], cols[worst], err[worst],
                                                                          bound[worst])
    return float((err / bound).max())


def test_config1_sgemm_1024_full_matrix(gpu):
    """BASELINE config 1: SGEMM NN 1024^3, alpha=1, beta=0, uniform[-1,1): every element,
    against the oracle's result and the exact product."""
    n = 1024
    A, B, C = oracle.uniform(n * n, 1, np.float32), oracle.uniform(n * n, 2, np.float32), oracle.uniform(n * n, 3, np.float32)
    want = C.copy()
    assert oracle.gemm(COL, NOTRANS, NOTRANS, n, n, n, 1.0, A, 0, n, B, 0, n, 0.0, want, 0, n) == 0
    st, got = gpu.gemm(COL, NOTRANS, NOTRANS, n, n, n, 1.0, A, 0, n, B, 0, n, 0.0, C, 0, n)
    assert st == 0
    A64, B64 = A.reshape(n, n).T.astype(np.float64), B.reshape(n, n).T.astype(np.float64)
    exact = A64 @ B64
    mag = np.abs(A64) @ np.abs(B64)
    bound = gemm_bound(n, mag, np.float32)
    assert np.all(np.abs(got.reshape(n, n).T - exact) <= bound)
    assert np.all(np.abs(want.reshape(n, n).T - exact) <= bound)      # the oracle sits inside the same bound
    assert np.all(np.abs(got.astype(np.float64) - want) <= 2 * bound.T.ravel())


def test_beta_zero_never_reads_c_and_alpha_zero(gpu):
    for dtype in (np.float32, np.float64):
        M, N, K = 70, 90, 50
        A, B = oracle.uniform(M * K, 1, dtype), oracle.uniform(K * N, 2, dtype)
        C = np.full(M * N, np.nan, dtype=dtype)
        want = C.copy()
        oracle.gemm(COL, NOTRANS, NOTRANS, M, N, K, 1.0, A, 0, M, B, 0, K, 0.0, want, 0, M)
        st, got = gpu.gemm(COL, NOTRANS, NOTRANS, M, N, K, 1.0, A, 0, M, B, 0, K, 0.0, C, 0, M)
        assert st == 0 and np.isfinite(got).all()
        np.testing.assert_allclose(got, want, rtol=0, atol=4 * K * np.finfo(dtype).eps)
        C1 = oracle.uniform(M * N, 3, dtype)
        st, got = gpu.gemm(COL, NOTRANS, NOTRANS, M, N, K, 0.0, A, 0, M, B, 0, K, 1.0, C1, 0, M)
        assert st == 0
        np.testing.assert_array_equal(got, C1)
        # K == 0: C <- beta * C (documented deviation from a reference bug); beta == 0 clears NaNs
        st, got = gpu.gemm(COL, NOTRANS, NOTRANS, M, N, 0, 1.0, A, 0, M, B, 0, 1, 0.5, C1, 0, M)
        assert st == 0
        np.testing.assert_array_equal(got, (0.5 * C1).astype(dtype))
        st, got = gpu.gemm(COL, NOTRANS, NOTRANS, M, N, 0, 1.0, A, 0, M, B, 0, 1, 0.0, C, 0, M)
        assert st == 0 and (got == 0).all()


EDGE_SHAPES = [(4097, 4095, 1031), (65536, 64, 4096), (64, 65536, 4096), (127, 129, 8192)]


@pytest.mark.parametrize("M,N,K", EDGE_SHAPES)
def test_config3_sgemm_edge_sweep(gpu, M, N, K):
    """BASELINE config 3: alpha=0.7, beta=-1.3, all four transposes, ld = rows+3, offsets
    5/7/11, uniform[-1,1).  Sampled elements (borders included) against the exact product;
    everything outside the M x N window of C must be bit-identical to the input."""
    dtype = np.float32
    alpha, beta = 0.7, -1.3
    offs = (5, 7, 11)
    for tA, tB in itertools.product([NOTRANS, TRANS], [NOTRANS, TRANS]):
        lda, ldb, ldc, na, nb, nc = _layout(COL, tA, tB, M, N, K, 3, offs)
        A, B, C = oracle.uniform(na, 1, dtype), oracle.uniform(nb, 2, dtype), oracle.uniform(nc, 3, dtype)
        st, got = gpu.gemm(COL, tA, tB, M, N, K, alpha, A, offs[0], lda, B, offs[1], ldb, beta, C, offs[2], ldc)
        assert st == 0
        _check_sampled(dtype, tA != NOTRANS, tB != NOTRANS, M, N, K, alpha, beta, A[offs[0]:], lda, B[offs[1]:], ldb,
                       C[offs[2]:], got[offs[2]:], ldc)
        mask = np.zeros(nc, dtype=bool)
        logical_view(mask, COL, NOTRANS, M, N, offs[2], ldc)[:] = True
        np.testing.assert_array_equal(got[~mask], C[~mask])
        assert not np.array_equal(got[mask], C[mask])


VECTOR_LIKE_SHAPES = [(8192, 1, 2048), (1, 8192, 2048), (5000, 3, 7), (3, 2000, 20000), (1, 1, 100000),
                      (70000, 2, 1), (33, 70000, 5), (4099, 61, 4099)]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("M,N,K", VECTOR_LIKE_SHAPES)
def test_vector_like_and_degenerate_shapes(gpu, dtype, M, N, K):
    """Matrix-vector, outer-product and dot-product shaped calls (one dimension of 1..3, another in
    the tens of thousands), all four transposes, padded leading dimensions and offsets: sampled
    elements against the exact product, surroundings of C untouched."""
    alpha, beta = 0.75, -0.5
    offs = (3, 9, 1)
    for tA, tB in itertools.product([NOTRANS, TRANS], [NOTRANS, TRANS]):
        lda, ldb, ldc, na, nb, nc = _layout(COL, tA, tB, M, N, K, 5, offs)
        A, B, C = oracle.uniform(na, 4, dtype), oracle.uniform(nb, 5, dtype), oracle.uniform(nc, 6, dtype)
        st, got = gpu.gemm(COL, tA, tB, M, N, K, alpha, A, offs[0], lda, B, offs[1], ldb, beta, C, offs[2], ldc)
        assert st == 0
        _check_sampled(dtype, tA != NOTRANS, tB != NOTRANS, M, N, K, alpha, beta, A[offs[0]:], lda, B[offs[1]:], ldb,
                       C[offs[2]:], got[offs[2]:], ldc, nsamp=500)
        mask = np.zeros(nc, dtype=bool)
        logical_view(mask, COL, NOTRANS, M, N, offs[2], ldc)[:] = True
        np.testing.assert_array_equal(got[~mask], C[~mask])


def _freivalds(torch, dA, dB, dC0, dC, tA, tB, n, alpha, beta):
    """C v == alpha opA (opB v) + beta C0 v in fp64 on the device; returns the relative defect."""
    v = torch.randn(n, dtype=torch.float64, device="cuda")
    A = dA.view(n, n).T.double() if not tA else dA.view(n, n).double()
    Bv = (dB.view(n, n).T.double() if not tB else dB.view(n, n).double()) @ v
    rhs = alpha * (A @ Bv) + beta * (dC0.view(n, n).T.double() @ v)
    lhs = dC.view(n, n).T.double() @ v
    return float((lhs - rhs).abs().max() / rhs.abs().max())


@pytest.mark.parametrize("cfg", ["config2_sgemm", "config4_dgemm"])
def test_full_size_8192(gpu, cfg):
    """BASELINE configs 2 and 4 at full size: sampled elements against the exact product, and
    a size-independent linearity check C v = alpha A (B v) + beta C0 v."""
    import torch
    import clblas_amd
    n = 8192
    if cfg == "config2_sgemm":
        dtype, tA, tB, alpha, beta = np.float32, NOTRANS, NOTRANS, 1.0, 1.0
        A, B, C = (oracle.uniform(n * n, s, dtype) for s in (1, 2, 3))
        fn = clblas_amd.sgemm
    else:
        dtype, tA, tB, alpha, beta = np.float64, NOTRANS, TRANS, 1.0, 0.5
        A, B, C = (oracle.normal(n * n, s, dtype) for s in (1, 2, 3))
        fn = clblas_amd.dgemm
    dA, dB, dC0 = (torch.from_numpy(x).cuda() for x in (A, B, C))
    dC = dC0.clone()
    st = fn(COL, tA, tB, n, n, n, alpha, dA, 0, n, dB, 0, n, beta, dC, 0, n)
    torch.cuda.synchronize()
    assert st == 0
    got = dC.cpu().numpy()
    _check_sampled(dtype, tA != NOTRANS, tB != NOTRANS, n, n, n, alpha, beta, A, n, B, n, C, got, n, nsamp=6000)
    defect = _freivalds(torch, dA, dB, dC0, dC, tA != NOTRANS, tB != NOTRANS, n, alpha, beta)
    assert defect <= 64 * n * np.finfo(dtype).eps, defect


def test_wide_leading_dimension_path(gpu):
    """Leading dimensions beyond the 32-bit panel offsets take the plain 64-bit kernel."""
    M, N, K = 4, 3, 5
    lda = 3 * 1024 * 1024
    A = oracle.integers(K * lda, 1, 10, np.float32)
    B = oracle.integers(K * N, 2, 10, np.float32)
    C = oracle.integers(M * N, 3, 10, np.float32)
    want = C.copy()
    oracle.gemm(COL, NOTRANS, NOTRANS, M, N, K, 2.0, A, 0, lda, B, 0, K, 3.0, want, 0, M)
    st, got = gpu.gemm(COL, NOTRANS, NOTRANS, M, N, K, 2.0, A, 0, lda, B, 0, K, 3.0, C, 0, M)
    assert st == 0
    np.testing.assert_array_equal(got, want)


def test_padding_of_inputs_is_never_used(gpu):
    """Everything outside the logical windows of A and B (leading-dimension padding, offsets,
    tails) is NaN: tile remainders in M, N and K must neither fault nor leak into C."""
    for dtype in (np.float32, np.float64):
        for (M, N, K) in [(70, 45, 37), (257, 130, 19), (33, 300, 130)]:
            for order, tA, tB in itertools.product([ROW, COL], [NOTRANS, TRANS], [NOTRANS, TRANS]):
                offs = (9, 3, 6)
                lda, ldb, ldc, na, nb, nc = _layout(order, tA, tB, M, N, K, 5, offs)
                A = np.full(na + 7, np.nan, dtype=dtype)
                B = np.full(nb + 7, np.nan, dtype=dtype)
                logical_view(A, order, tA, M, K, offs[0], lda)[:] = oracle.integers(M * K, 1, 9, dtype).reshape(M, K)
                logical_view(B, order, tB, K, N, offs[1], ldb)[:] = oracle.integers(K * N, 2, 9, dtype).reshape(K, N)
                C = oracle.integers(nc, 3, 9, dtype)
                want = C.copy()
                assert oracle.gemm(order, tA, tB, M, N, K, 2.0, A, offs[0], lda, B, offs[1], ldb, 1.0, want, offs[2],
                                   ldc) == 0
                st, got = gpu.gemm(order, tA, tB, M, N, K, 2.0, A, offs[0], lda, B, offs[1], ldb, 1.0, C, offs[2], ldc)
                assert st == 0
                np.testing.assert_array_equal(got, want, err_msg=str((dtype, M, N, K, order, tA, tB)))


def test_two_streams_and_teardown(gpu):
    """Calls on different streams are independent (each has its own split-K scratch), and the
    library keeps working after clblasTeardown released that scratch."""
    import torch
    import clblas_amd
    M, N, K = 100, 90, 4096            # few tiles, deep K: takes the split-K path
    la, lc = exact_int_limits(K, 1.0, 1.0, np.float32)
    A1, B1, C1 = (oracle.integers(n, s, la, np.float32) for n, s in ((M * K, 1), (K * N, 2), (M * N, 3)))
    A2, B2, C2 = (oracle.integers(n, s, la, np.float32) for n, s in ((M * K, 4), (K * N, 5), (M * N, 6)))
    w1, w2 = C1.copy(), C2.copy()
    oracle.gemm(COL, NOTRANS, NOTRANS, M, N, K, 1.0, A1, 0, M, B1, 0, K, 1.0, w1, 0, M)
    oracle.gemm(COL, NOTRANS, NOTRANS, M, N, K, 1.0, A2, 0, M, B2, 0, K, 1.0, w2, 0, M)
    for rep in range(2):
        d = [torch.from_numpy(x).cuda() for x in (A1, B1, C1, A2, B2, C2)]
        s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
        torch.cuda.synchronize()
        for _ in range(1):
            assert clblas_amd.sgemm(COL, NOTRANS, NOTRANS, M, N, K, 1.0, d[0], 0, M, d[1], 0, K, 1.0, d[2], 0, M,
                                    stream=s1) == 0
            assert clblas_amd.sgemm(COL, NOTRANS, NOTRANS, M, N, K, 1.0, d[3], 0, M, d[4], 0, K, 1.0, d[5], 0, M,
                                    stream=s2) == 0
        torch.cuda.synchronize()
        np.testing.assert_array_equal(d[2].cpu().numpy(), w1)
        np.testing.assert_array_equal(d[5].cpu().numpy(), w2)
        clblas_amd.teardown()          # second pass runs after the scratch was released
    assert clblas_amd.setup() == 0


def test_host_threads_on_their_own_streams(gpu):
    """Four host threads call the library at the same time, each on its own stream (ctypes
    releases the interpreter lock during a call): split-K SGEMM, whose scratch buffer is looked up
    per stream under the library's lock, and DTRSM with its packing buffer.  Exact-integer GEMM
    data, so every result must equal the oracle's."""
    import threading
    import torch
    import clblas_amd
    M, N, K = 100, 90, 4096
    la, _ = exact_int_limits(K, 1.0, 1.0, np.float32)
    n = 300
    jobs = []
    for t in range(4):
        A, B, C = (oracle.integers(sz, 10 * t + i, la, np.float32) for i, sz in enumerate((M * K, K * N, M * N)))
        want = C.copy()
        oracle.gemm(COL, NOTRANS, NOTRANS, M, N, K, 1.0, A, 0, M, B, 0, K, 1.0, want, 0, M)
        T = oracle.triangular(n, n, True, 50 + t, np.float64)
        X = oracle.uniform(n * 64, 60 + t, np.float64)
        wx = X.copy()
        assert oracle.trsm_naive(COL, LEFT, LOWER, NOTRANS, NONUNIT, n, 64, 1.0, T, 0, n, wx, 0, n) == 0
        jobs.append(dict(d=[torch.from_numpy(x).cuda() for x in (A, B, C, T, X)], C0=C, X0=X, want=want, wx=wx,
                         stream=torch.cuda.Stream(), err=None))
    torch.cuda.synchronize()

    def work(j):
        try:
            dA, dB, dC, dT, dX = j["d"]
            for _ in range(20):
                dC.copy_(torch.from_numpy(j["C0"]), non_blocking=False)
                dX.copy_(torch.from_numpy(j["X0"]), non_blocking=False)
                with torch.cuda.stream(j["stream"]):
                    st1 = clblas_amd.sgemm(COL, NOTRANS, NOTRANS, M, N, K, 1.0, dA, 0, M, dB, 0, K, 1.0, dC, 0, M)
                    st2 = clblas_amd.dtrsm(COL, LEFT, LOWER, NOTRANS, NONUNIT, n, 64, 1.0, dT, 0, n, dX, 0, n)
                j["stream"].synchronize()
                assert st1 == 0 and st2 == 0
                np.testing.assert_array_equal(dC.cpu().numpy(), j["want"])
                got = dX.cpu().numpy()
                assert np.abs(got - j["wx"]).max() <= 32 * n * np.finfo(np.float64).eps * np.abs(j["wx"]).max()
        except BaseException as e:  # reported by the main thread
            j["err"] = e

    threads = [threading.Thread(target=work, args=(j,)) for j in jobs]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    for j in jobs:
        if j["err"] is not None:
            raise j["err"]


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.complex64, np.complex128])
def test_sliced_tail_integer_exact(gpu, dtype):
    """More than 256 tiles with a partly filled last round: the tiles of that round are cut into
    K slices and finished by a reduction pass.  Exact-integer data, smallest tile forced so that
    a modest problem has 18 x 16 = 288 tiles (32 in the last round, K = 520 in 2 to 8 slices,
    by the panel depth of the type's smallest tile)."""
    M, N, K = 1100, 1000, 520
    cplx = np.dtype(dtype).kind == "c"
    alpha, beta = ((2 - 1j), (-1 + 2j)) if cplx else (3.0, -2.0)
    small_tile = {np.float32: 4, np.float64: 1, np.complex64: 1, np.complex128: 1}[dtype]
    for tA, tB in ((NOTRANS, NOTRANS), (TRANS, CONJ)):
        lda, ldb, ldc, na, nb, nc = _layout(COL, tA, tB, M, N, K, 1, (3, 5, 7))
        lim = 8 if cplx else exact_int_limits(K, alpha, beta, dtype)[0]
        A = oracle.integers(na, 1, lim, dtype)
        B = oracle.integers(nb, 2, lim, dtype)
        C = oracle.integers(nc, 3, 8, dtype)
        want = C.copy()
        assert oracle.gemm(COL, tA, tB, M, N, K, alpha, A, 3, lda, B, 5, ldb, beta, want, 7, ldc) == 0
        st, got = gpu.gemm(COL, tA, tB, M, N, K, alpha, A, 3, lda, B, 5, ldb, beta, C, 7, ldc, tile=small_tile)
        assert st == 0
        np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.complex64, np.complex128])
def test_many_workgroups_not_whole_rounds_integer_exact(gpu, dtype):
    """More than 512 workgroups in a launch that is not a whole number of rounds: the launch in
    which every other workgroup of the first round starts late, with and without a sliced tail.
    Exact-integer data, smallest tile forced: 31 x 29 = 899 tiles (no slicing: the last round is
    too full), 30 x 18 = 540 tiles (28 in the last round, sliced)."""
    cplx = np.dtype(dtype).kind == "c"
    alpha, beta = ((2 - 1j), (-1 + 2j)) if cplx else (3.0, -2.0)
    small_tile = {np.float32: 4, np.float64: 1, np.complex64: 1, np.complex128: 1}[dtype]
    for (M, N, K), (tA, tB) in (((1950, 1830, 150), (NOTRANS, TRANS)), ((1900, 1150, 600), (TRANS, NOTRANS))):
        lda, ldb, ldc, na, nb, nc = _layout(COL, tA, tB, M, N, K, 1, (3, 5, 7))
        lim = 8 if cplx else exact_int_limits(K, alpha, beta, dtype)[0]
        A = oracle.integers(na, 1, lim, dtype)
        B = oracle.integers(nb, 2, lim, dtype)
        C = oracle.integers(nc, 3, 8, dtype)
        want = C.copy()
        assert oracle.gemm(COL, tA, tB, M, N, K, alpha, A, 3, lda, B, 5, ldb, beta, want, 7, ldc) == 0
        for tile in (small_tile, None):
            st, got = gpu.gemm(COL, tA, tB, M, N, K, alpha, A, 3, lda, B, 5, ldb, beta, C, 7, ldc, tile=tile)
            assert st == 0
            np.testing.assert_array_equal(got, want, err_msg="%dx%dx%d tile %s" % (M, N, K, tile))


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.complex64, np.complex128])
def test_small_c_deep_k_integer_exact(gpu, dtype):
    """Small C, deep K: too few tiles for the 256 CUs, so the tile choice cuts K into ranges for one of
    the larger tiles (partial sums in the workspace, added up by a second pass).  Exact-integer data,
    default tile choice and every tile forced; odd offsets and leading dimensions."""
    cplx = np.dtype(dtype).kind == "c"
    alpha, beta = ((2 - 1j), (-1 + 2j)) if cplx else (3.0, -2.0)
    n_tiles = {np.float32: 7, np.float64: 4, np.complex64: 4, np.complex128: 4}[dtype]
    for (M, N, K), (tA, tB) in (((640, 520, 6000), (NOTRANS, NOTRANS)), ((300, 900, 5000), (TRANS, CONJ))):
        lda, ldb, ldc, na, nb, nc = _layout(COL, tA, tB, M, N, K, 1, (3, 5, 7))
        lim = 8 if cplx else exact_int_limits(K, alpha, beta, dtype)[0]
        A = oracle.integers(na, 1, lim, dtype)
        B = oracle.integers(nb, 2, lim, dtype)
        C = oracle.integers(nc, 3, 8, dtype)
        want = C.copy()
        assert oracle.gemm(COL, tA, tB, M, N, K, alpha, A, 3, lda, B, 5, ldb, beta, want, 7, ldc) == 0
        for tile in [None] + list(range(n_tiles)):
            st, got = gpu.gemm(COL, tA, tB, M, N, K, alpha, A, 3, lda, B, 5, ldb, beta, C, 7, ldc, tile=tile)
            assert st == 0
            np.testing.assert_array_equal(got, want, err_msg="%dx%dx%d tile %s" % (M, N, K, tile))
