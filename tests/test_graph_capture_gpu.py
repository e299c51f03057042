"""The entry points under HIP graph capture.

Once a stream's scratch buffers exist (one eager call of the same shapes on that stream), a call
only enqueues kernels: no allocation, no synchronisation, no memset.  A sequence of calls that
covers every kind of launch the library makes (plain tiles, a K split with its reduction pass, a
sliced tail with its reduction pass, TRSM's packing pass, leaves and update GEMMs, TRMM's copy
of B, SYRK's triangle) is captured once and replayed several times, with eager work and
synchronisations in between; every replay must reproduce the eager results bit for bit.
"""
import numpy as np
import pytest

import oracle
from helpers import COL, NOTRANS, TRANS, LEFT, LOWER, NONUNIT

pytestmark = pytest.mark.gpu


def test_calls_replay_from_a_hip_graph():
    import torch
    import clblas_amd
    assert torch.cuda.is_available()
    assert clblas_amd.setup() == 0

    def dev(x):
        return torch.from_numpy(x).cuda()

    f32, f64 = np.float32, np.float64
    # SGEMM 100 x 90 x 4096: few tiles, deep K -> split-K + reduction
    a1, b1, c1 = dev(oracle.uniform(100 * 4096, 1, f32)), dev(oracle.uniform(4096 * 90, 2, f32)), dev(oracle.uniform(100 * 90, 3, f32))
    # DGEMM 1100 x 1000 x 520 (NT): more than 256 tiles with a partly filled last round -> sliced tail
    a2, b2, c2 = dev(oracle.uniform(1100 * 520, 4, f64)), dev(oracle.uniform(1000 * 520, 5, f64)), dev(oracle.uniform(1100 * 1000, 6, f64))
    # DTRSM 600 x 300: packing pass, three leaves, two update GEMMs
    n = 600
    t = oracle.triangular(n, n, True, 7, f64)
    ta, tb = dev(t), dev(oracle.uniform(n * 300, 8, f64))
    # STRMM 300 x 200 and SSYRK 300 x 64
    ma, mb = dev(oracle.uniform(300 * 300, 9, f32)), dev(oracle.uniform(300 * 200, 10, f32))
    sa, sc = dev(oracle.uniform(300 * 64, 11, f32)), dev(oracle.uniform(300 * 300, 12, f32))
    # SSYRK 200 x 8192: a small C with a deep K runs as a K-split GEMM into a library buffer + a triangle pass
    da, dc = dev(oracle.uniform(200 * 8192, 13, f32)), dev(oracle.uniform(200 * 200, 14, f32))
    ins = [c1, c2, tb, mb, sc, dc]
    keep = [x.clone() for x in ins]

    def sequence():
        for x, k in zip(ins, keep):
            x.copy_(k)
        sts = [clblas_amd.sgemm(COL, NOTRANS, NOTRANS, 100, 90, 4096, 0.5, a1, 0, 100, b1, 0, 4096, -1.5, c1, 0, 100),
               clblas_amd.dgemm(COL, NOTRANS, TRANS, 1100, 1000, 520, 0.75, a2, 0, 1100, b2, 0, 1000, 0.5, c2, 0, 1100),
               clblas_amd.dtrsm(COL, LEFT, LOWER, NOTRANS, NONUNIT, n, 300, 2.0, ta, 0, n, tb, 0, n),
               clblas_amd.trmm("S", COL, LEFT, LOWER, NOTRANS, NONUNIT, 300, 200, 1.5, ma, 0, 300, mb, 0, 300),
               clblas_amd.syrk("S", COL, LOWER, NOTRANS, 300, 64, 1.0, sa, 0, 300, 0.5, sc, 0, 300),
               clblas_amd.syrk("S", COL, LOWER, NOTRANS, 200, 8192, 0.25, da, 0, 200, 0.5, dc, 0, 200)]
        assert sts == [0] * 6, sts

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        sequence()          # allocates this stream's scratch buffers
        sequence()
    stream.synchronize()
    eager = [x.clone() for x in ins]
    assert all(bool(torch.isfinite(x).all()) for x in eager)

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        sequence()
    for rep in range(4):
        for x in ins:
            x.fill_(float("nan"))
        # eager work of the library on another stream between the replays
        assert clblas_amd.sgemm(COL, NOTRANS, NOTRANS, 100, 90, 4096, 1.0, a1, 0, 100, b1, 0, 4096, 0.0,
                                torch.empty(100 * 90, device="cuda", dtype=torch.float32), 0, 100) == 0
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for i, (x, e) in enumerate(zip(ins, eager)):
            assert torch.equal(x, e), "replay %d, output %d differs from the eager result" % (rep, i)


def test_capture_needs_buffers_that_exist_and_reserve_provides_them():
    """A call that would have to allocate its scratch buffer while the stream is being captured
    returns clblasInvalidOperation, enqueues nothing and leaves the capture usable;
    clblasAmdReserveWorkspace makes the same calls capturable as the very first use of a stream;
    clblasAmdReleaseStream gives the buffers back."""
    import torch
    import clblas_amd
    assert clblas_amd.setup() == 0
    INVALID_OPERATION = -59
    f32, f64 = np.float32, np.float64

    def dev(x):
        return torch.from_numpy(x).cuda()

    a1, b1 = dev(oracle.uniform(100 * 4096, 1, f32)), dev(oracle.uniform(4096 * 90, 2, f32))
    c1 = dev(oracle.uniform(100 * 90, 3, f32))          # split-K: needs a workspace
    a0, b0 = dev(oracle.uniform(512 * 64, 4, f32)), dev(oracle.uniform(64 * 512, 5, f32))
    c0 = torch.zeros(512 * 512, device="cuda", dtype=torch.float32)   # one plain launch: needs none
    n = 600
    ta, tb = dev(oracle.triangular(n, n, True, 7, f64)), dev(oracle.uniform(n * 300, 8, f64))
    c1_keep, tb_keep = c1.clone(), tb.clone()

    def split_k():
        return clblas_amd.sgemm(COL, NOTRANS, NOTRANS, 100, 90, 4096, 0.5, a1, 0, 100, b1, 0, 4096, -1.5, c1, 0, 100)

    def plain():
        return clblas_amd.sgemm(COL, NOTRANS, NOTRANS, 512, 512, 64, 1.0, a0, 0, 512, b0, 0, 64, 0.0, c0, 0, 512)

    def trsm():
        return clblas_amd.dtrsm(COL, LEFT, LOWER, NOTRANS, NONUNIT, n, 300, 2.0, ta, 0, n, tb, 0, n)

    # eager results on the default stream
    assert split_k() == 0 and plain() == 0 and trsm() == 0
    torch.cuda.synchronize()
    want_c1, want_c0, want_tb = c1.clone(), c0.clone(), tb.clone()

    # 1. a stream the library has never seen: the call that needs a buffer is refused under capture
    stream = torch.cuda.Stream()
    c1.copy_(c1_keep); c0.zero_()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        st_split = split_k()
        st_plain = plain()
    assert st_split == INVALID_OPERATION, st_split
    assert st_plain == 0
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(c1, c1_keep), "the refused call must not have enqueued anything"
    assert torch.equal(c0, want_c0)
    del graph

    # 2. the same stream after reserving: the first uses of the buffers are inside the capture
    streams_before, _ = clblas_amd.workspace_stats()
    assert clblas_amd.reserve_workspace(4 << 20, 0, 4 << 20, stream=stream.cuda_stream) == 0
    streams_reserved, bytes_reserved = clblas_amd.workspace_stats()
    assert streams_reserved == streams_before + 1 and bytes_reserved >= (8 << 20)
    c1.copy_(c1_keep); tb.copy_(tb_keep)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        sts = [split_k(), trsm()]
    assert sts == [0, 0], sts
    assert clblas_amd.workspace_stats() == (streams_reserved, bytes_reserved), "a capture must not allocate"
    for _ in range(2):
        c1.copy_(c1_keep); tb.copy_(tb_keep)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(c1, want_c1) and torch.equal(tb, want_tb)
    del graph

    # 3. releasing the stream gives its buffers back
    assert clblas_amd.release_stream(stream.cuda_stream) == 0
    assert clblas_amd.workspace_stats()[0] == streams_before


def test_a_routine_of_several_launches_is_refused_before_its_first_launch():
    """DTRSM under capture with its packing buffer reserved but not the buffer its update GEMMs cut K
    into: the call must find that out before the packing pass and the first leaves - which overwrite B
    in place - are enqueued.  It returns clblasInvalidOperation, the capture stays usable and a replay
    leaves B as it was.  The same for a deep rank-k update (a GEMM into a library buffer followed by a
    triangle pass) with only one of its two buffers reserved."""
    import torch
    import clblas_amd
    assert clblas_amd.setup() == 0
    INVALID_OPERATION = -59
    f32, f64 = np.float32, np.float64

    def dev(x):
        return torch.from_numpy(x).cuda()

    n, nrhs = 1100, 100     # leaves of 512, 512, 76 rows; the last update is 76 x 100 x 1024: few tiles, deep K
    ta, tb = dev(oracle.triangular(n, n, True, 7, f64)), dev(oracle.uniform(n * nrhs, 8, f64))
    tb_keep = tb.clone()
    da, dc = dev(oracle.uniform(200 * 8192, 13, f32)), dev(oracle.uniform(200 * 200, 14, f32))
    dc_keep = dc.clone()
    probe = torch.zeros(16, device="cuda")

    def trsm():
        return clblas_amd.dtrsm(COL, LEFT, LOWER, NOTRANS, NONUNIT, n, nrhs, 2.0, ta, 0, n, tb, 0, n)

    def deep_syrk():
        return clblas_amd.syrk("S", COL, LOWER, NOTRANS, 200, 8192, 0.25, da, 0, 200, 0.5, dc, 0, 200)

    # eager, on the default stream: what the calls compute, and that they do ask for a GEMM buffer
    assert trsm() == 0 and deep_syrk() == 0
    torch.cuda.synchronize()
    want_tb, want_dc = tb.clone(), dc.clone()
    assert not torch.equal(want_tb, tb_keep)
    tb.copy_(tb_keep); dc.copy_(dc_keep)

    stream = torch.cuda.Stream()
    assert clblas_amd.reserve_workspace(0, 1 << 20, 4 << 20, stream=stream.cuda_stream) == 0   # no GEMM buffer
    stats = clblas_amd.workspace_stats()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        st_trsm = trsm()
        st_syrk = deep_syrk()
        probe.add_(1.0)          # the capture is still alive after the refusals
    assert st_trsm == INVALID_OPERATION, st_trsm
    assert st_syrk == INVALID_OPERATION, st_syrk
    assert clblas_amd.workspace_stats() == stats
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(tb, tb_keep), "the refused DTRSM must not have touched B"
    assert torch.equal(dc, dc_keep), "the refused SYRK must not have touched C"
    assert float(probe[0]) == 1.0
    del graph

    # with the missing buffer reserved the same capture goes through and replays to the eager results
    assert clblas_amd.reserve_workspace(8 << 20, 0, 0, stream=stream.cuda_stream) == 0
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        sts = [trsm(), deep_syrk()]
    assert sts == [0, 0], sts
    for _ in range(2):
        tb.copy_(tb_keep); dc.copy_(dc_keep)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(tb, want_tb) and torch.equal(dc, want_dc)
    del graph
    assert clblas_amd.release_stream(stream.cuda_stream) == 0


def test_a_gemm_made_of_several_launches_under_capture():
    """A GEMM whose last rows are split off as a product of their own (forced here with
    CLBLAS_AMD_GEMM_PEEL=2) is two launches, the second of which cuts K and needs a scratch buffer: captured
    on a stream without that buffer it is refused before the first launch - C untouched after a replay - and
    with the buffer in place it is captured and replays to the eager result bit for bit."""
    import torch
    import clblas_amd
    import gpu_util
    assert clblas_amd.setup() == 0
    INVALID_OPERATION = -59
    f32 = np.float32
    M, N, K = 1030, 1100, 4096      # 1024 x 1100 x 4096 in whole tiles + a strip of 6 rows: few tiles, deep K
    a = torch.from_numpy(oracle.uniform(M * K, 31, f32)).cuda()
    b = torch.from_numpy(oracle.uniform(K * N, 32, f32)).cuda()
    c = torch.from_numpy(oracle.uniform(M * N, 33, f32)).cuda()
    keep = c.clone()

    def gemm():
        return clblas_amd.sgemm(COL, NOTRANS, NOTRANS, M, N, K, 0.5, a, 0, M, b, 0, K, -1.5, c, 0, M)

    with gpu_util.debug_env(CLBLAS_AMD_GEMM_PEEL=2):
        n0 = clblas_amd.last_dispatch()[1]
        assert gemm() == 0
        torch.cuda.synchronize()
        assert clblas_amd.last_dispatch()[1] - n0 >= 3, "expected the main part, the strip and its reduction pass"
        eager = c.clone()
        c.copy_(keep)

        stream = torch.cuda.Stream()        # a stream that has no scratch buffers yet
        stats = clblas_amd.workspace_stats()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            st = gemm()
        assert st == INVALID_OPERATION, st
        assert clblas_amd.workspace_stats() == stats
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(c, keep), "the refused GEMM must not have touched C"
        del graph

        assert clblas_amd.reserve_workspace(8 << 20, 0, 0, stream=stream.cuda_stream) == 0
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            st = gemm()
        assert st == 0, st
        for rep in range(3):
            c.copy_(keep)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(c, eager), "replay %d differs from the eager result" % rep
        del graph
        assert clblas_amd.release_stream(stream.cuda_stream) == 0
