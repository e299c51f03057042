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
    ins = [c1, c2, tb, mb, sc]
    keep = [x.clone() for x in ins]

    def sequence():
        for x, k in zip(ins, keep):
            x.copy_(k)
        sts = [clblas_amd.sgemm(COL, NOTRANS, NOTRANS, 100, 90, 4096, 0.5, a1, 0, 100, b1, 0, 4096, -1.5, c1, 0, 100),
               clblas_amd.dgemm(COL, NOTRANS, TRANS, 1100, 1000, 520, 0.75, a2, 0, 1100, b2, 0, 1000, 0.5, c2, 0, 1100),
               clblas_amd.dtrsm(COL, LEFT, LOWER, NOTRANS, NONUNIT, n, 300, 2.0, ta, 0, n, tb, 0, n),
               clblas_amd.trmm("S", COL, LEFT, LOWER, NOTRANS, NONUNIT, 300, 200, 1.5, ma, 0, 300, mb, 0, 300),
               clblas_amd.syrk("S", COL, LOWER, NOTRANS, 300, 64, 1.0, sa, 0, 300, 0.5, sc, 0, 300)]
        assert sts == [0] * 5, sts

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
