#!/usr/bin/env python3
"""Benchmark of the xGEMM / xTRSM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--only sgemm|dgemm|dtrsm|cgemm|zgemm|level3|configs|deepk|trsm|tilemodel|vendor|tiles|copy]

A "step" is one call of the hot path on the headline workload (BASELINE config 2: SGEMM,
column-major NN, M=N=K=8192, tight leading dimensions, alpha=1, beta=1, inputs resident in
HBM).  Prints ONE JSON line.  `value` is SGEMM TFLOP/s using the reference's own flop
count 2*M*N*K (src/client/clfunc_xgemm.hpp:95-107); DGEMM (config 4) and DTRSM (config 5,
M*(M+1)*N flops, src/client/clfunc_xtrsm.hpp:70-92) are reported in `extra`, and so are CGEMM /
ZGEMM at the same size (8*M*N*K flops, clfunc_xgemm.hpp:95-107) and S/D SYRK, TRMM, SYMM.
`cpu_baseline` times the CPU oracle (a port of the reference arithmetic, OpenMP over the
host cores) on a bounded sample of the same workload; it is a reported baseline only.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP32_MATRIX = 157.3  # TFLOP/s, MI355X dense MFMA
PEAK_FP64_MATRIX = 78.6

TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "bench_8192_counters.md")


def profiled_sgemm_traffic(dispatch):
    """HBM-side bytes per launch of the SGEMM 8192^3 kernel, read from the tracked rocprofv3 summary
    (two --pmc runs, FETCH_SIZE and WRITE_SIZE, each scaled by what the same counter reads for a plain
    1 GiB device copy).  Counters cannot be read from inside this process, so the figure is the
    profile's - and it is only reported when the kernel that ran here (`dispatch`, the library's own
    description of its last launch) is the kernel the profile measured: same tile, one launch per call.
    Returns (bytes or None, note)."""
    import re
    m = re.search(r"<s,(\d+)x(\d+)x(\d+),", dispatch)
    if not m or "splits=1 " not in dispatch + " " or "tail_slices=1" not in dispatch:
        return None, "the launch is not a single plain GEMM kernel"
    tile = "gemm_mfma_kernel<float, %s, %s, %s," % m.groups()
    total, seen = 0.0, set()
    try:
        for line in open(TRAFFIC_PROFILE):
            cells = [c.strip() for c in line.split("|")]
            if len(cells) >= 6 and cells[1] == "sgemm" and cells[3] in ("FETCH_SIZE", "WRITE_SIZE"):
                if tile not in cells[2]:
                    return None, "profiles/bench_8192_counters.md was measured on %s, this run used %s" % (cells[2], tile)
                total += float(cells[5].split()[0]) * 1e9
                seen.add(cells[3])
    except OSError as e:
        return None, "no traffic profile: %s" % e
    if seen != {"FETCH_SIZE", "WRITE_SIZE"}:
        return None, "profiles/bench_8192_counters.md has no sgemm FETCH_SIZE / WRITE_SIZE rows"
    return total, "profiles/bench_8192_counters.md, kernel %s...>" % tile

COL, NOTRANS, TRANS = 1, 0, 1
LEFT, LOWER, NONUNIT = 0, 1, 1


def timed_calls(torch, call, steps, warmup, before_each=None):
    """Runs `call` warmup+steps times on torch's current stream; returns (wall seconds for the
    timed steps, mean per-launch milliseconds from HIP events recorded on that stream)."""
    for _ in range(warmup):
        if before_each:
            before_each()
        call()
    torch.cuda.synchronize()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    t0 = time.perf_counter()
    for i in range(steps):
        if before_each:
            before_each()
        starts[i].record()
        call()
        stops[i].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ev_ms = sum(s.elapsed_time(e) for s, e in zip(starts, stops)) / steps
    return wall, ev_ms


def timed_batch(torch, call, reps, warmup, batches=3):
    """Mean milliseconds per call of `reps` back-to-back calls between one pair of HIP events (best
    of `batches`): for launches of tens of microseconds, where an event pair per call would be
    a good part of what is measured."""
    for _ in range(warmup):
        call()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(batches):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(reps):
            call()
        stop.record()
        torch.cuda.synchronize()
        best = min(best, start.elapsed_time(stop) / reps)
    return best


TILE_MODEL_SHAPES = (
    (768, 768, 768), (1000, 1000, 1000), (1280, 1280, 1280), (1500, 1500, 1500), (1792, 1792, 1792), (2000, 2000, 2000),
    (2304, 2304, 2304), (2560, 2560, 2560), (3000, 3000, 3000), (3328, 3328, 3328), (3584, 3584, 3584), (3700, 3700, 3700),
    (4097, 4095, 1031), (5000, 1000, 1000), (1800, 2200, 2600), (4200, 1700, 900), (6000, 6000, 640), (4480, 4480, 2000),
    (3000, 1500, 1000), (1000, 3000, 1500), (5000, 5000, 700), (2500, 7000, 1200), (7000, 2500, 300), (1100, 1000, 520),
    (640, 520, 6000), (300, 900, 5000), (1024, 1024, 8192), (768, 768, 16384), (3000, 200, 6000), (200, 3000, 6000),
    (16384, 128, 2048), (128, 16384, 2048), (4096, 4096, 64), (4096, 4096, 256), (8192, 8192, 128), (6144, 6144, 6144),
    (5120, 5120, 5120), (2048, 2048, 2048), (4096, 4096, 4096), (1536, 1536, 1536),
)


def tile_model_block(torch, clblas_amd, gen):
    """Default tile choice against every forced tile (debug switch CLBLAS_AMD_GEMM_TILE), SGEMM and DGEMM,
    column-major NN, alpha = beta = 1.  Per shape: [default TFLOP/s, default tile, best forced TFLOP/s, best
    tile]; `mispicks` lists the shapes where the default runs more than 3 % behind a different, forced tile."""
    out = {}
    for name, dt, fn, ntiles in (("sgemm", torch.float32, clblas_amd.sgemm, 5), ("dgemm", torch.float64, clblas_amd.dgemm, 2)):
        rows, mispicks, worst = {}, [], 1.0
        for (M, N, K) in TILE_MODEL_SHAPES:
            if name == "dgemm" and M * N * K > 6.5e10:
                continue
            A = torch.rand(M * K, device="cuda", dtype=dt, generator=gen) * 2 - 1
            B = torch.rand(K * N, device="cuda", dtype=dt, generator=gen) * 2 - 1
            C = torch.zeros(M * N, device="cuda", dtype=dt)

            def call():
                st = fn(COL, NOTRANS, NOTRANS, M, N, K, 1.0, A, 0, M, B, 0, K, 1.0, C, 0, M)
                if st != 0:
                    raise RuntimeError("clblas %s returned %d" % (name, st))
            reps = int(min(40, max(4, 2e11 / (2.0 * M * N * K))))   # a few milliseconds per batch
            ms_default = timed_batch(torch, call, reps, 2, batches=3)
            import re
            default_tile = re.search(r"<\w,(\d+x\d+)x", clblas_amd.last_dispatch()[0]).group(1)
            best, best_tile, best_dims = None, -1, ""
            for tile in range(ntiles):
                os.environ["CLBLAS_AMD_GEMM_TILE"] = str(tile)
                clblas_amd.reload_debug_env()
                try:
                    ms = timed_batch(torch, call, reps, 2, batches=3)
                    dims = re.search(r"<\w,(\d+x\d+)x", clblas_amd.last_dispatch()[0]).group(1)
                finally:
                    os.environ.pop("CLBLAS_AMD_GEMM_TILE", None)
                    clblas_amd.reload_debug_env()
                if best is None or ms < best:
                    best, best_tile, best_dims = ms, tile, dims
            tf = lambda ms: round(2.0 * M * N * K / ms / 1e9, 1)
            key = "%dx%dx%d" % (M, N, K)
            rows[key] = [tf(ms_default), default_tile, tf(best), best_dims]
            ratio = best / ms_default if best_dims != default_tile else 1.0   # the same tile twice: timing noise
            worst = min(worst, ratio)
            if ratio < 0.97:
                mispicks.append(key)
            del A, B, C
        out[name] = {"shapes": rows, "mispicks": mispicks, "worst_default_over_best": round(worst, 3)}
    return out


def run_tiles_set(torch, clblas_amd, gen, reps):
    """The launches that profiles/tiles_counters.md reports on, each `reps` times, in a fixed order:
    config 1, the four config-3 shapes (NN and TN), a K split, a sliced tail, DTRSM at 8192 and 2048.
    Prints one JSON line with, per case, the number of kernels the library launched for it, so that a
    rocprofv3 counter file of the same run can be cut into cases by dispatch order."""
    cases = []

    def sgemm_case(name, M, N, K, tA, tB, alpha, beta, pad, offs):
        ra, ca = (K, M) if tA else (M, K)
        rb, cb = (N, K) if tB else (K, N)
        lda, ldb, ldc = ra + pad, rb + pad, M + pad
        A = torch.rand(offs[0] + lda * ca, device="cuda", dtype=torch.float32, generator=gen) * 2 - 1
        B = torch.rand(offs[1] + ldb * cb, device="cuda", dtype=torch.float32, generator=gen) * 2 - 1
        C = torch.rand(offs[2] + ldc * N, device="cuda", dtype=torch.float32, generator=gen) * 2 - 1
        torch.cuda.synchronize()
        n0 = clblas_amd.last_dispatch()[1]
        for _ in range(reps):
            st = clblas_amd.sgemm(COL, tA, tB, M, N, K, alpha, A, offs[0], lda, B, offs[1], ldb, beta, C, offs[2], ldc)
            if st != 0:
                raise RuntimeError("clblasSgemm returned %d" % st)
        torch.cuda.synchronize()
        desc, n1 = clblas_amd.last_dispatch()
        cases.append({"name": name, "calls": reps, "launches": n1 - n0, "flops_per_call": 2.0 * M * N * K,
                      "bytes_per_call": 4.0 * (M * K + K * N + M * N * (2 if beta != 0 else 1)), "last_gemm": desc})

    sgemm_case("config1 sgemm 1024x1024x1024 NN", 1024, 1024, 1024, NOTRANS, NOTRANS, 1.0, 0.0, 0, (0, 0, 0))
    for (M, N, K) in ((4097, 4095, 1031), (65536, 64, 4096), (64, 65536, 4096), (127, 129, 8192)):
        for tA, tag in ((NOTRANS, "NN"), (TRANS, "TN")):
            sgemm_case("config3 sgemm %dx%dx%d %s" % (M, N, K, tag), M, N, K, tA, NOTRANS, 0.7, -1.3, 3, (5, 7, 11))
    sgemm_case("K split: sgemm 1024x1024x8192 NN", 1024, 1024, 8192, NOTRANS, NOTRANS, 1.0, 1.0, 0, (0, 0, 0))
    sgemm_case("sliced tail: sgemm 2304x2304x2304 NN", 2304, 2304, 2304, NOTRANS, NOTRANS, 1.0, 1.0, 0, (0, 0, 0))
    for n in (8192, 2048):
        A = torch.rand(n * n, device="cuda", dtype=torch.float64, generator=gen) * 2 - 1
        A /= n
        A.view(n, n).diagonal().copy_(torch.rand(n, device="cuda", dtype=torch.float64, generator=gen) + 1)
        B0 = torch.randn(n * n, device="cuda", dtype=torch.float64, generator=gen)
        B = B0.clone()
        torch.cuda.synchronize()
        n0 = clblas_amd.last_dispatch()[1]
        for _ in range(reps):
            B.copy_(B0)
            st = clblas_amd.dtrsm(COL, LEFT, LOWER, NOTRANS, NONUNIT, n, n, 1.0, A, 0, n, B, 0, n)
            if st != 0:
                raise RuntimeError("clblasDtrsm returned %d" % st)
        torch.cuda.synchronize()
        cases.append({"name": "dtrsm %d left lower notrans nonunit" % n, "calls": reps,
                      "launches": clblas_amd.last_dispatch()[1] - n0, "flops_per_call": float(n) * (n + 1) * n,
                      "bytes_per_call": 8.0 * (n * (n + 1) / 2 + 2.0 * n * n)})
        del A, B, B0
    print(json.dumps({"metric": "tile set for the counter profile", "reps": reps, "cases": cases}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--size", type=int, default=8192, help="M=N=K (8192 is the BASELINE configuration)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", default="", help="run only sgemm, dgemm, dtrsm, cgemm, zgemm, level3, configs, deepk, trsm, vendor, tiles or copy "
                    "(profiling; copy = a plain 1 GiB device copy used to scale the HBM traffic counters; tiles = every tile "
                    "the five configurations use, --steps times each, for the counter profile)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (one MI355X per box); use --gpus 1")

    import torch
    import clblas_amd
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    torch.cuda.set_device(0)
    if clblas_amd.setup() != 0:
        sys.exit("bench.py: clblasSetup failed (library needs a gfx950 device)")

    n = args.size
    steps, warmup = args.steps, args.warmup
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1234)
    extra = {}
    result = None

    if args.only == "tiles":
        run_tiles_set(torch, clblas_amd, gen, max(1, min(args.steps, 5)))
        return

    if args.only == "copy":
        src = torch.rand(1 << 28, device="cuda", dtype=torch.float32, generator=gen)  # 1 GiB
        dst = torch.empty_like(src)
        wall, ev_ms = timed_calls(torch, lambda: dst.copy_(src), steps, warmup)
        print(json.dumps({"metric": "plain device copy, 1 GiB read + 1 GiB written per launch", "launch_ms": ev_ms,
                          "GBps": round(2 * 2 ** 30 / (ev_ms * 1e-3) / 1e9, 1)}))
        return

    # ---- SGEMM, BASELINE config 2 -------------------------------------------------------
    if args.only in ("", "sgemm"):
        A = torch.rand(n * n, device="cuda", dtype=torch.float32, generator=gen) * 2 - 1
        B = torch.rand(n * n, device="cuda", dtype=torch.float32, generator=gen) * 2 - 1
        C = torch.rand(n * n, device="cuda", dtype=torch.float32, generator=gen) * 2 - 1

        def sgemm():
            st = clblas_amd.sgemm(COL, NOTRANS, NOTRANS, n, n, n, 1.0, A, 0, n, B, 0, n, 1.0, C, 0, n)
            if st != 0:
                raise RuntimeError("clblasSgemm returned %d" % st)

        v = (torch.rand(n, device="cuda", dtype=torch.float64, generator=gen) * 2 - 1)
        c0v = C.view(n, n).T.double() @ v   # column-major C times v, before the timed calls
        c0abs_v = C.view(n, n).T.double().abs() @ v.abs()
        wall, ev_ms = timed_calls(torch, sgemm, steps, warmup)
        dispatch = clblas_amd.last_dispatch()[0]
        traffic, traffic_note = profiled_sgemm_traffic(dispatch) if n == 8192 else (None, "size is not 8192")
        # Self-check of the timed result: every call did C <- A B + C, so after `calls` of them
        # C v = C0 v + calls * A (B v).  Evaluated in double precision on the device.
        calls = steps + warmup
        Ad, Bd = A.view(n, n).T.double(), B.view(n, n).T.double()
        want = c0v + calls * (Ad @ (Bd @ v))
        got = C.view(n, n).T.double() @ v
        # Tolerance 8 u calls |C| |v| by elements of C v: far below the worst-case bound
        # calls (K + 2) u (...), so that a tile computed wrongly would show; the measured ratio is reported.
        del c0abs_v
        bound = 8 * calls * 2.0 ** -24 * (C.view(n, n).T.double().abs() @ v.abs())
        sgemm_check = float(((got - want).abs() / bound).max())
        del Ad, Bd, want, got, bound
        flops = 2.0 * n * n * n
        ms_per_step = wall * 1e3 / steps
        tflops = flops / (wall / steps) / 1e12
        kernel_tflops = flops / (ev_ms * 1e-3) / 1e12
        result = {
            "metric": "SGEMM TFLOP/s at %d^3 (col-major NN, alpha=1, beta=1) on 1 MI355X" % n,
            "value": round(tflops, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
            "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": "BASELINE config 2: SGEMM column-major NN M=N=K=%d, tight ld, alpha=1, beta=1, "
                                   "uniform[-1,1)" % n},
            "roofline": {"bound": "mfma", "achieved": round(kernel_tflops, 3), "peak": PEAK_FP32_MATRIX,
                         "unit": "TFLOP/s", "frac": round(kernel_tflops / PEAK_FP32_MATRIX, 4),
                         "traffic": traffic, "traffic_source": traffic_note,
                         "kernel": dispatch, "launch_ms": round(ev_ms, 4)},
        }
        extra["checked"] = {"sgemm": {"what": "C v = C0 v + calls A (B v) after the timed calls, in double precision",
                                      "tolerance": "8 u calls |C| |v|", "worst_error_over_tolerance": float("%.3g" % sgemm_check), "ok": sgemm_check <= 1.0}}
        if sgemm_check > 1.0:
            raise RuntimeError("SGEMM result fails its linearity check: %.3g of the bound" % sgemm_check)
        extra["sgemm_pct_of_fp32_matrix_peak"] = round(100 * tflops / PEAK_FP32_MATRIX, 2)
        del A, B, C

    # ---- DGEMM, BASELINE config 4 -------------------------------------------------------
    if args.only in ("", "dgemm"):
        A = torch.randn(n * n, device="cuda", dtype=torch.float64, generator=gen)
        B = torch.randn(n * n, device="cuda", dtype=torch.float64, generator=gen)
        C = torch.randn(n * n, device="cuda", dtype=torch.float64, generator=gen)

        def dgemm():
            st = clblas_amd.dgemm(COL, NOTRANS, TRANS, n, n, n, 1.0, A, 0, n, B, 0, n, 0.5, C, 0, n)
            if st != 0:
                raise RuntimeError("clblasDgemm returned %d" % st)

        v = (torch.rand(n, device="cuda", dtype=torch.float64, generator=gen) * 2 - 1)
        c0v = C.view(n, n).T @ v
        c0abs_v = C.view(n, n).T.abs() @ v.abs()
        wall, ev_ms = timed_calls(torch, dgemm, steps, warmup)
        dgemm_dispatch = clblas_amd.last_dispatch()[0]
        # C <- A B^T + C / 2 every call: C v = C0 v / 2^calls + (2 - 2^(1 - calls)) A (B^T v)
        calls = steps + warmup
        Am, Bm = A.view(n, n).T, B.view(n, n).T       # column-major views; B is stored N x K and used transposed
        want = c0v * 0.5 ** calls + (2 - 2.0 ** (1 - calls)) * (Am @ (Bm.T @ v))
        got = C.view(n, n).T @ v
        del c0abs_v
        bound = 8 * calls * 2.0 ** -53 * (C.view(n, n).T.abs() @ v.abs())
        dgemm_check = float(((got - want).abs() / bound).max())
        del want, got, bound
        if dgemm_check > 1.0:
            raise RuntimeError("DGEMM result fails its linearity check: %.3g of the bound" % dgemm_check)
        extra.setdefault("checked", {})["dgemm"] = {"what": "C v = C0 v / 2^calls + (2 - 2^(1-calls)) A (B^T v), in double precision",
                                                     "tolerance": "8 u calls |C| |v|", "worst_error_over_tolerance": float("%.3g" % dgemm_check), "ok": True}
        d_tflops = 2.0 * n * n * n / (wall / steps) / 1e12
        extra["dgemm"] = {"workload": "BASELINE config 4: DGEMM column-major NT %d^3, alpha=1, beta=0.5, normal(0,1)" % n,
                          "tflops": round(d_tflops, 3), "ms_per_call": round(wall * 1e3 / steps, 4),
                          "launch_ms": round(ev_ms, 4), "kernel": dgemm_dispatch,
                          "pct_of_fp64_matrix_peak": round(100 * d_tflops / PEAK_FP64_MATRIX, 2)}
        del A, B, C
    else:
        d_tflops = None

    # ---- DTRSM, BASELINE config 5 -------------------------------------------------------
    if args.only in ("", "dtrsm"):
        A = torch.rand(n * n, device="cuda", dtype=torch.float64, generator=gen) * 2 - 1
        A /= n
        Av = A.view(n, n)  # Av[c, r] is element (r, c) of the column-major matrix
        Av.diagonal().copy_(torch.rand(n, device="cuda", dtype=torch.float64, generator=gen) + 1)
        Av.copy_(torch.where(torch.ones(n, n, device="cuda", dtype=torch.bool).tril(-1), torch.full_like(Av, float("nan")), Av))
        B0 = torch.randn(n * n, device="cuda", dtype=torch.float64, generator=gen)
        B = B0.clone()

        def restore():
            B.copy_(B0)

        def dtrsm():
            st = clblas_amd.dtrsm(COL, LEFT, LOWER, NOTRANS, NONUNIT, n, n, 1.0, A, 0, n, B, 0, n)
            if st != 0:
                raise RuntimeError("clblasDtrsm returned %d" % st)

        tsteps = max(3, steps // 2)
        launches_before = clblas_amd.last_dispatch()[1]
        wall, ev_ms = timed_calls(torch, dtrsm, tsteps, 2, before_each=restore)
        t_tflops = float(n) * (n + 1) * n / (ev_ms * 1e-3) / 1e12
        # Residual of the last timed solve on sampled right-hand sides: ||L X - B|| / (||L|| ||X|| + ||B||)
        # by columns (inf-norms, double precision on the device) against 2 n eps.
        cols = torch.randint(0, n, (64,), device="cuda", generator=gen)
        L = torch.tril(torch.nan_to_num(Av.T))        # Av[c, r] is element (r, c)
        X, Bs = B.view(n, n).index_select(0, cols).T, B0.view(n, n).index_select(0, cols).T
        R = L @ X - Bs
        be = R.abs().amax(dim=0) / (float(L.abs().sum(dim=1).max()) * X.abs().amax(dim=0) + Bs.abs().amax(dim=0))
        dtrsm_check = float(be.max()) / (2 * n * 2.0 ** -52)
        del L, X, Bs, R
        if not (dtrsm_check <= 1.0):
            raise RuntimeError("DTRSM result fails its residual check: %.3g of the bound" % dtrsm_check)
        extra.setdefault("checked", {})["dtrsm"] = {"what": "backward error of 64 sampled right-hand sides against 2 n eps",
                                                     "worst_error_over_bound": float("%.3g" % dtrsm_check), "ok": True}
        extra["dtrsm"] = {"workload": "BASELINE config 5: DTRSM Left/Lower/NoTrans/NonUnit M=N=%d, alpha=1" % n,
                          "tflops": round(t_tflops, 3), "ms_per_call": round(ev_ms, 4),
                          "kernels_per_call": (clblas_amd.last_dispatch()[1] - launches_before) // (tsteps + 2),
                          "finite": bool(torch.isfinite(B).all().item())}
        if d_tflops:
            extra["dtrsm"]["pct_of_dgemm_rate"] = round(100 * t_tflops / d_tflops, 2)
        del A, B, B0

    # ---- CGEMM / ZGEMM at the same size (no BASELINE configuration; the neighbours of the path) ----
    for name, dt, fn, peak in (("cgemm", torch.complex64, clblas_amd.cgemm, PEAK_FP32_MATRIX),
                               ("zgemm", torch.complex128, clblas_amd.zgemm, PEAK_FP64_MATRIX)):
        if args.only not in ("", name):
            continue
        rdt = torch.float32 if dt == torch.complex64 else torch.float64
        A, B, C = (torch.view_as_complex(torch.rand(n * n, 2, device="cuda", dtype=rdt, generator=gen) * 2 - 1)
                   for _ in range(3))

        def cgemm():
            st = fn(COL, NOTRANS, NOTRANS, n, n, n, 1.0 + 0.5j, A, 0, n, B, 0, n, 0.5 - 0.25j, C, 0, n)
            if st != 0:
                raise RuntimeError("clblas%s returned %d" % (name, st))

        csteps = max(3, steps // 2)
        wall, ev_ms = timed_calls(torch, cgemm, csteps, 2)
        c_tflops = 8.0 * n * n * n / (ev_ms * 1e-3) / 1e12
        extra[name] = {"workload": "%s column-major NN %d^3, alpha=1+0.5i, beta=0.5-0.25i, uniform[-1,1)" % (name.upper(), n),
                       "tflops": round(c_tflops, 3), "launch_ms": round(ev_ms, 4),
                       "pct_of_matrix_peak": round(100 * c_tflops / peak, 2)}
        del A, B, C

    # ---- SYRK / TRMM / SYMM / SYR2K and the complex-only routines at the same size (useful flops only: the reference client's counts) ----
    if args.only in ("", "level3"):
        lv = {}
        for pre, dt, peak in (("S", torch.float32, PEAK_FP32_MATRIX), ("D", torch.float64, PEAK_FP64_MATRIX)):
            A = torch.rand(n * n, device="cuda", dtype=dt, generator=gen) * 2 - 1
            B0 = torch.rand(n * n, device="cuda", dtype=dt, generator=gen) * 2 - 1
            B = B0.clone()
            C = torch.rand(n * n, device="cuda", dtype=dt, generator=gen) * 2 - 1
            cases = (
                ("syrk", float(n) * (n + 1) * n, None,
                 lambda: clblas_amd.syrk(pre, COL, LOWER, NOTRANS, n, n, 1.0, A, 0, n, 1.0, C, 0, n)),
                ("trmm", float(n) * (n + 1) * n, lambda: B.copy_(B0),
                 lambda: clblas_amd.trmm(pre, COL, LEFT, LOWER, NOTRANS, NONUNIT, n, n, 1.0, A, 0, n, B, 0, n)),
                ("symm", 2.0 * n * n * n, None,
                 lambda: clblas_amd.symm(pre, COL, LEFT, LOWER, n, n, 1.0, A, 0, n, B0, 0, n, 1.0, C, 0, n)),
                ("syr2k", 2.0 * n * n * n + n, None,
                 lambda: clblas_amd.syr2k(pre, COL, LOWER, NOTRANS, n, n, 1.0, A, 0, n, B0, 0, n, 1.0, C, 0, n)),
            )
            for name, fl, before, fn in cases:
                def call(fn=fn, name=name):
                    st = fn()
                    if st != 0:
                        raise RuntimeError("clblas%s%s returned %d" % (pre, name, st))
                wall, ev_ms = timed_calls(torch, call, max(3, steps // 4), 2, before_each=before)
                tf = fl / (ev_ms * 1e-3) / 1e12
                lv[pre.lower() + name] = {"tflops": round(tf, 2), "ms_per_call": round(ev_ms, 4),
                                          "pct_of_matrix_peak": round(100 * tf / peak, 1)}
            del A, B, B0, C
        # complex types: the Hermitian routines and the triangular solve (flop counts of the reference client)
        for pre, dt, peak in (("C", torch.complex64, PEAK_FP32_MATRIX), ("Z", torch.complex128, PEAK_FP64_MATRIX)):
            rdt = torch.float32 if dt == torch.complex64 else torch.float64
            A, B0, C = (torch.view_as_complex(torch.rand(n * n, 2, device="cuda", dtype=rdt, generator=gen) * 2 - 1)
                        for _ in range(3))
            B = B0.clone()
            T = A / n  # well-conditioned triangle: small off-diagonal entries, diagonal in [1, 2)
            T.view(n, n).diagonal().copy_(torch.rand(n, device="cuda", dtype=rdt, generator=gen) + 1)
            trsm = clblas_amd.ctrsm if pre == "C" else clblas_amd.ztrsm
            cases = (
                ("herk", 4.0 * n * n * (n + 1), None,
                 lambda: clblas_amd.herk(pre, COL, LOWER, NOTRANS, n, n, 1.0, A, 0, n, 1.0, C, 0, n)),
                ("her2k", 8.0 * n * n * n + 2 * n, None,
                 lambda: clblas_amd.her2k(pre, COL, LOWER, NOTRANS, n, n, 1.0 + 0.5j, A, 0, n, B0, 0, n, 1.0, C, 0, n)),
                ("hemm", 8.0 * n * n * n, None,
                 lambda: clblas_amd.hemm(pre, COL, LEFT, LOWER, n, n, 1.0 + 0.5j, A, 0, n, B0, 0, n, 1.0, C, 0, n)),
                ("trsm", 4.0 * n * (n + 1) * n, lambda: B.copy_(B0),
                 lambda: trsm(COL, LEFT, LOWER, NOTRANS, NONUNIT, n, n, 1.0, T, 0, n, B, 0, n)),
            )
            for name, fl, before, fn in cases:
                def call(fn=fn, name=name):
                    st = fn()
                    if st != 0:
                        raise RuntimeError("clblas%s%s returned %d" % (pre, name, st))
                wall, ev_ms = timed_calls(torch, call, max(3, steps // 4), 2, before_each=before)
                tf = fl / (ev_ms * 1e-3) / 1e12
                lv[pre.lower() + name] = {"tflops": round(tf, 2), "ms_per_call": round(ev_ms, 4),
                                          "pct_of_matrix_peak": round(100 * tf / peak, 1)}
            if not bool(torch.isfinite(torch.view_as_real(B)).all().item()):
                raise RuntimeError("clblas%strsm produced non-finite values" % pre)
            del A, B, B0, C, T
        lv["workload"] = "column-major, lower, left, no transpose, N=M=K=%d, alpha=beta=1 (complex: alpha=1+0.5i)" % n
        extra["level3"] = lv

    # ---- BASELINE configs 1 and 3: SGEMM 1024^3 and the edge-shape sweep (ld = rows + 3, offsets 5/7/11,
    #      alpha = 0.7, beta = -1.3, all four transposes).  Each against its own bound: MFMA time and HBM time
    #      of the algorithmic bytes 4 (MK + KN + 2 MN). ----
    if args.only in ("", "configs"):
        shapes = {}

        def sgemm_case(M, N, K, tA, tB, alpha, beta, pad, offs):
            ra, ca = (K, M) if tA else (M, K)   # rows x columns as stored (column-major)
            rb, cb = (N, K) if tB else (K, N)
            lda, ldb, ldc = ra + pad, rb + pad, M + pad
            A = torch.rand(offs[0] + lda * ca, device="cuda", dtype=torch.float32, generator=gen) * 2 - 1
            B = torch.rand(offs[1] + ldb * cb, device="cuda", dtype=torch.float32, generator=gen) * 2 - 1
            C = torch.rand(offs[2] + ldc * N, device="cuda", dtype=torch.float32, generator=gen) * 2 - 1

            def call():
                st = clblas_amd.sgemm(COL, tA, tB, M, N, K, alpha, A, offs[0], lda, B, offs[1], ldb, beta, C, offs[2],
                                      ldc)
                if st != 0:
                    raise RuntimeError("clblasSgemm returned %d" % st)
            return timed_batch(torch, call, 20 if 2.0 * M * N * K > 1e10 else 100, 5)

        ms = sgemm_case(1024, 1024, 1024, NOTRANS, NOTRANS, 1.0, 0.0, 0, (0, 0, 0))
        shapes["config1 1024x1024x1024 NN"] = {"ms": round(ms, 4), "tflops": round(2.0 * 1024 ** 3 / ms / 1e9, 2)}
        for (M, N, K) in ((4097, 4095, 1031), (65536, 64, 4096), (64, 65536, 4096), (127, 129, 8192)):
            flops = 2.0 * M * N * K
            nbytes = 4.0 * (M * K + K * N + 2.0 * M * N)
            row = {"mfma_bound_ms": round(flops / (PEAK_FP32_MATRIX * 1e12) * 1e3, 4),
                   "hbm_bound_ms": round(nbytes / 8e12 * 1e3, 4)}
            for tA, tB, tag in ((NOTRANS, NOTRANS, "NN"), (NOTRANS, TRANS, "NT"), (TRANS, NOTRANS, "TN"),
                                (TRANS, TRANS, "TT")):
                ms = sgemm_case(M, N, K, tA, tB, 0.7, -1.3, 3, (5, 7, 11))
                row[tag] = {"ms": round(ms, 4), "tflops": round(flops / ms / 1e9, 2),
                            "GBps": round(nbytes / ms / 1e6, 1)}
            shapes["config3 %dx%dx%d" % (M, N, K)] = row
        # What the memory system gives a plain streaming kernel on this box (1 GiB read + 1 GiB written):
        # the yardstick for the HBM-side figures of the skinny shapes above.
        src = torch.empty(1 << 28, device="cuda", dtype=torch.float32)
        dst = torch.empty_like(src)
        copy_ms = timed_batch(torch, lambda: dst.copy_(src), 5, 2)
        shapes["plain_device_copy_GBps"] = round(2 * 2 ** 30 / copy_ms / 1e6, 1)
        del src, dst
        extra["sgemm_configs_1_and_3"] = shapes

    # ---- Small C, deep K: fewer tiles than CUs, so the tile choice cuts K into ranges (column-major NN,
    #      alpha = beta = 1); the vendor BLAS behind torch.mm on the same product beside it. ----
    if args.only in ("", "deepk"):
        dk = {}
        for name, dt, fn, peak in (("sgemm", torch.float32, clblas_amd.sgemm, PEAK_FP32_MATRIX),
                                   ("dgemm", torch.float64, clblas_amd.dgemm, PEAK_FP64_MATRIX)):
            for (M, N, K) in ((1024, 1024, 16384), (768, 768, 16384), (3000, 200, 6000)):
                A = torch.rand(K, M, device="cuda", dtype=dt, generator=gen) * 2 - 1   # column-major M x K
                B = torch.rand(N, K, device="cuda", dtype=dt, generator=gen) * 2 - 1   # column-major K x N
                C = torch.zeros(N, M, device="cuda", dtype=dt)

                def call():
                    st = fn(COL, NOTRANS, NOTRANS, M, N, K, 1.0, A, 0, M, B, 0, K, 1.0, C, 0, M)
                    if st != 0:
                        raise RuntimeError("clblas %s returned %d" % (name, st))
                ms = timed_batch(torch, call, 20, 3)
                vendor_ms = timed_batch(torch, lambda: torch.mm(B, A, out=C), 20, 3)   # C^T = B^T A^T, row-major
                tf = 2.0 * M * N * K / ms / 1e9
                dk["%s %dx%dx%d" % (name, M, N, K)] = {
                    "ms": round(ms, 4), "tflops": round(tf, 2), "pct_of_matrix_peak": round(100 * tf / peak, 1),
                    "torch_mm_tflops": round(2.0 * M * N * K / vendor_ms / 1e9, 2)}
                del A, B, C
        extra["small_c_deep_k"] = dk

    # ---- TRSM below 8192 (left, lower, no transpose, non-unit; square B, alpha = 1): a chain of short
    #      dependent launches (packing pass, leaves of 512 equations, GEMM updates).  Each solve overwrites B
    #      with a solution of similar size (diagonal 1..2, off-diagonal < 1/n), so calls can be repeated in
    #      place.  The vendor's torch.linalg.solve_triangular on the same box beside it. ----
    if args.only in ("", "trsm"):
        ts = {}
        for name, dt, fn in (("dtrsm", torch.float64, clblas_amd.dtrsm), ("strsm", torch.float32, clblas_amd.strsm)):
            for m in (512, 1024, 2048, 4096):
                A = (torch.rand(m, m, device="cuda", dtype=dt, generator=gen) - 0.5) / m     # column-major
                A.diagonal().copy_(torch.rand(m, device="cuda", dtype=dt, generator=gen) + 1)
                B = torch.rand(m, m, device="cuda", dtype=dt, generator=gen)

                def call():
                    st = fn(COL, LEFT, LOWER, NOTRANS, NONUNIT, m, m, 1.0, A, 0, m, B, 0, m)
                    if st != 0:
                        raise RuntimeError("clblas %s returned %d" % (name, st))
                ms = timed_batch(torch, call, 20, 3)
                launches = clblas_amd.last_dispatch()[1]
                call()
                launches = clblas_amd.last_dispatch()[1] - launches
                Lt = torch.tril(A.T).contiguous()      # the same triangle as a row-major torch matrix
                vendor_ms = timed_batch(torch, lambda: torch.linalg.solve_triangular(Lt, B, upper=False), 5, 2)
                flops = float(m) * (m + 1) * m
                ts["%s %d" % (name, m)] = {"ms": round(ms, 4), "tflops": round(flops / ms / 1e9, 2), "kernels_per_call": launches,
                                           "torch_solve_triangular_tflops": round(flops / vendor_ms / 1e9, 2)}
                del A, B, Lt
        extra["trsm_sizes"] = ts

    # ---- The tile choice against the best forced tile, on shapes that are not whole rounds of any tile:
    #      tracks how well the cost model in the launcher (choose_tile) fits the kernels as they are now. ----
    if args.only in ("", "tilemodel"):
        extra["tile_model"] = tile_model_block(torch, clblas_amd, gen)

    # ---- Yardstick: the vendor BLAS that torch calls (rocBLAS / hipBLASLt) on the same box, same sizes.
    #      Not the reference and not a target of the parity tests: it shows what the part gives a
    #      tuned library.  FP32 without TF32-style shortcuts. ----
    if args.only in ("", "vendor"):
        torch.backends.cuda.matmul.allow_tf32 = False
        vy = {}
        for name, dt, fl in (("sgemm", torch.float32, 2.0), ("dgemm", torch.float64, 2.0),
                             ("cgemm", torch.complex64, 8.0), ("zgemm", torch.complex128, 8.0)):
            real = torch.float32 if dt in (torch.float32, torch.complex64) else torch.float64
            shape = (n, n, 2) if dt.is_complex else (n, n)
            mk = lambda: torch.rand(shape, device="cuda", dtype=real, generator=gen) * 2 - 1
            A, B = mk(), mk()
            if dt.is_complex:
                A, B = torch.view_as_complex(A), torch.view_as_complex(B)
            C = torch.empty(n, n, device="cuda", dtype=dt)
            ms = timed_batch(torch, lambda: torch.mm(A, B, out=C), 5, 2)
            vy["torch_mm_" + name] = {"tflops": round(fl * n ** 3 / ms / 1e9, 2), "ms": round(ms, 3)}
            del A, B, C
        T = torch.tril(torch.rand(n, n, device="cuda", dtype=torch.float64, generator=gen) * 2 - 1) / n
        T.diagonal().copy_(torch.rand(n, device="cuda", dtype=torch.float64, generator=gen) + 1)
        Bt = torch.randn(n, n, device="cuda", dtype=torch.float64, generator=gen)
        ms = timed_batch(torch, lambda: torch.linalg.solve_triangular(T, Bt, upper=False), 3, 1)
        vy["torch_solve_triangular_f64"] = {"tflops": round(float(n) * (n + 1) * n / ms / 1e9, 2), "ms": round(ms, 3)}
        vy["workload"] = "square, N=%d, row-major torch tensors, no transposes, beta=0" % n
        del T, Bt
        extra["vendor_yardstick"] = vy

    # ---- CPU baseline: the oracle (port of the reference arithmetic) on the host cores ----
    cpu = None
    if not args.no_cpu and args.only == "":
        import numpy as np
        import oracle
        m_s, n_s, k_s = n, n, n           # the whole workload (about 10 s on 16 host cores)
        a = oracle.uniform(m_s * k_s, 1, np.float32)
        b = oracle.uniform(k_s * n_s, 2, np.float32)
        c = oracle.uniform(m_s * n_s, 3, np.float32)
        oracle.gemm(COL, NOTRANS, NOTRANS, 256, 64, 256, 1.0, a, 0, m_s, b, 0, k_s, 1.0, c, 0, m_s)  # warm-up
        t0 = time.perf_counter()
        oracle.gemm(COL, NOTRANS, NOTRANS, m_s, n_s, k_s, 1.0, a, 0, m_s, b, 0, k_s, 1.0, c, 0, m_s)
        dt = time.perf_counter() - t0
        cpu = {"value": round(2.0 * m_s * n_s * k_s / dt / 1e12, 5), "unit": "TFLOP/s", "cores": oracle.num_threads(),
               "kind": "port",
               "sample": "oracle SGEMM NN, M=%d N=%d K=%d, one call (%.1f s); the reference clBLAS itself needs an "
                         "OpenCL device (PoCL), which this image does not have" % (m_s, n_s, k_s, dt)}

    if result is None:
        result = {"metric": "partial run (--only %s)" % args.only, "value": None, "unit": "TFLOP/s", "n_gpus": 1,
                  "steps": steps, "warmup": warmup}
    result["cpu_baseline"] = cpu
    result["extra"] = extra
    print(json.dumps(result))


if __name__ == "__main__":
    main()
