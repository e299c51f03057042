#!/usr/bin/env python3
"""Benchmark of the xGEMM / xTRSM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--only sgemm|dgemm|dtrsm|cgemm|zgemm|level3|configs|deepk|small|big|trsm|host|tilemodel|vendor|tiles|copy]

A "step" is one call of the hot path on the headline workload (BASELINE config 2: SGEMM,
column-major NN, M=N=K=8192, tight leading dimensions, alpha=1, beta=1, inputs resident in
HBM).  Prints ONE JSON line.  `value` is SGEMM TFLOP/s using the reference's own flop
count 2*M*N*K (src/client/clfunc_xgemm.hpp:95-107); DGEMM (config 4) and DTRSM (config 5,
M*(M+1)*N flops, src/client/clfunc_xtrsm.hpp:70-92) are reported in `extra`, and so are CGEMM /
ZGEMM at the same size (8*M*N*K flops, clfunc_xgemm.hpp:95-107) and S/D SYRK, TRMM, SYMM.
`cpu_baseline` times the CPU oracle (a port of the reference arithmetic, OpenMP over the
host cores) on the same seeded inputs - configs 2 and 1 in full, configs 4 and 5 on stated
sub-problems - and says what a run-time probe of the box's OpenCL loader found for running
the reference itself on a CPU device; it is a reported baseline only.
Inputs of the five BASELINE configurations come from a counter-based generator (one seed per
matrix) that is evaluated on the device and checked against the parity tests' CPU generator.
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


def profiled_traffic(workload, dispatch, kernels_per_call=None):
    """HBM-side bytes per call of one of the 8192 workloads ("sgemm", "dgemm", "dtrsm"), read from the
    tracked rocprofv3 summary (two --pmc runs, FETCH_SIZE and WRITE_SIZE, each scaled by what the same
    counter reads for a plain 1 GiB device copy).  Counters cannot be read from inside this process, so
    the figure is the profile's - and it is only reported when what ran here is what the profile
    measured: for the GEMMs the same tile in one plain launch (`dispatch` is the library's own
    description of its last launch), for DTRSM the same number of kernels per call and the same tile
    in its largest update.  Returns (bytes or None, note)."""
    import re
    letter = {"sgemm": "s", "dgemm": "d", "dtrsm": "d"}[workload]
    ctype = {"s": "float", "d": "double"}[letter]
    m = re.search(r"<%s,(\d+)x(\d+)x(\d+)," % letter, dispatch or "")
    if not m:
        return None, "no GEMM launch on record"
    tile = "gemm_mfma_kernel<%s, %s, %s, %s," % ((ctype,) + m.groups())
    try:
        lines = open(TRAFFIC_PROFILE).read().splitlines()
    except OSError as e:
        return None, "no traffic profile: %s" % e
    if workload == "dtrsm":
        prof_kernels, total, tile_seen = None, None, False
        for line in lines:
            mk = re.match(r"\* dtrsm: (\d+) kernels per call", line)
            if mk:
                prof_kernels = int(mk.group(1))
            mt = re.match(r"\* dtrsm: ([0-9.]+) GB per call", line)
            if mt:
                total = float(mt.group(1)) * 1e9
            cells = [c.strip() for c in line.split("|")]
            if len(cells) >= 6 and cells[1] == "dtrsm" and tile in cells[2]:
                tile_seen = True
        if total is None or prof_kernels is None:
            return None, "profiles/bench_8192_counters.md has no whole-call dtrsm figure with its kernel count"
        if prof_kernels != kernels_per_call or not tile_seen:
            return None, "profiles/bench_8192_counters.md measured %d kernels per call%s, this run launched %s" % (
                prof_kernels, "" if tile_seen else " without %s...>" % tile, kernels_per_call)
        return total, "profiles/bench_8192_counters.md, whole call of %d kernels" % prof_kernels
    if "splits=1 " not in dispatch + " " or "tail_slices=1" not in dispatch:
        return None, "the launch is not a single plain GEMM kernel"
    total, seen = 0.0, set()
    for line in lines:
        cells = [c.strip() for c in line.split("|")]
        if len(cells) >= 6 and cells[1] == workload and cells[3] in ("FETCH_SIZE", "WRITE_SIZE"):
            if tile not in cells[2]:
                return None, "profiles/bench_8192_counters.md was measured on %s, this run used %s" % (cells[2], tile)
            total += float(cells[5].split()[0]) * 1e9
            seen.add(cells[3])
    if seen != {"FETCH_SIZE", "WRITE_SIZE"}:
        return None, "profiles/bench_8192_counters.md has no %s FETCH_SIZE / WRITE_SIZE rows" % workload
    return total, "profiles/bench_8192_counters.md, kernel %s...>" % tile

COL, NOTRANS, TRANS = 1, 0, 1
LEFT, LOWER, NONUNIT = 0, 1, 1

# One seed per matrix (A, B, C take seed, seed + 1, seed + 2); the CPU baseline draws the same streams.
SEEDS = {"sgemm": 1, "dgemm": 11, "dtrsm": 21, "sgemm_config1": 31, "sgemm_config3": 41}


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


# ---- Synthetic inputs: the counter-based generator of the parity tests, evaluated on the device ----
# Value i of stream `seed` is mix(mix(seed) + i * GOLD) with the splitmix64 finaliser `mix`; uniform[-1,1)
# in FP32 takes the top 24 bits (exactly representable), FP64 takes 53 bits; normal(0,1) is Box-Muller
# on values 2i and 2i+1 of the stream.  One seed per matrix.  tests/test_bench_inputs.py checks these
# functions against the CPU generator the GPU parity tests draw from, so the bench and the tests see
# the same matrices for the same seeds.  (torch has no unsigned 64-bit arithmetic: int64 products wrap
# to the same bits, and a logical right shift is an arithmetic one with the sign copies masked off.)

def vendor_rate(torch, call, reps, warmup, work, batches=3):
    """TFLOP/s of a yardstick call of the vendor library that torch uses, or None with the reason on stderr:
    the yardstick is a courtesy column, and a failure inside it (rocBLAS has refused its own workspace
    allocation for solve_triangular in a process that holds many GB in torch's cache) must not take the
    bench line with it."""
    try:
        ms = timed_batch(torch, call, reps, warmup, batches=batches)
        return round(work / ms / 1e9, 2), round(ms, 4)
    except Exception as e:   # noqa: BLE001 - anything the vendor path raises
        sys.stderr.write("bench.py: vendor yardstick unavailable: %s\n" % str(e).splitlines()[0][:200])
        torch.cuda.synchronize()
        return None, None

def _s64(x):
    return x - (1 << 64) if x >= (1 << 63) else x


_GOLD, _MIX1, _MIX2 = _s64(0x9E3779B97F4A7C15), _s64(0xBF58476D1CE4E5B9), _s64(0x94D049BB133111EB)


def _lsr(torch, z, s):
    return (z >> s) & ((1 << (64 - s)) - 1)


def _mix64(torch, z):
    z = z + _GOLD
    z = (z ^ _lsr(torch, z, 30)) * _MIX1
    z = (z ^ _lsr(torch, z, 27)) * _MIX2
    return z ^ _lsr(torch, z, 31)


def _mix64_int(z):
    m = (1 << 64) - 1
    z = (z + 0x9E3779B97F4A7C15) & m
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & m
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & m
    return z ^ (z >> 31)


def stream_u64(torch, seed, first, count, device, stride=1, offset=0):
    """Values first*stride+offset, (first+1)*stride+offset, ... of stream `seed`, as int64 bit patterns."""
    i = torch.arange(first, first + count, device=device, dtype=torch.int64) * stride + offset
    return _mix64(torch, i * _GOLD + _s64(_mix64_int(seed & ((1 << 64) - 1))))


def _in_chunks(torch, n, device, dtype, piece, chunk=1 << 24):
    out = torch.empty(n, device=device, dtype=dtype)
    for first in range(0, n, chunk):
        count = min(chunk, n - first)
        out[first:first + count] = piece(first, count)
    return out


def gen_uniform(torch, n, seed, dtype, device="cuda"):
    """n values uniform in [-1, 1) from stream `seed`."""
    if dtype == torch.float32:
        return _in_chunks(torch, n, device, dtype, lambda f, c: (
            _lsr(torch, stream_u64(torch, seed, f, c, device), 40).double() * (1.0 / 8388608.0) - 1.0).float())
    return _in_chunks(torch, n, device, dtype, lambda f, c: (
        2.0 * (_lsr(torch, stream_u64(torch, seed, f, c, device), 11).double() * (1.0 / 9007199254740992.0)) - 1.0))


def gen_normal(torch, n, seed, dtype, device="cuda"):
    """n values from normal(0, 1): Box-Muller on values 2i, 2i+1 of stream `seed`."""
    import math

    def piece(f, c):
        u1 = 1.0 - _lsr(torch, stream_u64(torch, seed, f, c, device, 2, 0), 11).double() * (1.0 / 9007199254740992.0)
        u2 = _lsr(torch, stream_u64(torch, seed, f, c, device, 2, 1), 11).double() * (1.0 / 9007199254740992.0)
        return (torch.sqrt(-2.0 * torch.log(u1)) * torch.cos((2.0 * math.pi) * u2)).to(dtype)
    return _in_chunks(torch, n, device, dtype, piece)


def gen_triangular(torch, n, seed, dtype, device="cuda"):
    """Column-major n x n (tight ld) lower triangle: strict part uniform[-1,1)/n, diagonal uniform[1,2),
    NaN above the diagonal (element (r, c) is value r + c n of stream `seed`)."""
    unit = _in_chunks(torch, n * n, device, torch.float64, lambda f, c: (
        _lsr(torch, stream_u64(torch, seed, f, c, device), 11).double() * (1.0 / 9007199254740992.0)))
    U = unit.view(n, n)                       # U[c, r] is element (r, c)
    A = (2.0 * U - 1.0) / float(n)
    A.diagonal().copy_(1.0 + U.diagonal())
    upper = torch.ones(n, n, device=device, dtype=torch.bool).tril(-1)   # c > r in this view
    A.masked_fill_(upper, float("nan"))
    return A.to(dtype).reshape(-1)


def opencl_cpu_probe():
    """What the OpenCL loader on this box offers for running the reference clBLAS on the host cores:
    enumerates the platforms and asks each for CL_DEVICE_TYPE_CPU devices.  Returns (usable, text)."""
    import ctypes
    import ctypes.util
    name = ctypes.util.find_library("OpenCL") or "libOpenCL.so.1"
    try:
        cl = ctypes.CDLL(name)
    except OSError as e:
        return False, "no OpenCL loader (%s)" % e
    try:
        nplat = ctypes.c_uint(0)
        rc = cl.clGetPlatformIDs(0, None, ctypes.byref(nplat))
        if rc != 0 or nplat.value == 0:
            return False, "%s loads, clGetPlatformIDs -> code %d, %d platforms" % (name, rc, nplat.value)
        plats = (ctypes.c_void_p * nplat.value)()
        cl.clGetPlatformIDs(nplat.value, plats, None)
        seen, cpus = [], 0
        for p in plats:
            buf = ctypes.create_string_buffer(256)
            cl.clGetPlatformInfo(ctypes.c_void_p(p), 0x0902, 256, buf, None)            # CL_PLATFORM_NAME
            ncpu, nall = ctypes.c_uint(0), ctypes.c_uint(0)
            rc_cpu = cl.clGetDeviceIDs(ctypes.c_void_p(p), ctypes.c_uint64(2), 0, None, ctypes.byref(ncpu))   # CL_DEVICE_TYPE_CPU
            rc_all = cl.clGetDeviceIDs(ctypes.c_void_p(p), ctypes.c_uint64(0xFFFFFFFF), 0, None, ctypes.byref(nall))
            if rc_cpu != 0:
                ncpu.value = 0
            if rc_all != 0:
                nall.value = 0
            cpus += ncpu.value
            seen.append("'%s': %d CPU devices (code %d), %d devices of any type (code %d)" % (
                buf.value.decode(errors="replace"), ncpu.value, rc_cpu, nall.value, rc_all))
        return cpus > 0, "%s: %d platform(s): %s" % (name, nplat.value, "; ".join(seen))
    except Exception as e:   # a loader without these entry points
        return False, "%s: probe failed: %s" % (name, e)


TILE_MODEL_SHAPES = (
    # small products: a few hundred tiles of 64x64 at most (one launch of smaller tiles against a K split)
    (384, 384, 384), (512, 512, 512), (640, 640, 640), (512, 1024, 512), (800, 600, 400), (896, 896, 896), (512, 512, 2048),
    (768, 768, 768), (1000, 1000, 1000), (1280, 1280, 1280), (1500, 1500, 1500), (1792, 1792, 1792), (2000, 2000, 2000),
    (2304, 2304, 2304), (2560, 2560, 2560), (3000, 3000, 3000), (3328, 3328, 3328), (3584, 3584, 3584), (3700, 3700, 3700),
    (4097, 4095, 1031), (5000, 1000, 1000), (1800, 2200, 2600), (4200, 1700, 900), (6000, 6000, 640), (4480, 4480, 2000),
    (3000, 1500, 1000), (1000, 3000, 1500), (5000, 5000, 700), (2500, 7000, 1200), (7000, 2500, 300), (1100, 1000, 520),
    (640, 520, 6000), (300, 900, 5000), (1024, 1024, 8192), (768, 768, 16384), (3000, 200, 6000), (200, 3000, 6000),
    (16384, 128, 2048), (128, 16384, 2048), (4096, 4096, 64), (4096, 4096, 256), (8192, 8192, 128), (6144, 6144, 6144),
    (5120, 5120, 5120), (2048, 2048, 2048), (4096, 4096, 4096), (1536, 1536, 1536),
    (8192, 8192, 8192), (8192, 8192, 2048), (8192, 8192, 512),      # the headline shape and its shorter relatives
    # beyond 8192: tens of rounds of tiles, edges that are no multiples of a tile, odd leading dimensions
    (10000, 10000, 10000), (9000, 9000, 9000), (12000, 12000, 4096), (16000, 16000, 2048), (20000, 20000, 8192),
    (11111, 9999, 5000), (8320, 8320, 8192), (20000, 20000, 256), (12000, 12000, 512), (16000, 16000, 128),
    # one or two rows / columns of tiles over a deep K: the operand that is streamed from HBM is read once
    (10000, 100, 10000), (100, 10000, 10000), (12000, 100, 3000), (16384, 64, 10000), (5000, 200, 8192),
    (100, 5000, 20000), (7000, 300, 5000), (30000, 40, 3000), (9000, 130, 9000), (50000, 50, 5000), (20000, 200, 4096),
)


def tile_model_block(torch, clblas_amd, gen, keep_forced=False):
    """Default tile choice against every forced tile (debug switch CLBLAS_AMD_GEMM_TILE), SGEMM and DGEMM,
    column-major NN, alpha = beta = 1.  Per shape: [default TFLOP/s, default tile, best forced TFLOP/s, best
    tile]; `mispicks` lists the shapes where the default runs more than 3 % behind a different, forced tile."""
    out = {}
    for name, dt, fn in (("sgemm", torch.float32, clblas_amd.sgemm), ("dgemm", torch.float64, clblas_amd.dgemm)):
        ntiles = len(clblas_amd.tile_model_query(name[0], 1024, 1024, 1024)["tiles"])
        rows, mispicks, worst, forced = {}, [], 1.0, {}
        for (M, N, K) in TILE_MODEL_SHAPES:
            if name == "dgemm" and M * N * K > 6.5e10 and M not in (8192, 9000, 10000, 12000):
                continue
            A = torch.rand(M * K, device="cuda", dtype=dt, generator=gen) * 2 - 1
            B = torch.rand(K * N, device="cuda", dtype=dt, generator=gen) * 2 - 1
            C = torch.zeros(M * N, device="cuda", dtype=dt)

            def call():
                st = fn(COL, NOTRANS, NOTRANS, M, N, K, 1.0, A, 0, M, B, 0, K, 1.0, C, 0, M)
                if st != 0:
                    raise RuntimeError("clblas %s returned %d" % (name, st))
            # a few milliseconds per batch (the small products, of some 10 us, in batches of 200)
            reps = int(min(200 if 2.0 * M * N * K < 2e9 else 40, max(2, 2e11 / (2.0 * M * N * K))))
            ms_default = timed_batch(torch, call, reps, 2, batches=3)
            import re
            default_tile = re.search(r"<\w,(\d+x\d+)x", clblas_amd.last_dispatch()[0]).group(1)
            default_desc = clblas_amd.last_dispatch()[0]
            best, best_tile, best_dims, per_tile = None, -1, "", []
            for tile in range(ntiles):
                os.environ["CLBLAS_AMD_GEMM_TILE"] = str(tile)
                clblas_amd.reload_debug_env()
                try:
                    ms = timed_batch(torch, call, reps, 2, batches=3)
                    desc = clblas_amd.last_dispatch()[0]
                    dims = re.search(r"<\w,(\d+x\d+)x", desc).group(1)
                finally:
                    os.environ.pop("CLBLAS_AMD_GEMM_TILE", None)
                    clblas_amd.reload_debug_env()
                # [milliseconds, K ranges, tail slices] of the forced tile: what clblas_amd/fit_tile_model.py fits to
                per_tile.append([round(ms, 5), int(re.search(r"splits=(\d+)", desc).group(1)),
                                 int(re.search(r"tail_slices=(\d+)", desc).group(1))])
                if best is None or ms < best:
                    best, best_tile, best_dims = ms, tile, dims
                if desc == default_desc:
                    # the very launch the default makes, timed a second time: the better of the two counts for
                    # the default (the first measurement of a shape runs right behind its allocations)
                    ms_default = min(ms_default, ms)
            tf = lambda ms: round(2.0 * M * N * K / ms / 1e9, 1)
            key = "%dx%dx%d" % (M, N, K)
            rows[key] = [tf(ms_default), default_tile, tf(best), best_dims]
            forced[key] = {"default_ms": round(ms_default, 5), "default_splits": int(re.search(r"splits=(\d+)", default_desc).group(1)),
                           "tiles": per_tile}
            ratio = best / ms_default if best_dims != default_tile else 1.0   # the same tile twice: timing noise
            worst = min(worst, ratio)
            if ratio < 0.97:
                mispicks.append(key)
            del A, B, C
        out[name] = {"shapes": rows, "mispicks": mispicks, "worst_default_over_best": round(worst, 3)}
        if keep_forced:
            out[name]["forced_ms"] = forced
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
    ap.add_argument("--only", default="", help="run only sgemm, dgemm, dtrsm, cgemm, zgemm, level3, configs, deepk, small, big, trsm, vendor, tiles or copy "
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
        A = gen_uniform(torch, n * n, SEEDS["sgemm"], torch.float32)
        B = gen_uniform(torch, n * n, SEEDS["sgemm"] + 1, torch.float32)
        C = gen_uniform(torch, n * n, SEEDS["sgemm"] + 2, torch.float32)

        def sgemm():
            st = clblas_amd.sgemm(COL, NOTRANS, NOTRANS, n, n, n, 1.0, A, 0, n, B, 0, n, 1.0, C, 0, n)
            if st != 0:
                raise RuntimeError("clblasSgemm returned %d" % st)

        v = (torch.rand(n, device="cuda", dtype=torch.float64, generator=gen) * 2 - 1)
        c0v = C.view(n, n).T.double() @ v   # column-major C times v, before the timed calls
        c0abs_v = C.view(n, n).T.double().abs() @ v.abs()
        wall, ev_ms = timed_calls(torch, sgemm, steps, warmup)
        dispatch = clblas_amd.last_dispatch()[0]
        traffic, traffic_note = profiled_traffic("sgemm", dispatch) if n == 8192 else (None, "size is not 8192")
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
        A = gen_normal(torch, n * n, SEEDS["dgemm"], torch.float64)
        B = gen_normal(torch, n * n, SEEDS["dgemm"] + 1, torch.float64)
        C = gen_normal(torch, n * n, SEEDS["dgemm"] + 2, torch.float64)

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
        d_kernel_tflops = 2.0 * n * n * n / (ev_ms * 1e-3) / 1e12
        d_traffic, d_note = profiled_traffic("dgemm", dgemm_dispatch) if n == 8192 else (None, "size is not 8192")
        extra["dgemm"] = {"workload": "BASELINE config 4: DGEMM column-major NT %d^3, alpha=1, beta=0.5, normal(0,1)" % n,
                          "tflops": round(d_tflops, 3), "ms_per_call": round(wall * 1e3 / steps, 4),
                          "pct_of_fp64_matrix_peak": round(100 * d_tflops / PEAK_FP64_MATRIX, 2),
                          "roofline": {"bound": "mfma", "achieved": round(d_kernel_tflops, 3), "peak": PEAK_FP64_MATRIX,
                                       "unit": "TFLOP/s", "frac": round(d_kernel_tflops / PEAK_FP64_MATRIX, 4),
                                       "traffic": d_traffic, "traffic_source": d_note, "kernel": dgemm_dispatch,
                                       "launch_ms": round(ev_ms, 4)}}
        del A, B, C
    else:
        d_tflops = None

    # ---- DTRSM, BASELINE config 5 -------------------------------------------------------
    if args.only in ("", "dtrsm"):
        A = gen_triangular(torch, n, SEEDS["dtrsm"], torch.float64)   # NaN above the diagonal: must not be read
        Av = A.view(n, n)  # Av[c, r] is element (r, c) of the column-major matrix
        B0 = gen_normal(torch, n * n, SEEDS["dtrsm"] + 1, torch.float64)
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
        trsm_dispatch, trsm_launches_after = clblas_amd.last_dispatch()
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
        kernels_per_call = (trsm_launches_after - launches_before) // (tsteps + 2)
        t_traffic, t_note = profiled_traffic("dtrsm", trsm_dispatch, kernels_per_call) if n == 8192 else (None, "size is not 8192")
        extra["dtrsm"] = {"workload": "BASELINE config 5: DTRSM Left/Lower/NoTrans/NonUnit M=N=%d, alpha=1; A: strict lower triangle "
                                      "uniform[-1,1)/M, diagonal uniform[1,2), NaN above; B normal(0,1)" % n,
                          "tflops": round(t_tflops, 3), "ms_per_call": round(ev_ms, 4),
                          "kernels_per_call": kernels_per_call,
                          "finite": bool(torch.isfinite(B).all().item()),
                          # one call = all of its kernels on one stream: achieved = M (M + 1) N flops over the call's time
                          "roofline": {"bound": "mfma", "achieved": round(t_tflops, 3), "peak": PEAK_FP64_MATRIX,
                                       "unit": "TFLOP/s", "frac": round(t_tflops / PEAK_FP64_MATRIX, 4),
                                       "traffic": t_traffic, "traffic_source": t_note,
                                       "kernel": "%d kernels per call; last update: %s" % (kernels_per_call, trsm_dispatch),
                                       "launch_ms": round(ev_ms, 4)}}
        if d_tflops:
            extra["dtrsm"]["pct_of_dgemm_rate"] = round(100 * t_tflops / d_tflops, 2)
        del A, B, B0

    # Everything from here to the CPU baseline is beside the point of the line (the three BASELINE workloads
    # above are its point): if one of these blocks raises, the blocks after it are skipped, the error is
    # recorded in `extra.extras_error` and on stderr, and the line is printed all the same.
    try:
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

            def sgemm_case(M, N, K, tA, tB, alpha, beta, pad, offs, seed):
                ra, ca = (K, M) if tA else (M, K)   # rows x columns as stored (column-major)
                rb, cb = (N, K) if tB else (K, N)
                lda, ldb, ldc = ra + pad, rb + pad, M + pad
                A = gen_uniform(torch, offs[0] + lda * ca, seed, torch.float32)
                B = gen_uniform(torch, offs[1] + ldb * cb, seed + 1, torch.float32)
                C = gen_uniform(torch, offs[2] + ldc * N, seed + 2, torch.float32)

                bound = clblas_amd.bind("clblasSgemm", COL, tA, tB, M, N, K, alpha, A, offs[0], lda, B, offs[1], ldb, beta, C, offs[2], ldc)

                def call():
                    if bound() != 0:
                        raise RuntimeError("clblasSgemm failed")
                return timed_batch(torch, call, 20 if 2.0 * M * N * K > 1e10 else 100, 5)

            ms = sgemm_case(1024, 1024, 1024, NOTRANS, NOTRANS, 1.0, 0.0, 0, (0, 0, 0), SEEDS["sgemm_config1"])
            shapes["config1 1024x1024x1024 NN"] = {"ms": round(ms, 4), "tflops": round(2.0 * 1024 ** 3 / ms / 1e9, 2)}
            for (M, N, K) in ((4097, 4095, 1031), (65536, 64, 4096), (64, 65536, 4096), (127, 129, 8192)):
                flops = 2.0 * M * N * K
                nbytes = 4.0 * (M * K + K * N + 2.0 * M * N)
                row = {"mfma_bound_ms": round(flops / (PEAK_FP32_MATRIX * 1e12) * 1e3, 4),
                       "hbm_bound_ms": round(nbytes / 8e12 * 1e3, 4)}
                for tA, tB, tag in ((NOTRANS, NOTRANS, "NN"), (NOTRANS, TRANS, "NT"), (TRANS, NOTRANS, "TN"),
                                    (TRANS, TRANS, "TT")):
                    ms = sgemm_case(M, N, K, tA, tB, 0.7, -1.3, 3, (5, 7, 11), SEEDS["sgemm_config3"])
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
                    vendor_tf, _ = vendor_rate(torch, lambda: torch.mm(B, A, out=C), 20, 3, 2.0 * M * N * K)   # C^T = B^T A^T, row-major
                    tf = 2.0 * M * N * K / ms / 1e9
                    dk["%s %dx%dx%d" % (name, M, N, K)] = {
                        "ms": round(ms, 4), "tflops": round(tf, 2), "pct_of_matrix_peak": round(100 * tf / peak, 1),
                        "torch_mm_tflops": vendor_tf}
                    del A, B, C
            extra["small_c_deep_k"] = dk

        # ---- Small products: a few hundred 64x64 tiles at most, which the 64x32 / 32x32 tiles cover in one launch
        #      (column-major NN, alpha = 1, beta = 0; timed through `bind`: a call takes some 10 us); the vendor BLAS
        #      behind torch.mm on the same product beside it. ----
        if args.only in ("", "small"):
            sp = {}
            for name, sym, dt, flop in (("sgemm", "clblasSgemm", torch.float32, 2.0), ("dgemm", "clblasDgemm", torch.float64, 2.0),
                                        ("cgemm", "clblasCgemm", torch.complex64, 8.0), ("zgemm", "clblasZgemm", torch.complex128, 8.0)):
                for (M, N, K) in ((512, 512, 512), (704, 704, 704), (512, 1024, 512), (1024, 1024, 1024)):
                    real = torch.float32 if dt in (torch.float32, torch.complex64) else torch.float64
                    mk = lambda r, c: (torch.rand(r, c, device="cuda", dtype=real, generator=gen) * 2 - 1).to(dt)
                    A, B = mk(K, M), mk(N, K)      # column-major M x K and K x N
                    C = torch.zeros(N, M, device="cuda", dtype=dt)
                    bound = clblas_amd.bind(sym, COL, NOTRANS, NOTRANS, M, N, K, 1.0, A, 0, M, B, 0, K, 0.0, C, 0, M)

                    def call():
                        if bound() != 0:
                            raise RuntimeError("%s failed" % sym)
                    ms = timed_batch(torch, call, 100, 5)
                    kernel = clblas_amd.last_dispatch()[0]
                    vendor_tf, vendor_ms = vendor_rate(torch, lambda: torch.mm(B, A, out=C), 100, 5, flop * M * N * K)
                    sp["%s %dx%dx%d" % (name, M, N, K)] = {
                        "us": round(ms * 1e3, 2), "tflops": round(flop * M * N * K / ms / 1e9, 2),
                        "torch_mm_us": None if vendor_ms is None else round(vendor_ms * 1e3, 2), "kernel": kernel}
                    del A, B, C
            extra["small_products"] = sp

        # ---- Beyond 8192: the part has 288 GB, and matrices of 16384 .. 32768 are ordinary there (1 .. 8.6 GB each).
        #      Column-major NN / left-lower-notrans-nonunit, alpha = beta = 1, tight leading dimensions. ----
        if args.only in ("", "big"):
            big = {}
            for name, dt, fn, peak, dim, reps in (("sgemm 16384", torch.float32, clblas_amd.sgemm, PEAK_FP32_MATRIX, 16384, 3),
                                                ("dgemm 16384", torch.float64, clblas_amd.dgemm, PEAK_FP64_MATRIX, 16384, 2),
                                                ("sgemm 32768", torch.float32, clblas_amd.sgemm, PEAK_FP32_MATRIX, 32768, 1),
                                                ("sgemm 20000x20000x8192", torch.float32, clblas_amd.sgemm, PEAK_FP32_MATRIX, (20000, 20000, 8192), 3)):
                M, N, K = dim if isinstance(dim, tuple) else (dim, dim, dim)
                A = torch.rand(M * K, device="cuda", dtype=dt, generator=gen) * 2 - 1
                B = torch.rand(K * N, device="cuda", dtype=dt, generator=gen) * 2 - 1
                C = torch.zeros(M * N, device="cuda", dtype=dt)

                def call():
                    st = fn(COL, NOTRANS, NOTRANS, M, N, K, 1.0, A, 0, M, B, 0, K, 1.0, C, 0, M)
                    if st != 0:
                        raise RuntimeError("clblas %s returned %d" % (name, st))
                ms = timed_batch(torch, call, reps, 1, batches=2)
                tf = 2.0 * M * N * K / ms / 1e9
                big[name] = {"ms": round(ms, 3), "tflops": round(tf, 2), "pct_of_matrix_peak": round(100 * tf / peak, 1),
                             "kernel": clblas_amd.last_dispatch()[0]}
                del A, B, C
            for name, dt, fn, peak, dim in (("dtrsm 16384", torch.float64, clblas_amd.dtrsm, PEAK_FP64_MATRIX, 16384),
                                          ("strsm 16384", torch.float32, clblas_amd.strsm, PEAK_FP32_MATRIX, 16384),
                                          ("dtrsm 12000", torch.float64, clblas_amd.dtrsm, PEAK_FP64_MATRIX, 12000)):
                A = (torch.rand(dim * dim, device="cuda", dtype=dt, generator=gen) * 2 - 1) / dim
                A.view(dim, dim).diagonal().copy_(torch.rand(dim, device="cuda", dtype=dt, generator=gen) + 1)
                B = torch.randn(dim * dim, device="cuda", dtype=dt, generator=gen)

                def call():
                    st = fn(COL, LEFT, LOWER, NOTRANS, NONUNIT, dim, dim, 1.0, A, 0, dim, B, 0, dim)
                    if st != 0:
                        raise RuntimeError("clblas %s returned %d" % (name, st))
                n0 = clblas_amd.last_dispatch()[1]
                call()
                launches = clblas_amd.last_dispatch()[1] - n0
                ms = timed_batch(torch, call, 2, 0, batches=2)
                tf = dim * (dim + 1.0) * dim / ms / 1e9
                big[name] = {"ms": round(ms, 3), "tflops": round(tf, 2), "pct_of_matrix_peak": round(100 * tf / peak, 1),
                             "kernels_per_call": launches, "finite": bool(torch.isfinite(B).all())}
                del A, B
            extra["beyond_8192"] = big
            torch.cuda.empty_cache()   # tens of GB of freed matrices: back to the device, not kept in torch's cache

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

                    # (arguments converted once: at 512 the Python wrapper's share of a call would be a third of it)
                    bound = clblas_amd.bind("clblas" + name.capitalize(), COL, LEFT, LOWER, NOTRANS, NONUNIT, m, m, 1.0, A, 0, m, B, 0, m)

                    def call():
                        if bound() != 0:
                            raise RuntimeError("clblas %s failed" % name)
                    ms = timed_batch(torch, call, 50, 5)
                    launches = clblas_amd.last_dispatch()[1]
                    call()
                    launches = clblas_amd.last_dispatch()[1] - launches
                    Lt = torch.tril(A.T).contiguous()      # the same triangle as a row-major torch matrix
                    flops = float(m) * (m + 1) * m
                    vendor_tf, _ = vendor_rate(torch, lambda: torch.linalg.solve_triangular(Lt, B, upper=False), 5, 2, flops)
                    ts["%s %d" % (name, m)] = {"ms": round(ms, 4), "tflops": round(flops / ms / 1e9, 2), "kernels_per_call": launches,
                                               "torch_solve_triangular_tflops": vendor_tf}
                    del A, B, Lt
            extra["trsm_sizes"] = ts

        # ---- Host time per call: 10 000 back-to-back calls, CPU clock around the enqueue loop only (the device
        #      is drained before and after, outside the clock).  Calls go straight to the C symbols with
        #      prebuilt ctypes arguments; `ctypes_floor_us` is the same loop on a call that fails validation
        #      at once (M = 0), i.e. the cost of getting from Python into the library and back.  When the
        #      device is slower than the host the loop blocks on the full queue, so `us_per_call` is an upper
        #      bound on the host cost and never less than the device time per call. ----
        if args.only in ("", "host"):
            import ctypes
            lib = clblas_amd.load_library()
            sz, vp, dbl = ctypes.c_size_t, ctypes.c_void_p, ctypes.c_double
            m = 512
            A = gen_triangular(torch, m, 51, torch.float64)
            A = torch.nan_to_num(A)
            B = gen_uniform(torch, m * m, 52, torch.float64)
            C = torch.zeros(m * m, device="cuda", dtype=torch.float64)
            stream = vp(torch.cuda.current_stream().cuda_stream)
            host = {}

            def loop(f, argv, calls):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(calls):
                    f(*argv)
                dt = time.perf_counter() - t0
                torch.cuda.synchronize()
                return dt / calls * 1e6

            def gemm_args(mm):
                return (COL, NOTRANS, NOTRANS, sz(mm), sz(m), sz(m), dbl(1.0), vp(A.data_ptr()), sz(0), sz(m), vp(B.data_ptr()), sz(0),
                        sz(m), dbl(0.0), vp(C.data_ptr()), sz(0), sz(m), stream)

            def trsm_args(mm):
                return (COL, LEFT, LOWER, NOTRANS, NONUNIT, sz(mm), sz(m), dbl(1.0), vp(A.data_ptr()), sz(0), sz(m), vp(B.data_ptr()),
                        sz(0), sz(m), stream)
            for name, f, mk in (("dgemm_512", lib.clblasDgemm, gemm_args), ("dtrsm_512", lib.clblasDtrsm, trsm_args)):
                if f(*mk(m)) != 0:
                    raise RuntimeError("%s failed" % name)
                n0 = clblas_amd.last_dispatch()[1]
                us = min(loop(f, mk(m), 10000) for _ in range(2))
                kernels = (clblas_amd.last_dispatch()[1] - n0) / 20000.0
                floor = loop(f, mk(0), 10000)
                host[name] = {"us_per_call": round(us, 2), "ctypes_floor_us": round(floor, 2), "kernels_per_call": kernels}
            del A, B, C
            extra["host_enqueue_us"] = host

        # ---- The tile choice against the best forced tile, on shapes that are not whole rounds of any tile:
        #      tracks how well the cost model in the launcher (choose_tile) fits the kernels as they are now. ----
        if args.only in ("", "tilemodel"):
            # (--only tilemodel also keeps every forced tile's time: the input of clblas_amd/fit_tile_model.py)
            extra["tile_model"] = tile_model_block(torch, clblas_amd, gen, keep_forced=args.only == "tilemodel")

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
                tf, ms = vendor_rate(torch, lambda: torch.mm(A, B, out=C), 5, 2, fl * n ** 3)
                vy["torch_mm_" + name] = {"tflops": tf, "ms": ms}
                del A, B, C
            T = torch.tril(torch.rand(n, n, device="cuda", dtype=torch.float64, generator=gen) * 2 - 1) / n
            T.diagonal().copy_(torch.rand(n, device="cuda", dtype=torch.float64, generator=gen) + 1)
            Bt = torch.randn(n, n, device="cuda", dtype=torch.float64, generator=gen)
            tf, ms = vendor_rate(torch, lambda: torch.linalg.solve_triangular(T, Bt, upper=False), 3, 1, float(n) * (n + 1) * n)
            vy["torch_solve_triangular_f64"] = {"tflops": tf, "ms": ms}
            vy["workload"] = "square, N=%d, row-major torch tensors, no transposes, beta=0" % n
            del T, Bt
            extra["vendor_yardstick"] = vy

    except Exception as e:   # noqa: BLE001 - whatever an extra raises must not cost the headline
        extra["extras_error"] = "%s: %s" % (type(e).__name__, str(e).splitlines()[0][:300] if str(e) else "")
        sys.stderr.write("bench.py: an extra block failed, the rest of the extras are skipped: %s\n" % extra["extras_error"])
        try:
            torch.cuda.synchronize()
        except Exception:   # noqa: BLE001
            pass

    # ---- CPU baseline: the oracle (port of the reference arithmetic) on the host cores, same seeds as the
    #      GPU legs; config 2 and config 1 in full, configs 4 and 5 on stated sub-problems (the same
    #      streams at the smaller size).  The reference library itself would need a CPU OpenCL device:
    #      the probe below reports what this box's OpenCL loader offers. ----
    cpu = None
    if not args.no_cpu and args.only == "":
        import numpy as np
        import oracle
        usable, seen = opencl_cpu_probe()
        pocl = ("reference-on-PoCL: unavailable (%s%s)" % (
            seen, "; a CPU device is present but no reference libclBLAS is built for it" if usable else ""))

        def clock(f):
            t0 = time.perf_counter()
            st = f()
            if st not in (0, None):
                raise RuntimeError("oracle call returned %s" % st)
            return time.perf_counter() - t0

        m_s = n                         # config 2, the whole workload (about 10 s on 16 host cores)
        a = oracle.uniform(m_s * m_s, SEEDS["sgemm"], np.float32)
        b = oracle.uniform(m_s * m_s, SEEDS["sgemm"] + 1, np.float32)
        c = oracle.uniform(m_s * m_s, SEEDS["sgemm"] + 2, np.float32)
        oracle.gemm(COL, NOTRANS, NOTRANS, 256, 64, 256, 1.0, a, 0, m_s, b, 0, m_s, 1.0, c, 0, m_s)  # warm-up
        dt = clock(lambda: oracle.gemm(COL, NOTRANS, NOTRANS, m_s, m_s, m_s, 1.0, a, 0, m_s, b, 0, m_s, 1.0, c, 0, m_s))
        cpu = {"value": round(2.0 * m_s ** 3 / dt / 1e12, 5), "unit": "TFLOP/s", "cores": oracle.num_threads(),
               "kind": "port",
               "sample": "config 2 in full: oracle SGEMM NN %d^3, one call, %.1f s" % (m_s, dt),
               "reference_on_pocl": pocl}
        del a, b, c
        others = {}
        m1 = 1024                       # config 1 in full
        a = oracle.uniform(m1 * m1, SEEDS["sgemm_config1"], np.float32)
        b = oracle.uniform(m1 * m1, SEEDS["sgemm_config1"] + 1, np.float32)
        c = oracle.uniform(m1 * m1, SEEDS["sgemm_config1"] + 2, np.float32)
        dt = min(clock(lambda: oracle.gemm(COL, NOTRANS, NOTRANS, m1, m1, m1, 1.0, a, 0, m1, b, 0, m1, 0.0, c, 0, m1))
                 for _ in range(3))
        others["config1_sgemm_1024"] = {"value": round(2.0 * m1 ** 3 / dt / 1e12, 5), "unit": "TFLOP/s",
                                        "sample": "config 1 in full: SGEMM NN 1024^3, beta=0, best of 3 calls, %.3f s" % dt}
        # The reference's own CPU code for this operation - the naive gemm its kernel-test tool checks device
        # results against (src/library/tools/ktest/naive/naive_blas.cpp, compiled from the reference tree by
        # oracle/Makefile) - on config 1 in full: one thread, a plain triple loop.
        try:
            cr = c.copy()
            dt_ref = clock(lambda: oracle.ref_gemm(COL, NOTRANS, NOTRANS, m1, m1, m1, 1.0, a, m1, b, m1, 0.0, cr, m1))
            others["config1_sgemm_1024_reference_naive_blas"] = {
                "value": round(2.0 * m1 ** 3 / dt_ref / 1e12, 6), "unit": "TFLOP/s", "cores": 1, "kind": "reference",
                "sample": "config 1 in full through the reference's naive_blas.cpp gemm<float>, one call, %.1f s" % dt_ref}
            del cr
        except Exception as e:   # the checker library is only there when it was built from the reference tree
            others["config1_sgemm_1024_reference_naive_blas"] = {"value": None, "sample": "not available: %s" % e}
        m4 = min(n, 2048)               # config 4 on its leading 2048^3 problem (flops scale with M N K: x%d for the whole)
        a = oracle.normal(m4 * m4, SEEDS["dgemm"], np.float64)
        b = oracle.normal(m4 * m4, SEEDS["dgemm"] + 1, np.float64)
        c = oracle.normal(m4 * m4, SEEDS["dgemm"] + 2, np.float64)
        dt = clock(lambda: oracle.gemm(COL, NOTRANS, TRANS, m4, m4, m4, 1.0, a, 0, m4, b, 0, m4, 0.5, c, 0, m4))
        others["config4_dgemm"] = {"value": round(2.0 * m4 ** 3 / dt / 1e12, 5), "unit": "TFLOP/s",
                                   "sample": "config 4 at M=N=K=%d (1/%d of the flops of %d^3): DGEMM NT, alpha=1, beta=0.5, "
                                             "one call, %.2f s" % (m4, (n // m4) ** 3, n, dt)}
        m5 = min(n, 4096)               # config 5 at 4096: the reference's blocked algorithm (inverted 128-blocks + GEMM sweeps)
        a = oracle.triangular(m5, m5, True, SEEDS["dtrsm"], np.float64)
        b = oracle.normal(m5 * m5, SEEDS["dtrsm"] + 1, np.float64)
        dt = clock(lambda: oracle.trsm_blocked(COL, LEFT, LOWER, NOTRANS, NONUNIT, m5, m5, 1.0, a, 0, m5, b, 0, m5))
        others["config5_dtrsm"] = {"value": round(float(m5) * (m5 + 1) * m5 / dt / 1e12, 5), "unit": "TFLOP/s",
                                   "sample": "config 5 at M=N=%d (1/%d of the flops of %d): oracle restatement of gpu_dtrsm128, "
                                             "one call, %.2f s" % (m5, (n // m5) ** 3, n, dt)}
        del a, b, c
        cpu["other_configs"] = others

    if result is None:
        result = {"metric": "partial run (--only %s)" % args.only, "value": None, "unit": "TFLOP/s", "n_gpus": 1,
                  "steps": steps, "warmup": warmup}
    result["cpu_baseline"] = cpu
    # The bulky tables first, the other two BASELINE workloads last: a reader of the end of the line sees them.
    last = ("sgemm_configs_1_and_3", "trsm_sizes", "host_enqueue_us", "checked", "sgemm_pct_of_fp32_matrix_peak", "dgemm", "dtrsm")
    result["extra"] = {k: extra[k] for k in sorted(extra, key=lambda k: last.index(k) if k in last else -1)}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
