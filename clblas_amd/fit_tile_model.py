#!/usr/bin/env python3
"""Refits the parameters of the SGEMM / DGEMM tile choice model to measured times.

    python bench.py --only tilemodel --no-cpu > tilemodel.json        (on the GPU: every tile forced on some 60 shapes)
    python -m clblas_amd.fit_tile_model tilemodel.json                 (anywhere: needs no GPU)

The launcher (clblas_amd/csrc/gemm_launch.hpp, choose_tile) prices every tile of a type's table for a
product and takes the cheapest; each tile carries these fitted numbers: `eff` (share of the MFMA peak it
is credited with), `alone` (factor when a workgroup has its CU to itself), `k0` (fixed time per
workgroup, as a depth), `tail_extra` (price of a sliced last round, in rounds), `split_gain` (factor on
`eff` in a launch that cuts K into ranges) and `streamed_gain` (factor on `eff` where the operands are too
large for the memory-side cache and come from HBM).  This script takes the
times of every forced tile on every shape from bench.py, evaluates the library's own model through
clblasAmdTileModelQuery with trial parameters set through clblasAmdTileModelParam - the model is not
restated here - and searches, one step of one parameter at a time over a grid around its present value
(always the step that helps most), for the setting with the least regret

    regret = sum over shapes of  time(tile the model picks) / time(best tile) - 1,

counting a pick that is more than 3 % behind the best as one extra percent each (those are what
bench.py reports as mispicks).  Shapes whose forced runs cut K into ranges are left out of the fit (a
forced tile splits by rule, the model's own pick by price: their times do not say what the model's pick
would cost) and listed separately.  Prints the table before and after and the parameters as the
arguments of make_tile_entry in gemm_f32.hip / gemm_f64.hip; it changes no file.
"""
import json
import sys

import clblas_amd

# (k0 and tail_extra first: they say where a tile loses - short K, a sliced last round - and leave its
# credit on long, whole rounds alone; eff moves only where those two cannot explain the times)
GRIDS = {"k0": [-40, -20, -10, 10, 20, 40, 80],
         "tail_extra": [-0.1, -0.05, -0.02, 0.02, 0.05, 0.1, 0.2],
         "alone": [-0.1, -0.05, -0.03, 0.03, 0.05, 0.1],
         "eff": [-0.04, -0.03, -0.02, -0.01, 0.01, 0.02, 0.03, 0.04],
         "split_gain": [-0.06, -0.04, -0.02, 0.02, 0.04, 0.06],
         "streamed_gain": [-0.1, -0.05, -0.02, 0.02, 0.05, 0.1]}
LIMITS = {"eff": (0.6, 1.0), "alone": (0.5, 1.0), "k0": (0.0, 300.0), "tail_extra": (0.0, 1.0), "split_gain": (0.8, 1.2),
          "streamed_gain": (0.5, 1.0)}


def shapes_of(block):
    """[(M, N, K, [ms per tile], [K ranges per tile]), ...] and the keys of shapes that cannot be used (none of
    the forced runs is what the model itself would launch: every tile's forced run cut K by the rule while the
    default did not, or the other way round)."""
    fit, skipped = [], []
    for key, rec in block["forced_ms"].items():
        M, N, K = (int(x) for x in key.split("x"))
        fit.append((M, N, K, [t[0] for t in rec["tiles"]], [t[1] for t in rec["tiles"]]))
    return fit, skipped


def regret(letter, shapes, detail=False):
    """Sum over the shapes of time(picked tile) / time(best tile) - 1, plus a percent for every pick more than
    3 % behind.  A forced tile cuts K by the launcher's rule, the model's own pick by price: where the pick's
    number of K ranges differs from its forced run's, the forced time of that tile is only an estimate of what
    the pick costs; it is used all the same, with a percent on top (a fit must not be able to hide a bad pick
    in a launch nobody timed), and the shape is shown with "?" in the table."""
    total, rows = 0.0, []
    for M, N, K, ms, ranges in shapes:
        q = clblas_amd.tile_model_query(letter, M, N, K)
        pick = q["tile"]
        known = q["splits"] == ranges[pick]
        r = ms[pick] / min(ms) - 1.0
        total += r + (0.01 if r > 0.03 else 0.0) + (0.0 if known else 0.01)
        if detail:
            rows.append(("%dx%dx%d" % (M, N, K), q["tiles"][pick] + ("" if known else " ?"), q["tiles"][ms.index(min(ms))], r))
    return (total, rows) if detail else total


def twins(letter, ntiles):
    """Tiles that are each other's transpose (128x64 and 64x128) and carry the same parameters are moved
    together: changing one of a pair alone only hands its picks to the other.  {first tile: [tiles]}."""
    dims = [tuple(int(x) for x in d.split("x")) for d in clblas_amd.tile_model_query(letter, 1024, 1024, 1024)["tiles"]]
    params = [[clblas_amd.tile_model_param(letter, t, p) for p in GRIDS] for t in range(ntiles)]
    groups, seen = {}, set()
    for t in range(ntiles):
        if t in seen:
            continue
        groups[t] = [u for u in range(t, ntiles) if u == t or (params[u] == params[t] and dims[u][:2] == dims[t][1::-1]
                                                                 and dims[u][2] == dims[t][2])]
        seen.update(groups[t])
    return groups


def fit(letter, shapes, ntiles, sweeps=12):
    """Steepest descent over single steps: every round tries each step of each parameter of each tile
    (twins together) from where the model stands, takes the one that lowers the regret most - the smaller
    step on a tie - and stops when none lowers it.  So the parameters move as little as the times ask for."""
    groups = twins(letter, ntiles)
    for _ in range(sweeps):
        base = regret(letter, shapes)
        best = None  # (regret, relative size of the step, name, {tile: value})
        # (a pair of twins moves together, and each of the two alone: that is how they come apart where the
        # times ask for it)
        moves = list(groups.items()) + [(t, [t]) for g in groups.values() if len(g) > 1 for t in g]
        for tile, group in moves:
            for name, steps in GRIDS.items():
                here = {t: clblas_amd.tile_model_param(letter, t, name) for t in group}
                for d in steps:
                    there = {t: min(max(here[t] + d, LIMITS[name][0]), LIMITS[name][1]) for t in group}
                    for t in group:
                        clblas_amd.tile_model_param(letter, t, name, there[t])
                    cand = (regret(letter, shapes), abs(d) / max(abs(x) for x in steps), name, there)
                    if cand[0] < base - 1e-9 and (best is None or cand[:2] < best[:2]):
                        best = cand
                for t in group:
                    clblas_amd.tile_model_param(letter, t, name, here[t])
        if best is None:
            break
        for t, v in best[3].items():
            clblas_amd.tile_model_param(letter, t, best[2], v)


def main(path):
    data = json.load(open(path))
    model = data["extra"]["tile_model"] if "extra" in data else data
    for letter, name in (("s", "sgemm"), ("d", "dgemm")):
        if name not in model or "forced_ms" not in model[name]:
            print("%s: no forced-tile times in %s (run bench.py --only tilemodel)" % (name, path))
            continue
        shapes, skipped = shapes_of(model[name])
        ntiles = len(shapes[0][3])
        skipped = [r[0] for r in regret(letter, shapes, detail=True)[1] if r[1].endswith("?")]
        before, rows_before = regret(letter, shapes, detail=True)
        params_before = [[clblas_amd.tile_model_param(letter, t, p) for p in GRIDS] for t in range(ntiles)]
        fit(letter, shapes, ntiles)
        after, rows_after = regret(letter, shapes, detail=True)
        print("== %s: %d shapes, of which %d only estimate the present pick (its K ranges differ from the forced run's: %s)" % (
            name, len(shapes), len(skipped), ", ".join(skipped)))
        print("   regret %.4f -> %.4f; picks more than 3 %% behind the best tile: %d -> %d" % (
            before, after, sum(r[3] > 0.03 for r in rows_before), sum(r[3] > 0.03 for r in rows_after)))
        for b, a in zip(rows_before, rows_after):
            if b[1] != a[1] or a[3] > 0.015:
                print("   %-18s before %-11s (%+5.1f %%)   after %-11s (%+5.1f %%)   best %s" % (
                    b[0], b[1], 100 * b[3], a[1], 100 * a[3], a[2]))
        q = clblas_amd.tile_model_query(letter, 1024, 1024, 1024)
        print("   parameters (%s), before -> after:" % ", ".join(GRIDS))
        for t in range(ntiles):
            now = [clblas_amd.tile_model_param(letter, t, p) for p in GRIDS]
            print("     tile %d %-11s %s -> %s" % (t, q["tiles"][t], ["%.3g" % v for v in params_before[t]], ["%.3g" % v for v in now]))


if __name__ == "__main__":
    if len(sys.argv) != 2:
        sys.exit(__doc__)
    main(sys.argv[1])
