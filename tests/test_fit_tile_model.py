"""The tile-model fitting script on synthetic times (no GPU: the model is a host function of the library).

Times per tile are made from the model's own costs, so the model as shipped has no regret on them; a
parameter is then moved by one step of the fit's grid through clblasAmdTileModelParam, far enough to change a
pick, and the fit has to bring the regret back to zero."""
import json

import pytest

import clblas_amd
from clblas_amd import fit_tile_model

SHAPES = [(2048, 2048, 2048), (4096, 4096, 4096), (3000, 3000, 3000), (8192, 8192, 512), (1500, 1500, 1500),
          (5000, 1000, 1000), (1100, 1000, 520), (8192, 8192, 8192), (2560, 2560, 2560), (6144, 6144, 6144)]


def synthetic_block(letter):
    """The "forced_ms" block bench.py --only tilemodel writes, with times proportional to the model's costs."""
    forced = {}
    for (M, N, K) in SHAPES:
        q = clblas_amd.tile_model_query(letter, M, N, K)
        assert q["splits"] == 1
        forced["%dx%dx%d" % (M, N, K)] = {"default_splits": 1,
                                          "tiles": [[c * K * 1e-9, 1, 1] for c in q["costs"]]}
    # (none of these shapes cuts K, so every pick is one of the timed launches)
    return {"forced_ms": forced}


@pytest.fixture
def restore_params():
    saved = {(l, t, p): clblas_amd.tile_model_param(l, t, p)
             for l, n in (("s", 7), ("d", 4)) for t in range(n) for p in fit_tile_model.GRIDS}
    yield
    for (l, t, p), v in saved.items():
        clblas_amd.tile_model_param(l, t, p, v)


@pytest.mark.parametrize("letter,ntiles", [("s", 7), ("d", 4)])
def test_model_has_no_regret_on_its_own_costs_and_fit_repairs_a_spoiled_parameter(letter, ntiles, restore_params):
    block = synthetic_block(letter)
    shapes, skipped = fit_tile_model.shapes_of(block)
    assert len(shapes) == len(SHAPES) and not skipped
    assert fit_tile_model.regret(letter, shapes) == pytest.approx(0.0, abs=1e-12)
    # spoil one parameter by one step of the fit's own grid: the first such step that costs something
    spoil = None
    for tile in range(ntiles):
        for name, steps in fit_tile_model.GRIDS.items():
            here = clblas_amd.tile_model_param(letter, tile, name)
            for d in steps:
                if -d not in steps:
                    continue
                clblas_amd.tile_model_param(letter, tile, name, here + d)
                r = fit_tile_model.regret(letter, shapes)
                clblas_amd.tile_model_param(letter, tile, name, here)
                if r > 0.005 and spoil is None:
                    spoil = (tile, name, here + d, r)
    assert spoil is not None, "no single grid step changes a pick on these shapes"
    tile, name, value, spoiled = spoil
    clblas_amd.tile_model_param(letter, tile, name, value)
    assert fit_tile_model.regret(letter, shapes) == pytest.approx(spoiled)
    fit_tile_model.fit(letter, shapes, ntiles)
    assert fit_tile_model.regret(letter, shapes) == pytest.approx(0.0, abs=1e-12)


def test_main_prints_a_report(tmp_path, capsys, restore_params):
    path = tmp_path / "tilemodel.json"
    path.write_text(json.dumps({"extra": {"tile_model": {"sgemm": synthetic_block("s"), "dgemm": synthetic_block("d")}}}))
    fit_tile_model.main(str(path))
    out = capsys.readouterr().out
    assert "== sgemm: %d shapes" % len(SHAPES) in out and "== dgemm" in out
    assert "regret 0.0000 -> 0.0000" in out


@pytest.mark.parametrize("letter", ["s", "d", "c", "z"])
def test_small_products_take_the_small_tiles_and_deep_or_large_ones_do_not(letter):
    """The choice model is a host function: a product of a few hundred 64x64 tiles goes to a 64x32 / 32x32 tile
    in one K range, the same C over a deep K to the K-split 64x64 tile, a large product to a large tile; and the
    last entry of every table is the 64x64 tile that takes the K ranges."""
    q = clblas_amd.tile_model_query(letter, 512, 512, 512)
    tiles = q["tiles"]
    assert tiles[-1].startswith("64x64x") and len(tiles) >= 4
    small = [i for i, t in enumerate(tiles) if t.startswith("64x32x") or t.startswith("32x32x")]
    assert len(small) == 2 and max(small) < len(tiles) - 1
    assert q["tile"] in small and q["splits"] == 1
    for sh in ((448, 448, 448), (800, 600, 400), (512, 1024, 512)):
        q = clblas_amd.tile_model_query(letter, *sh)
        assert q["tile"] in small and q["splits"] == 1, (sh, q)
    q = clblas_amd.tile_model_query(letter, 256, 256, 8192)       # deep K: ranges of the 64x64 tile (or a larger one)
    assert q["tile"] not in small and q["splits"] > 1, q
    q = clblas_amd.tile_model_query(letter, 8192, 8192, 8192)
    assert q["tile"] not in small and q["splits"] == 1, q
    # 32-wide tiles are not taken where one operand is streamed from HBM and only a few columns wide
    q = clblas_amd.tile_model_query(letter, 16384, 64, 10000)
    assert not tiles[q["tile"]].startswith("32x32x"), q
