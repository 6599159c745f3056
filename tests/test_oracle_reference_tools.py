"""The reference's own test inputs and the one tool among them that carries expectations
(src/backend/tests/accum_weight_map.cpp), run against the oracle."""
import numpy as np
import pytest

import oracle_lib
import reference_tools as R


def test_mt19937_known_answers():
    """std::mt19937's 10000th output from the default seed is fixed by the C++ standard (4123659995); numpy's legacy
    generator uses the same seeding and must agree on any other seed."""
    chk = R.fixture()["mt19937_check"]
    assert int(R.Mt19937(chk["seed"]).raw(chk["index"] + 1)[-1]) == chk["value"]
    for seed in (R.SEED_RENDER, R.SEED_RASTER_BWD):
        want = np.random.RandomState(seed).randint(0, 2 ** 32, size=3000, dtype=np.uint64).astype(np.uint32)
        assert np.array_equal(R.Mt19937(seed).raw(3000), want)


def test_tool_world_ranges_and_lens_rows():
    w, _ = R.tool_world(R.SEED_RENDER)
    assert w["means"].shape == (3000, 3) and w["features_sh"].shape == (3000, 15, 3)
    assert -4 <= w["means"][:, :2].min() and w["means"][:, :2].max() <= 4
    assert -2 <= w["means"][:, 2].min() and w["means"][:, 2].max() <= 8 and w["means"][:, 2].max() > 4
    assert -5 <= w["log_scales"].min() and w["log_scales"].max() <= -1.5
    assert -3 <= w["opacity_logits"].min() and w["opacity_logits"].max() <= 5
    assert np.allclose(R.tool_lens(1, 1), 0.7 * np.array([0.05, -0.01, 0.0012, -0.002, 0, 0, 0, 0]), rtol=1e-6)
    assert not R.tool_lens(0, 0).any()


def _forward(pkg, cam, packed):
    sc, _ = R.tool_scene(pkg, R.SEED_RASTER_BWD, cam)
    n, w, h = sc.n, sc.width, sc.height
    o = oracle_lib
    full = o.projection_fwd(sc)
    p = o.pack_projection(full) if packed else full
    m = p["visible"] if packed else n
    counts = o.tile_count(m, p["aabb"], p["xy"], p["conic"], p["opac"], w, h)
    ids, flat, _ = o.tile_write(m, p["aabb"], p["sort_depth"], p["xy"], p["conic"], p["opac"], o.inclusive_sum(counts), w, h)
    nt = sc.tile_w * sc.tile_h
    sk, sv = o.sort_pairs(ids, flat, 0, 32 + o.tile_n_bits(nt))
    offs = o.tile_offsets(sk, nt)
    f = o.raster_fwd(m, p, w, h, offs, sv)
    xy = np.full((n, 2), -1e9, np.float32)
    vis = full["aabb"][:, 2] > full["aabb"][:, 0]
    xy[vis] = full["xy"][vis]
    return sc, m, p, offs, sv, f, xy


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("mode", [1, 2, 3])
def test_accum_weight_map_reaches_the_right_splats(pkg, packed, mode):
    other = {}
    for cam in (0, 1):
        other[cam] = _forward(pkg, cam, False)[6]
    for cam in (0, 1):
        sc, m, p, offs, sv, f, xy = _forward(pkg, cam, packed)
        z3, z1 = np.zeros((sc.height, sc.width, 3), np.float32), np.zeros((sc.height, sc.width), np.float32)

        def run(amap):
            g = oracle_lib.raster_bwd(m, p, sc.width, sc.height, offs, sv, f, z3, z1, z1, with_abs=False, accum_mode=mode,
                                      accum_map=amap, gaussian_ids=p["gaussian_ids"] if packed else None, n_world=sc.n)
            return R.accum_finalize(g["accum_weight"], sc.n, mode)
        R.accum_weight_map_checks(run, xy, other[1 - cam], mode, f"oracle {'packed' if packed else 'plain'} mode {mode} cam {cam}")
