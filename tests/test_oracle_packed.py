"""The packed (compacted) form of the projection outputs, restated on the oracle
(oracle_lib.pack_projection / pipeline_packed), pinned against the unpacked chain: packing only
renumbers rows, so every later result must be the unpacked one up to that renumbering, bit for bit
(the per-splat gradient sums are added in the same sorted-pair order in both)."""
import numpy as np
import pytest


@pytest.mark.parametrize("seed,camera_model", [(31, 0), (32, 3)])
def test_packed_chain_is_the_unpacked_chain_renumbered(pkg, oracle, seed, camera_model):
    sc = pkg.scenes.tiny_scene(n=900, width=96, height=64, seed=seed, camera_model=camera_model)
    sc.means[::5, 2] = -10.0 if camera_model == 0 else sc.means[::5, 2]   # cull every fifth splat (pinhole)
    if camera_model == 3:
        sc.opacity_logits[::5] = -9.0                                     # below 1/255: culled
    u = oracle.pipeline(sc)
    p = oracle.pipeline_packed(sc)
    gids = p["proj"]["gaussian_ids"]
    vis = np.nonzero(u["proj"]["aabb"][:, 2] > u["proj"]["aabb"][:, 0])[0]
    assert 0 < gids.size < sc.n
    assert np.array_equal(gids, vis) and np.all(np.diff(gids) > 0)
    assert p["proj"]["visible"] == u["proj"]["visible"]
    # mask rule of the packed kernel == keep rule of the unpacked one: culled rows carry a zero aabb
    assert not np.any(u["proj"]["aabb"][np.setdiff1d(np.arange(sc.n), gids)])
    assert np.array_equal(p["counts"], u["counts"][gids])
    assert p["pads"] == 0
    assert np.array_equal(p["sorted_ids"], u["sorted_ids"])
    assert np.array_equal(gids[p["sorted_flat"]], u["sorted_flat"])
    assert np.array_equal(p["offsets"], u["offsets"])
    for k in ["rgb", "depth", "T", "last_ids"]:
        assert np.array_equal(p["fwd"][k], u["fwd"][k]), k
    for k in ["v_xy", "v_depth", "v_conic", "v_opac", "v_rgb"]:
        assert np.array_equal(p["vscreen"][k], u["vscreen"][k][gids]), k
        assert not np.any(np.delete(u["vscreen"][k], gids, axis=0)), k
    for k in u["grads"]:
        assert np.array_equal(p["grads"][k], u["grads"][k]), k


def test_packed_all_culled(pkg, oracle):
    sc = pkg.scenes.tiny_scene(n=50, width=40, height=24, seed=1)
    sc.means[:, 2] = -10.0
    p = oracle.pipeline_packed(sc)
    assert p["proj"]["visible"] == 0 and p["isect_ids"].size == 0
    assert not np.any(p["offsets"]) and np.all(p["fwd"]["T"] == 1.0)
    assert not any(np.any(v) for v in p["grads"].values())
