"""GPU: the C++ host layer (reference-shaped launch functions + engine call order) against the
oracle, in both stage orders, and the behaviours the engine relies on."""
import dataclasses

import numpy as np
import pytest

from gpu_pipeline import world_grad_check

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def H(pkg):
    from spirula_studio_amd import host, lib
    host.load()
    return host, lib


def _check(eng, ref, sc):
    assert np.array_equal(eng.cache("sorted_ids"), ref["sorted_ids"])
    assert np.array_equal(eng.cache("sorted_flat"), ref["sorted_flat"])
    assert np.array_equal(eng.cache("offsets"), ref["offsets"])
    assert np.array_equal(eng.cache("aabb").reshape(-1, 4), ref["proj"]["aabb"])
    assert np.array_equal(eng.cache("radii"), ref["proj"]["radii"])
    rgb, depth, T = eng.render()
    assert np.abs(rgb - ref["fwd"]["rgb"]).max() <= 1e-4
    assert np.abs(T - ref["fwd"]["T"]).max() <= 1e-4
    assert np.array_equal(eng.cache("last_ids").reshape(sc.height, sc.width), ref["fwd"]["last_ids"])
    g = eng.grads()
    floors = ref.get("grad_floors")
    if floors is None:
        import oracle_lib
        floors = ref["grad_floors"] = oracle_lib.world_grad_floors(sc, ref)
    for k, v in g.items():
        world_grad_check(v, ref["grads"][k], sc.n, f"engine/{k}", elem_floor=floors[k])
    return g


@pytest.mark.parametrize("native", [False, True])
def test_engine_matches_oracle(pkg, oracle, H, native):
    host, lib = H
    sc = pkg.scenes.make_scene(1, n=30000, width=320, height=240, parity_variant=True)
    ref = oracle.pipeline(sc)
    eng = host.Engine(sc, fuse_tile_count=native, visible_list=native, packed_rows=native, overwrite_world_grads=native,
                      packed_vscreen=native, tile_sort=native)
    eng.forward()
    eng.backward()
    g1 = _check(eng, ref, sc)
    # a second forward+backward on the same inputs: zero-fills honoured, nothing accumulates
    eng.forward()
    eng.backward()
    g2 = _check(eng, ref, sc)
    for k in g1:
        assert np.allclose(g1[k], g2[k], rtol=2e-3, atol=1e-6)


def _check_deferred(eng, ref, sc):
    """_check for an iteration whose key arrays were sized without the count: the keys are their first n_isects entries."""
    K = ref["sorted_ids"].size
    assert eng.n_isects == K
    ids, flat = eng.cache("sorted_ids"), eng.cache("sorted_flat")
    assert ids.size == flat.size and ids.size > K
    assert np.array_equal(ids[:K], ref["sorted_ids"]) and np.array_equal(flat[:K], ref["sorted_flat"])
    assert np.array_equal(eng.cache("offsets"), ref["offsets"].ravel())
    rgb, depth, T = eng.render()
    assert np.abs(rgb - ref["fwd"]["rgb"]).max() <= 1e-4
    assert np.abs(T - ref["fwd"]["T"]).max() <= 1e-4
    assert np.array_equal(eng.cache("last_ids").reshape(sc.height, sc.width), ref["fwd"]["last_ids"])
    for k, v in eng.grads().items():
        world_grad_check(v, ref["grads"][k], sc.n, f"engine-deferred/{k}")


@pytest.mark.parametrize("packed", [False, True])
def test_engine_leaves_the_counts_on_the_device(pkg, oracle, H, packed):
    """deferred_counts: the first iteration reads its intersection count as the reference does; the following ones
    size the key arrays from the last count and wait for nothing between the projection and the compositing. Same
    keys, ranges, image and gradients; a count that outgrows the arrays makes the backward raise before any gradient
    is used, and the next iteration reads its count again."""
    host, lib = H
    sc = pkg.scenes.make_scene(1, n=30000, width=320, height=240, parity_variant=True)
    if packed:
        sc.means[::3, 2] = -10.0
    ref = oracle.pipeline_packed(sc) if packed else oracle.pipeline(sc)
    K = ref["sorted_ids"].size
    eng = host.Engine(sc, packed_projection=packed, visible_list=not packed, deferred_counts=True)
    assert eng.deferred_capacity == 0
    eng.forward(); eng.backward()                     # blocking: learns the capacity
    assert eng.n_isects == K and eng.cache("sorted_ids").size == K
    assert eng.deferred_capacity == K + K // 16 + 65536
    for _ in range(2):                                # deferred
        eng.forward(); eng.backward()
        if packed:
            assert eng.n_isects == K and np.array_equal(eng.cache("sorted_ids")[:K], ref["sorted_ids"])
            rgb, _, T = eng.render()
            assert np.abs(rgb - ref["fwd"]["rgb"]).max() <= 1e-4
            for k, v in eng.grads().items():
                world_grad_check(v, ref["grads"][k], sc.n, f"engine-deferred-packed/{k}")
        else:
            _check_deferred(eng, ref, sc)
        assert eng.cache("sorted_ids").size == K + K // 16 + 65536
    # arrays too small for the count: the forward still runs (on the keys that fit), the backward refuses
    eng.set_deferred_counts(True, capacity=K // 2)
    eng.forward()
    with pytest.raises(lib.SsrError, match="did not fit"):
        eng.backward()
    assert eng.deferred_capacity == 0
    eng.forward(); eng.backward()                     # reads its count again
    assert eng.n_isects == K and eng.cache("sorted_ids").size == K
    for k, v in eng.grads().items():
        world_grad_check(v, ref["grads"][k], sc.n, f"engine-after-overflow/{k}")
    # the count query itself reports the overflow
    eng.set_deferred_counts(True, capacity=K - 1)
    eng.forward()
    with pytest.raises(lib.SsrError, match="did not fit"):
        eng.n_isects
    eng.set_deferred_counts(False, 0)


def test_engine_fused_step_refuses_an_intersection_that_did_not_fit(pkg, oracle, H):
    """With the counts left on the device, the fused optimizer checks them before it steps: no parameter moves on
    gradients that miss fragments, and the repeated iteration takes the step the blocking engine takes."""
    host, lib = H
    sc = pkg.scenes.make_scene(1, n=20000, width=320, height=240, parity_variant=True)
    h = dict(lr_means=1.6e-4, lr_quats=1e-3, lr_scales=5e-3, lr_opacs=5e-2, lr_features_dc=2.5e-3, lr_features_sh=1.25e-4)
    plain = host.Engine(sc)
    plain.forward(); plain.backward_fused_optimizer(h, 1)
    want = plain.params()
    K = plain.n_isects
    eng = host.Engine(sc, deferred_counts=True)
    before = eng.params()
    eng.set_deferred_counts(True, capacity=K // 3)
    eng.forward()
    with pytest.raises(lib.SsrError, match="did not fit"):
        eng.backward_fused_optimizer(h, 1)
    now = eng.params()
    for k in oracle.WORLD_KEYS:
        assert np.array_equal(now[k], before[k]), k
    eng.set_deferred_counts(True, capacity=K + 1000)   # fits: nothing is read back before the step
    eng.forward(); eng.backward_fused_optimizer(h, 1)
    got = eng.params()
    for k in oracle.WORLD_KEYS:
        assert np.allclose(got[k], want[k], rtol=1e-4, atol=1e-6), k
    eng.set_deferred_counts(False, 0)


def test_engine_quantized_and_equirect(pkg, oracle, H):
    host, lib = H
    for cfg, kw in [(3, dict(n=20000, width=320, height=192)), (5, dict(n=30000, width=512, height=256))]:
        sc = pkg.scenes.make_scene(cfg, **kw)
        ref = oracle.pipeline(sc)
        eng = host.Engine(sc)
        eng.forward()
        eng.backward()
        _check(eng, ref, sc)
    sc = pkg.scenes.make_scene(3, n=20000, width=320, height=192, sh_codec=0)
    pkg.scenes.apply_sh_codec(sc, 1, bounds_stride=256)
    ref = oracle.pipeline(sc)
    eng = host.Engine(sc)
    eng.forward()
    eng.backward()
    _check(eng, ref, sc)


def test_engine_wide_lens_cameras(pkg, oracle, H):
    """The engine on a fisheye with a thin-prism lens and on a pinhole with the rational model: camera model
    and distortion arrive as the reference's strings plus a [1, 8] coefficient row."""
    host, lib = H
    S = pkg.scenes
    for model, tier in [(S.CAM_FISHEYE, S.LENS_THIN_PRISM), (S.CAM_EQUISOLID, S.LENS_NONE), (S.CAM_PINHOLE, S.LENS_RATIONAL)]:
        sc = S.tiny_scene(n=3000, width=256, height=192, seed=51, camera_model=model)
        if model == S.CAM_PINHOLE:
            sc.intrins = np.array([150.0, 155.0, 128.0, 96.0], np.float32)
            sc.viewmat[2, 3] = 2.6
        sc = S.with_lens(sc, tier)
        ref = oracle.pipeline(sc)
        assert ref["proj"]["visible"] > 100
        eng = host.Engine(sc)
        eng.forward()
        eng.backward()
        _check(eng, ref, sc)


@pytest.mark.parametrize("packed", [False, True])
def test_engine_mip_primitive(pkg, oracle, H, packed):
    """forward_3dgs("mip"): the antialiased variant through the engine, the backward, and two fused optimizer
    steps (the reference instantiates the same functions with antialiased = true)."""
    host, lib = H
    S = pkg.scenes
    sc = S.tiny_scene(n=3000, width=256, height=192, seed=59)
    sc.log_scales -= 2.0
    sc.antialiased = True
    ref = oracle.pipeline_packed(sc) if packed else oracle.pipeline(sc)
    plain = oracle.pipeline(dataclasses.replace(sc, antialiased=False), backward=False)
    assert np.abs(plain["fwd"]["rgb"] - ref["fwd"]["rgb"]).max() > 0.02         # a different image than "3dgs"
    eng = host.Engine(sc, packed_projection=packed)
    eng.forward()
    eng.backward()
    _check(eng, ref, sc)
    h = dict(lr_means=1.6e-4, lr_quats=1e-3, lr_scales=5e-3, lr_opacs=5e-2, lr_features_dc=2.5e-3, lr_features_sh=1.25e-4,
             max_gauss_ratio=6.0, scale_regularization_weight=0.01, mcmc_opacity_reg_weight=0.01, mcmc_scale_reg_weight=0.01,
             quat_norm_reg_weight=0.02, sh_reg_weight=0.05)
    eng2 = host.Engine(sc, packed_projection=packed)
    eng2.forward()
    eng2.backward_fused_optimizer(h, 1)
    P = {k: np.ascontiguousarray(getattr(sc, k), np.float32).copy() for k in oracle.WORLD_KEYS}
    g1 = {k: np.zeros_like(v) for k, v in P.items()}
    g2 = {k: np.zeros_like(v) for k, v in P.items()}
    r = oracle.pipeline(sc)
    oracle.fused_projection_bwd_optimizer(sc, r["proj"]["aabb"], r["vscreen"], P, g1, g2, h, step=1)
    got = eng2.params()
    lrs = dict(means="lr_means", quats="lr_quats", log_scales="lr_scales", opacity_logits="lr_opacs",
               features_dc="lr_features_dc", features_sh="lr_features_sh")
    for k in oracle.WORLD_KEYS:      # first Adam step: +-lr per element, sign decided by the gradient
        far = np.abs(got[k].astype(np.float64) - P[k]) > 0.05 * h[lrs[k]]
        assert far.mean() < 5e-3, (k, float(far.mean()))


@pytest.mark.parametrize("packed", [False, True])
def test_engine_camera_pose_gradient(pkg, oracle, H, packed):
    """projection_3dgs_backward with v_viewmats through the adapter (the reference's engine passes null; its
    launch function and parity tool do not): dL/dR and dL/dt summed over the visible splats, on a rotated
    camera with a lens, next to unchanged world gradients."""
    host, lib = H
    S = pkg.scenes
    sc = S.tiny_scene(n=3000, width=256, height=192, seed=53)
    sc.intrins = np.array([150.0, 155.0, 128.0, 96.0], np.float32)
    c, s_ = np.cos(0.2), np.sin(0.2)
    sc.viewmat = np.array([[c, 0, s_, 0.3], [0, 1, 0, -0.2], [-s_, 0, c, 3.0], [0, 0, 0, 1]], np.float32)
    sc = S.with_lens(sc, S.LENS_OPENCV)
    ref = oracle.pipeline(sc)
    assert ref["proj"]["visible"] > 100
    want = oracle.projection_bwd(sc, ref["proj"]["aabb"], ref["vscreen"], pose=True)["v_viewmat"].astype(np.float64)
    eng = host.Engine(sc, packed_projection=packed)
    eng.forward()
    got = eng.backward_with_pose_grad().astype(np.float64)
    _check(eng, ref, sc)
    assert not np.any(got[3]) and np.abs(want[:3]).min() > 0
    print(f"  pose gradient: max err / max {np.abs(got - want).max() / np.abs(want).max():.3e}", flush=True)
    assert np.abs(got - want).max() <= 1e-3 * np.abs(want).max(), (got, want)
    # accumulated into, not overwritten: a second backward on a fresh buffer gives the same sums again
    again = eng.backward_with_pose_grad().astype(np.float64)
    assert np.abs(again - got).max() <= 1e-4 * np.abs(want).max()


def test_engine_overwrite_without_list(pkg, oracle, H):
    host, lib = H
    sc = pkg.scenes.make_scene(4, n=40000, width=480, height=270)
    ref = oracle.pipeline(sc)
    eng = host.Engine(sc, fuse_tile_count=True, visible_list=False, packed_rows=False, overwrite_world_grads=True)
    eng.forward()
    eng.backward()
    _check(eng, ref, sc)


def test_lazy_gradient_zeroing_follows_the_camera(pkg, oracle, H):
    """With few visible splats only the rows written by the previous backward are re-zeroed; after a
    camera move the rows of splats that left the view must read zero again."""
    host, lib = H
    import ctypes as C
    sc = pkg.scenes.make_scene(4, n=60000, width=480, height=270)
    eng = host.Engine(sc)
    for _ in range(2):
        eng.forward()
        eng.backward()
    ref = oracle.pipeline(sc)
    assert ref["proj"]["visible"] * 2 < sc.n
    _check(eng, ref, sc)
    # look the other way: a different set of splats is visible
    sc.viewmat = np.array([[-1, 0, 0, 0], [0, 1, 0, 0], [0, 0, -1, 0.5], [0, 0, 0, 1]], np.float32)
    vm, it = np.ascontiguousarray(sc.viewmat), np.ascontiguousarray(sc.intrins, np.float32)
    host.check(eng.h.ssrh_set_camera_params(sc.width, sc.height, b"PINHOLE", b"NONE", vm.ctypes.data, it.ctypes.data, None, 1))
    eng.forward()
    eng.backward()
    ref2 = oracle.pipeline(sc)
    vis1 = ref["proj"]["aabb"][:, 2] > ref["proj"]["aabb"][:, 0]
    vis2 = ref2["proj"]["aabb"][:, 2] > ref2["proj"]["aabb"][:, 0]
    assert (vis1 & ~vis2).sum() > 1000
    g = _check(eng, ref2, sc)
    assert not np.any(g["v_sh"][~vis2]) and not np.any(g["v_means"][~vis2])


def _check_packed(eng, ref, sc):
    q = ref["proj"]
    m = q["visible"]
    assert np.array_equal(eng.cache("gaussian_ids"), q["gaussian_ids"])
    assert eng.cache("camera_ids").size == m and not np.any(eng.cache("camera_ids"))
    assert np.array_equal(eng.cache("aabb").reshape(-1, 4), q["aabb"])
    for k in ["xy", "depth", "conic", "opac", "rgb"]:
        assert np.array_equal(eng.cache(k).view(np.uint32), q[k].reshape(-1).view(np.uint32)), k
    assert np.array_equal(eng.cache("radii"), q["radii"])
    assert np.array_equal(eng.cache("sorted_ids"), ref["sorted_ids"])
    assert np.array_equal(eng.cache("sorted_flat"), ref["sorted_flat"])
    assert np.array_equal(eng.cache("offsets"), ref["offsets"])
    rgb, depth, T = eng.render()
    assert np.abs(rgb - ref["fwd"]["rgb"]).max() <= 1e-4
    assert np.abs(T - ref["fwd"]["T"]).max() <= 1e-4
    assert np.array_equal(eng.cache("last_ids").reshape(sc.height, sc.width), ref["fwd"]["last_ids"])
    assert eng.cache("v_xy").size == 2 * m
    g = eng.grads()
    for k, v in g.items():
        world_grad_check(v, ref["grads"][k], sc.n, f"engine/{k}")
    return g


@pytest.mark.parametrize("native", [False, True])
def test_engine_packed_projection(pkg, oracle, H, native):
    """forward_3dgs(packed=true): the reference's product default (src/config/TrainConfig.h:285)."""
    host, lib = H
    sc = pkg.scenes.make_scene(1, n=30000, width=320, height=240, parity_variant=True)
    sc.means[::3, 2] = -10.0   # a third of the splats behind the camera
    ref = oracle.pipeline_packed(sc)
    eng = host.Engine(sc, fuse_tile_count=native, visible_list=False, packed_rows=native, overwrite_world_grads=native,
                      packed_projection=True)
    for _ in range(2):   # twice: zero-fills honoured, nothing accumulates
        eng.forward()
        eng.backward()
        _check_packed(eng, ref, sc)


@pytest.mark.parametrize("world_rows", [False, True], ids=["gathered", "world-rows"])
def test_engine_packed_follows_the_camera_and_handles_nothing_visible(pkg, oracle, H, world_rows):
    """world-rows: the packed projection keeps the visible splats' parameters (64 bytes each, in four planes) for the projection
    backward (Options::packed_world_rows); the rows must follow every new projection."""
    host, lib = H
    sc = pkg.scenes.make_scene(4, n=60000, width=480, height=270)
    eng = host.Engine(sc, packed_projection=True, packed_world_rows=world_rows)
    for _ in range(2):
        eng.forward()
        eng.backward()
    ref = oracle.pipeline_packed(sc)
    assert 0 < ref["proj"]["visible"] * 2 < sc.n
    _check_packed(eng, ref, sc)

    def look(viewmat):
        sc.viewmat = np.asarray(viewmat, np.float32)
        vm, it = np.ascontiguousarray(sc.viewmat), np.ascontiguousarray(sc.intrins, np.float32)
        host.check(eng.h.ssrh_set_camera_params(sc.width, sc.height, b"PINHOLE", b"NONE", vm.ctypes.data, it.ctypes.data, None, 1))
        eng.forward()
        eng.backward()
        r = oracle.pipeline_packed(sc)
        g = _check_packed(eng, r, sc)
        vis = np.zeros(sc.n, bool)
        vis[r["proj"]["gaussian_ids"]] = True
        assert not np.any(g["v_sh"][~vis]) and not np.any(g["v_means"][~vis])
        return r

    look([[-1, 0, 0, 0], [0, 1, 0, 0], [0, 0, -1, 0.5], [0, 0, 0, 1]])       # the other way
    r = look([[1, 0, 0, 0], [0, 1, 0, 0], [0, 0, 1, -1000.0], [0, 0, 0, 1]])   # everything behind the camera
    assert r["proj"]["visible"] == 0
    rgb, depth, T = eng.render()
    assert np.all(T == 1.0) and not np.any(rgb)
    look([[1, 0, 0, 0], [0, 1, 0, 0], [0, 0, 1, 0], [0, 0, 0, 1]])             # and back


@pytest.mark.parametrize("packed", [False, True])
def test_engine_fused_optimizer_scale_agnostic_means(pkg, oracle, H, packed):
    """One step with OptimConfig::use_scale_agnostic_mean (the reference's default): the means move by
    lr * (covariance-weighted gradient) / (gradient x 0.6 radii). A component whose own gradient is almost
    zero takes a huge, rounding-dependent step in the reference too, so the steps are compared relatively
    and a small fraction of such components is allowed to differ."""
    host, lib = H
    sc = pkg.scenes.make_scene(1, n=20000, width=320, height=240, parity_variant=True)
    if packed:
        sc.means[::3, 2] = -10.0
    h = dict(lr_means=1.6e-4, lr_quats=1e-3, lr_scales=5e-3, lr_opacs=5e-2, lr_features_dc=2.5e-3, lr_features_sh=1.25e-4,
             max_gauss_ratio=6.0, scale_regularization_weight=0.01, mcmc_opacity_reg_weight=0.01, mcmc_scale_reg_weight=0.01,
             quat_norm_reg_weight=0.02, sh_reg_weight=0.05)
    eng = host.Engine(sc, packed_projection=packed)
    eng.forward()
    eng.backward_fused_optimizer(h, 1, scale_agnostic_mean=True)
    got = eng.params()
    P = {k: np.ascontiguousarray(getattr(sc, k), np.float32).copy() for k in oracle.WORLD_KEYS}
    g1 = {k: np.zeros_like(v) for k, v in P.items()}
    g2 = {k: np.zeros_like(v) for k, v in P.items()}
    r = oracle.pipeline(sc, backward=True)
    oracle.fused_projection_bwd_optimizer(sc, r["proj"]["aabb"], r["vscreen"], P, g1, g2, h, step=1, radii=r["proj"]["radii"])
    want = P["means"].astype(np.float64) - sc.means
    step = got["means"].astype(np.float64) - sc.means
    vis = r["proj"]["aabb"][:, 2] > r["proj"]["aabb"][:, 0]
    assert not np.any(step[~vis]) and not np.any(want[~vis])          # no gradient, no step
    assert np.abs(want[vis]).max() > 10 * h["lr_means"]                # not the plain Adam step
    far = np.abs(step - want) > 0.05 * np.abs(want) + 1e-7
    assert far[vis].mean() < 0.01, float(far[vis].mean())
    for k in ["quats", "log_scales", "opacity_logits", "features_dc"]:  # the other parameters take the plain step
        d = np.abs(got[k].astype(np.float64) - P[k])
        assert (d > 0.05 * 5e-2).mean() < 2e-3, k


@pytest.mark.parametrize("schedule", [0, 1])
def test_engine_backward_schedule_forced(pkg, oracle, H, schedule):
    """The engine with either cut of the compositing backward forced (the adapter otherwise picks one from the tiles
    per visible splat): same keys, image and gradients, and the loss-map weight sums of the fused step."""
    host, lib = H
    sc = pkg.scenes.make_scene(1, n=30000, width=320, height=240, parity_variant=True)
    ref = oracle.pipeline(sc)
    eng = host.Engine(sc, backward_schedule=schedule)
    for _ in range(2):
        eng.forward()
        eng.backward()
        _check(eng, ref, sc)
    amap = np.random.default_rng(6).uniform(0, 1, (sc.height, sc.width)).astype(np.float32)
    d_map = lib.DeviceArray.from_host(amap)
    eng.set_loss_map(d_map.ptr, 3)
    eng.forward()
    eng.backward_fused_optimizer(dict(lr_means=1.6e-4, lr_quats=1e-3, lr_scales=5e-3, lr_opacs=5e-2, lr_features_dc=2.5e-3,
                                      lr_features_sh=1.25e-4), 1)
    aw = eng.cache("accum_weight")
    r = oracle.pipeline(sc, backward=True, variant=dict(dist_type=0, median=False, accum_mode=3, accum_map=amap))
    want = r["vscreen"]["accum_weight"]
    assert np.allclose(aw[:want.size], want, rtol=1e-3, atol=1e-6) and (aw[:sc.n] > 0).sum() > 1000
    eng.set_loss_map(None, 0)


@pytest.mark.parametrize("packed,accum_mode", [(False, 3), (True, 3), (False, 1), (True, 2)])
def test_engine_fused_step_accumulates_the_loss_map(pkg, oracle, H, packed, accum_mode):
    """The training step of the reference accumulates its loss map per splat in the same compositing backward that
    feeds the fused optimizer (EngineTrainStep.cpp:256-258): with a map set, the engine's fused step leaves the
    oracle's accumulated weights, and the parameters take exactly the step they take without a map."""
    host, lib = H
    sc = pkg.scenes.make_scene(1, n=20000, width=320, height=240, parity_variant=True)
    if packed:
        sc.means[::3, 2] = -10.0
    h = dict(lr_means=1.6e-4, lr_quats=1e-3, lr_scales=5e-3, lr_opacs=5e-2, lr_features_dc=2.5e-3, lr_features_sh=1.25e-4)
    amap = np.random.default_rng(5).uniform(0, 1, (sc.height, sc.width)).astype(np.float32)
    d_map = lib.DeviceArray.from_host(amap)
    kw = dict(fuse_tile_count=True, visible_list=not packed, packed_rows=True, overwrite_world_grads=True,
              packed_projection=packed, packed_vscreen=True, tile_sort=True)
    eng = host.Engine(sc, **kw)
    eng.set_loss_map(d_map.ptr, accum_mode)
    eng.forward()
    eng.backward_fused_optimizer(h, 1)
    aw = eng.cache("accum_weight")
    got = eng.params()
    r = oracle.pipeline(sc, backward=True, variant=dict(dist_type=0, median=False, accum_mode=accum_mode, accum_map=amap))
    ref = r["vscreen"]["accum_weight"]
    assert np.allclose(aw[:ref.size], ref, rtol=1e-3, atol=1e-6) and (aw[:sc.n] > 0).sum() > 1000
    eng.set_loss_map(None, 0)
    plain = host.Engine(sc, **kw)
    plain.forward()
    plain.backward_fused_optimizer(h, 1)
    base = plain.params()
    for k in oracle.WORLD_KEYS:   # the map adds outputs, it changes no gradient (summation order aside)
        assert np.allclose(got[k], base[k], rtol=1e-4, atol=1e-6), k


@pytest.mark.parametrize("packed,non_sh_bits", [(False, 32), (True, 32), (False, 16), (True, 16)])
def test_engine_fused_optimizer_quantization_level_1(pkg, oracle, H, packed, non_sh_bits):
    """Training steps at OptimConfig::quantization_level 1 (the reference's default): the engine keeps the SH
    coefficients as 16-bit codes that the forward reads and the fused optimizer rewrites in place, and their Adam
    moments as 8-bit cells; against the oracle running the same loop on its own copy. non_sh_bits 16: the moments
    of the other five tensors as 16-bit cells as well (OptimConfig::non_sh_optim_bits, what the reference's trainer
    sets at this level)."""
    host, lib = H
    S = pkg.scenes
    sc = S.make_scene(1, n=20000, width=320, height=240, parity_variant=True, sh_codec=0)
    if packed:
        sc.means[::3, 2] = -10.0
    S.apply_sh_codec(sc, 2, bounds_stride=256 * 45)
    h = dict(lr_means=1.6e-4, lr_quats=1e-3, lr_scales=5e-3, lr_opacs=5e-2, lr_features_dc=2.5e-3, lr_features_sh=2.5e-3,
             max_gauss_ratio=6.0, scale_regularization_weight=0.01, mcmc_opacity_reg_weight=0.01, mcmc_scale_reg_weight=0.01,
             quat_norm_reg_weight=0.02, sh_reg_weight=0.05)
    n, R = sc.n, 45
    nb = (n + 255) // 256
    eng = host.Engine(sc, packed_projection=packed)
    import copy
    ref = copy.deepcopy(sc)        # keeps the 16-bit codec: the oracle's forward decodes ref.sh_packed / ref.sh_bounds
    q = dict(state_packed=np.zeros(n * R, np.uint16), state_bounds=np.zeros((nb, 4), np.float32),
             value_packed=np.ascontiguousarray(sc.sh_packed).view(np.uint16).copy(),
             value_bounds=np.ascontiguousarray(sc.sh_bounds, np.float32).reshape(nb, 2).copy(), num_sh_buffer=15)
    P = {k: np.ascontiguousarray(getattr(sc, k), np.float32).copy() for k in oracle.WORLD_KEYS[:5]}
    g1 = {k: np.zeros_like(v) for k, v in P.items()}
    g2 = {k: np.zeros_like(v) for k, v in P.items()}
    start = oracle.decode_sh_values(q, n)
    ns = None
    if non_sh_bits == 16:
        ns, g1, g2 = oracle.zero_non_sh_state(n), None, None
    for step in (1, 2, 3):
        eng.forward()
        eng.backward_fused_optimizer(h, step, quantization_level=1, non_sh_optim_bits=non_sh_bits)
        for k in P:
            setattr(ref, k, P[k])
        ref.sh_packed, ref.sh_bounds = q["value_packed"].copy(), q["value_bounds"].copy()
        r = oracle.pipeline(ref, backward=True)
        oracle.fused_projection_bwd_optimizer_q(ref, r["proj"]["aabb"], r["vscreen"], P, q, g1, g2, h, step=step, non_sh=ns)
        if ns is not None:
            e1, e2 = oracle.decode_non_sh_state(eng.non_sh_quant_state(), n)
            o1, o2 = oracle.decode_non_sh_state(ns, n)
            for k in oracle.NON_SH_KEYS:
                a, b = e1[k].reshape(n, -1).astype(np.float64), o1[k].reshape(n, -1).astype(np.float64)
                assert np.isfinite(a).all() and np.abs(b).max() > 0
                scale = np.abs(b).max(axis=1, keepdims=True) + 1e-12
                assert (np.abs(a - b) > 0.05 * scale + 1e-9).mean() < 0.02, (k, step)
                a, b = e2[k].reshape(n, -1).astype(np.float64), o2[k].reshape(n, -1).astype(np.float64)
                assert (np.abs(a - b) > 0.05 * b + 1e-14).mean() < 0.02, (k, step)
        eq = eng.sh_quant_state()
        got, want = oracle.decode_sh_values(eq, n), oracle.decode_sh_values(q, n)
        far = np.abs(got - want) > 0.05 * h["lr_features_sh"] + 1e-6
        assert far.mean() < 5e-3, (step, float(far.mean()))
        assert np.abs(got - want).max() <= 2.5 * step * h["lr_features_sh"] + 1e-5
        assert np.allclose(eq["value_bounds"], q["value_bounds"], atol=2.5 * step * h["lr_features_sh"])
        m1, m2 = oracle.decode_sh_moments(eq, n)
        w1, w2 = oracle.decode_sh_moments(q, n)
        assert np.isfinite(m1).all() and np.isfinite(m2).all()
        scale = np.abs(w1).max(axis=1, keepdims=True) + 1e-12
        assert ((np.abs(m1 - w1) > 0.05 * scale + 1e-9).mean()) < 0.02, step
    assert np.abs(want - start).max() > 2 * h["lr_features_sh"]          # the coefficients moved, step after step
    eng.forward()                                                      # and the forward renders the updated codes
    for k in P:
        setattr(ref, k, P[k])
    ref.sh_packed, ref.sh_bounds = q["value_packed"].copy(), q["value_bounds"].copy()
    r = oracle.pipeline(ref, backward=False)
    rgb, depth, T = eng.render()
    assert np.abs(rgb - r["fwd"]["rgb"]).max() < 0.05      # three sign-sensitive first Adam steps apart
    # exactly what the engine now holds, rendered by the oracle: the forward reads the rewritten codes and bounds
    got_p, got_q = eng.params(), eng.sh_quant_state()
    for k in P:
        setattr(ref, k, got_p[k])
    ref.sh_packed, ref.sh_bounds = got_q["value_packed"], got_q["value_bounds"]
    r = oracle.pipeline(ref, backward=False)
    assert np.abs(rgb - r["fwd"]["rgb"]).max() < 1e-4


def test_engine_packed_fused_optimizer_with_nothing_visible(pkg, oracle, H):
    """No packed rows at all: no projection gradient, but every splat still decays its moments and takes
    the regularizer step (the reference's kernel runs over all N splats whatever is visible)."""
    host, lib = H
    sc = pkg.scenes.tiny_scene(n=2000, width=96, height=64, seed=71)
    sc.viewmat = np.array([[1, 0, 0, 0], [0, 1, 0, 0], [0, 0, 1, -1000.0], [0, 0, 0, 1]], np.float32)   # all behind
    eng = host.Engine(sc, packed_projection=True)
    eng.forward()
    assert eng.n_isects == 0
    h = dict(lr_means=1.6e-4, lr_quats=1e-3, lr_scales=5e-3, lr_opacs=5e-2, lr_features_dc=2.5e-3, lr_features_sh=1.25e-4,
             max_gauss_ratio=6.0, scale_regularization_weight=0.01, mcmc_opacity_reg_weight=0.01, mcmc_scale_reg_weight=0.01,
             quat_norm_reg_weight=0.02, sh_reg_weight=0.05)
    before = eng.params()
    eng.backward_fused_optimizer(h, 1)
    after = eng.params()
    P = {k: np.ascontiguousarray(before[k], np.float32).copy() for k in oracle.WORLD_KEYS}
    g1 = {k: np.zeros_like(v) for k, v in P.items()}
    g2 = {k: np.zeros_like(v) for k, v in P.items()}
    vs = dict(v_xy=np.zeros((sc.n, 2), np.float32), v_depth=np.zeros(sc.n, np.float32), v_conic=np.zeros((sc.n, 3), np.float32),
              v_opac=np.zeros(sc.n, np.float32), v_rgb=np.zeros((sc.n, 3), np.float32))
    oracle.fused_projection_bwd_optimizer(sc, np.zeros((sc.n, 4), np.float32), vs, P, g1, g2, h, step=1)
    assert np.array_equal(after["means"], before["means"])    # no gradient reaches the means
    assert np.abs(after["opacity_logits"] - before["opacity_logits"]).max() > 0.01    # the opacity regularizer moved it
    for k in oracle.WORLD_KEYS:
        assert np.abs(after[k].astype(np.float64) - P[k]).max() <= 0.05 * 5e-2, k


def test_engine_tile_mask_is_one_shot(pkg, oracle, H):
    host, lib = H
    sc = pkg.scenes.make_scene(1, n=20000, width=320, height=240, parity_variant=True)
    mask = np.zeros((240, 320), np.uint8)
    mask[60:150, 100:260] = 1
    live = oracle.compute_tile_active(mask, sc.width, sc.height)
    assert 0 < live.sum() < live.size
    for packed in (False, True):
        eng = host.Engine(sc, packed_projection=packed)
        eng.set_tile_mask(mask)
        eng.forward()
        eng.backward()
        if packed:
            _check_packed(eng, oracle.pipeline_packed(sc, tile_active=live), sc)
        else:
            _check(eng, oracle.pipeline(sc, tile_active=live), sc)
        eng.forward()          # the map is not inherited by the next forward
        eng.backward()
        if packed:
            _check_packed(eng, oracle.pipeline_packed(sc), sc)
        else:
            _check(eng, oracle.pipeline(sc), sc)


@pytest.mark.parametrize("packed", [False, True])
def test_engine_fused_optimizer_training_steps(pkg, oracle, H, packed):
    """Three training steps with the projection backward folded into Adam, against the oracle running
    the same loop (forward, compositing backward, fused optimizer) on its own copy of the parameters;
    also on the packed projection outputs (forward_3dgs(packed=true), the reference's training default),
    where the splats behind the camera have no row and only decay their moments."""
    import copy
    host, lib = H
    sc = pkg.scenes.make_scene(1, n=20000, width=320, height=240, parity_variant=True)
    if packed:
        sc.means[::3, 2] = -10.0
    ref_sc = copy.deepcopy(sc)
    h = dict(lr_means=1.6e-4, lr_quats=1e-3, lr_scales=5e-3, lr_opacs=5e-2, lr_features_dc=2.5e-3,
             lr_features_sh=1.25e-4, max_gauss_ratio=6.0, scale_regularization_weight=0.01,
             mcmc_opacity_reg_weight=0.01, mcmc_scale_reg_weight=0.01, quat_norm_reg_weight=0.02, sh_reg_weight=0.05)
    lrs = dict(means="lr_means", quats="lr_quats", log_scales="lr_scales", opacity_logits="lr_opacs",
               features_dc="lr_features_dc", features_sh="lr_features_sh")
    if packed:
        h.update(erank_reg_weight=0.05, erank_reg_weight_s3=0.01)
    eng = host.Engine(sc, packed_projection=packed)
    P = {k: np.ascontiguousarray(getattr(ref_sc, k), np.float32).copy() for k in oracle.WORLD_KEYS}
    g1 = {k: np.zeros_like(v) for k, v in P.items()}
    g2 = {k: np.zeros_like(v) for k, v in P.items()}
    for step in (1, 2, 3):
        eng.forward()
        eng.backward_fused_optimizer(h, step)
        for k in oracle.WORLD_KEYS:
            setattr(ref_sc, k, P[k])
        r = oracle.pipeline(ref_sc, backward=True)
        oracle.fused_projection_bwd_optimizer(ref_sc, r["proj"]["aabb"], r["vscreen"], P, g1, g2, h, step=step)
        got = eng.params()
        for k in oracle.WORLD_KEYS:
            d = np.abs(got[k].astype(np.float64) - P[k])
            lr = h[lrs[k]]
            # first steps move every parameter by about lr * sign(gradient): a gradient that rounds to the
            # other side of zero moves it the other way, so a few elements may differ by a step or two
            far = d > 0.05 * lr + 1e-6
            assert far.mean() < 2e-3, (step, k, float(far.mean()))
            assert d.max() <= 2.5 * step * lr + 1e-6, (step, k, float(d.max()))
    # the render of the updated model still matches
    eng.forward()
    for k in oracle.WORLD_KEYS:
        setattr(ref_sc, k, P[k])
    r = oracle.pipeline(ref_sc, backward=False)
    rgb, depth, T = eng.render()
    assert np.abs(rgb - r["fwd"]["rgb"]).max() < 0.02


@pytest.mark.parametrize("packed", [False, True])
def test_engine_compositing_variants(pkg, oracle, H, packed):
    """forward_3dgs(output_median, dist_type) and a backward fed the distortion / median cotangents and
    a pixel weight map to accumulate per splat (indexed by world row also in packed mode)."""
    host, lib = H
    sc = pkg.scenes.make_scene(1, n=20000, width=240, height=160, parity_variant=True)
    sc.means[::3, 2] = -10.0
    rng = np.random.default_rng(5)
    h, w = sc.height, sc.width
    cot = dict(v_dist_rgb=rng.uniform(-1, 1, (h, w, 3)).astype(np.float32), v_dist_depth=rng.uniform(-1, 1, (h, w)).astype(np.float32),
               v_median=rng.uniform(-1, 1, (h, w)).astype(np.float32), accum_map=rng.uniform(0, 1, (h, w)).astype(np.float32))
    va = dict(dist_type=2, median=False, accum_mode=3, **cot)
    eng = host.Engine(sc, packed_projection=packed)
    eng.set_variants(dist_type=2, median=True)
    eng.forward()
    eng.backward_with_variants(cot["v_dist_rgb"], cot["v_dist_depth"], None, cot["accum_map"], accum_mode=3)
    # oracle: unpacked chain; packing only renumbers rows, the accumulated weights are per world row
    r = oracle.pipeline(sc, variant=va)
    rm = oracle.pipeline(sc, backward=False, variant=dict(median=True))
    assert np.abs(eng.cache("dist_rgb").reshape(h, w, 3) - r["fwd"]["dist_rgb"]).max() <= 1e-4
    assert np.abs(eng.cache("dist_depth").reshape(h, w) - r["fwd"]["dist_depth"]).max() <= 1e-4
    med = rm["fwd"]["median"]
    assert (np.abs(eng.cache("median").reshape(h, w) - med) <= 1e-4 * np.maximum(1, np.abs(med))).all()
    rgb, depth, T = eng.render()
    assert (np.abs(depth - r["fwd"]["depth"]) <= 1e-4 * np.maximum(1, r["fwd"]["depth"])).all()
    aw = eng.cache("accum_weight")
    assert aw.size == 2 * sc.n
    assert np.allclose(aw, r["vscreen"]["accum_weight"], rtol=1e-3, atol=1e-6) and (aw[:sc.n] > 0).sum() > 100
    g = eng.grads()
    for k, v in g.items():
        world_grad_check(v, r["grads"][k], sc.n, f"engine-variants/{k}")
    # a forward with distortion needs its cotangent in the backward
    assert eng.h.ssrh_backward_from_render_grad(eng.d_vrgb.ptr, eng.d_vdepth.ptr, eng.d_vT.ptr) != 0
    assert b"distortion" in eng.h.ssrh_last_error()


def test_unsupported_variants_raise(pkg, H):
    host, lib = H
    sc = pkg.scenes.tiny_scene(n=50, width=32, height=32)
    eng = host.Engine(sc)
    h = host.load()
    assert h.ssrh_forward_3dgs(b"3dgut", 3, 0, 0, 0) != 0
    assert b"not built" in h.ssrh_last_error()
    for dist in (3, 4):   # DN, RGB_DN: the 3dgs pixel has no normal channel
        assert h.ssrh_forward_3dgs(b"3dgs", 3, 0, 0, dist) != 0
        assert b"normal" in h.ssrh_last_error()
    vm, it = np.ascontiguousarray(sc.viewmat, np.float32), np.ascontiguousarray(sc.intrins, np.float32)
    for model, lens, word in [(b"FISHEYE", b"RATIONAL", b"RATIONAL"), (b"EQUIRECTANGULAR", b"OPENCV", b"OPENCV"),
                              (b"ORTHOGRAPHIC", b"NONE", b"ORTHOGRAPHIC"), (b"PINHOLE", b"BROWN", b"BROWN")]:
        assert h.ssrh_set_camera_params(32, 32, model, lens, vm.ctypes.data, it.ctypes.data, None, 1) == 0
        assert h.ssrh_forward_3dgs(b"3dgs", 3, 0, 0, 0) != 0
        assert word in h.ssrh_last_error()


def test_runtime_contract(pkg, H):
    """The checklist of src/backend/vulkan/tests/vk_runtime_smoke.cpp:44-160."""
    host, lib = H
    L = lib.load()
    lib.check(L.ssr_init(0))
    assert L.ssr_device_malloc(0) is None
    d = L.ssr_device_malloc(1 << 20)
    assert d and L.ssr_is_device_pointer(d) == 1 and L.ssr_is_device_pointer(d + 4096) == 1
    p = L.ssr_host_malloc_pinned(4096)
    assert p and L.ssr_is_device_pointer(p) == 0            # pinned host memory is not a device pointer
    a = np.arange(1000, dtype=np.int32)
    assert L.ssr_is_device_pointer(a.ctypes.data) == 0
    # all copy kinds, including Auto routing
    lib.check(L.ssr_memcpy(d, a.ctypes.data, a.nbytes, lib.H2D, None, 0))
    d2 = L.ssr_device_malloc(a.nbytes)
    lib.check(L.ssr_memcpy(d2, d, a.nbytes, lib.AUTO, None, 0))
    b = np.zeros_like(a)
    lib.check(L.ssr_memcpy(b.ctypes.data, d2, a.nbytes, lib.AUTO, None, 0))
    assert np.array_equal(a, b)
    # memset with an unaligned byte tail
    lib.check(L.ssr_memset(d + 1, 0xAB, 1001, None, 0))
    c = np.zeros(1004, np.uint8)
    lib.check(L.ssr_memcpy(c.ctypes.data, d, 1004, lib.D2H, None, 0))
    assert c[0] == 0 and np.all(c[1:1002] == 0xAB) and c[1002] != 0xAB
    # pinned async readback fenced by an event
    ev = L.ssr_event_create()
    lib.check(L.ssr_memcpy(p, d2, 4000, lib.D2H, None, 1))
    lib.check(L.ssr_event_record(ev, None))
    lib.check(L.ssr_event_synchronize(ev))
    import ctypes as C
    assert np.array_equal(np.frombuffer((C.c_int32 * 1000).from_address(p), np.int32), a)
    # timing events
    e0, e1 = L.ssr_event_create(), L.ssr_event_create()
    lib.check(L.ssr_event_record(e0, None))
    lib.check(L.ssr_fill_u32(d, 7, (1 << 20) // 4, None))
    lib.check(L.ssr_event_record(e1, None))
    ms = C.c_float(-1)
    lib.check(L.ssr_event_elapsed_ms(e0, e1, C.byref(ms)))
    assert ms.value >= 0
    # sticky error: reported once, cleared by the read
    assert L.ssr_memcpy(None, None, 16, lib.H2D, None, 0) != 0
    assert L.ssr_last_error() != b"" and L.ssr_last_error() == b""
    for e in (ev, e0, e1):
        L.ssr_event_destroy(e)
    L.ssr_device_free(d); L.ssr_device_free(d2); L.ssr_host_free_pinned(p)


@pytest.mark.parametrize("native,deferred", [(False, False), (True, False), (True, True)])
def test_engine_two_cameras(pkg, oracle, H, native, deferred):
    """[C = 2] viewmats through the adapter (the reference's entry points take [C,4,4] cameras and render C
    images in one pass: ProjectionFwd_kernel.cuh:60-110, IntersectTile.cu:215-262, RasterizationFwd.cu grid
    {C, tile_h, tile_w}). Against the oracle run once per camera: image c's keys carry tile ids offset by
    c * tiles and row ids offset by c * N, its pixels and last ids are the single camera's, the world
    gradients and radii combine both cameras, and each camera gets its own pose gradient."""
    import copy
    host, lib = H
    S = pkg.scenes
    base = S.tiny_scene(n=3000, width=250, height=180, seed=71)   # ragged edge tiles in both directions
    cams = []
    for k, (ang, t) in enumerate([(0.2, (0.3, -0.2, 3.0)), (-0.35, (-0.4, 0.1, 3.4))]):
        c, s_ = np.cos(ang), np.sin(ang)
        vm = np.array([[c, 0, s_, t[0]], [0, 1, 0, t[1]], [-s_, 0, c, t[2]], [0, 0, 0, 1]], np.float32)
        it = np.array([150.0 + 20 * k, 155.0 - 10 * k, 125.0, 90.0 + 5 * k], np.float32)
        cams.append((vm, it))
    rng = np.random.default_rng(5)
    h, w, n = base.height, base.width, base.n
    v_rgb = rng.standard_normal((2, h, w, 3)).astype(np.float32)
    v_depth = rng.standard_normal((2, h, w)).astype(np.float32)
    v_T = rng.standard_normal((2, h, w)).astype(np.float32)
    refs, poses = [], []
    for k, (vm, it) in enumerate(cams):
        sc = copy.deepcopy(base)
        sc.viewmat, sc.intrins = vm, it
        sc.v_rgb, sc.v_depth, sc.v_T = v_rgb[k], v_depth[k], v_T[k]
        ref = oracle.pipeline(sc)
        assert ref["proj"]["visible"] > 100 and ref["sorted_ids"].size > 1000
        refs.append(ref)
        poses.append(oracle.projection_bwd(sc, ref["proj"]["aabb"], ref["vscreen"], pose=True)["v_viewmat"].astype(np.float64))
    both = copy.deepcopy(base)
    both.viewmat = np.stack([c[0] for c in cams])
    both.intrins = np.stack([c[1] for c in cams])
    both.v_rgb, both.v_depth, both.v_T = v_rgb, v_depth, v_T
    # deferred: the second pass leaves the intersection count on the device (arrays sized from the first pass)
    eng = host.Engine(both, fuse_tile_count=native, visible_list=native, packed_rows=native, overwrite_world_grads=native,
                      packed_vscreen=native, tile_sort=native, deferred_counts=deferred)
    tiles = ((w + 15) // 16) * ((h + 15) // 16)
    for rep in range(2):   # the second pass: zero-fills honoured, nothing accumulates
        eng.forward()
        got_pose = eng.backward_with_pose_grad().astype(np.float64)
        n0 = refs[0]["sorted_ids"].size
        K = n0 + refs[1]["sorted_ids"].size
        assert eng.n_isects == K
        assert eng.cache("sorted_ids").size == (K + K // 16 + 65536 if deferred and rep else K)
        assert np.array_equal(eng.cache("sorted_ids")[:K],
                              np.concatenate([refs[0]["sorted_ids"], refs[1]["sorted_ids"] + (np.int64(tiles) << 32)]))
        assert np.array_equal(eng.cache("sorted_flat")[:K], np.concatenate([refs[0]["sorted_flat"], refs[1]["sorted_flat"] + n]))
        assert np.array_equal(eng.cache("offsets"),
                              np.concatenate([refs[0]["offsets"].reshape(-1), refs[1]["offsets"].reshape(-1) + n0]))
        assert np.array_equal(eng.cache("aabb").reshape(2, n, 4), np.stack([r["proj"]["aabb"] for r in refs]))
        assert np.array_equal(eng.cache("radii"), np.maximum(refs[0]["proj"]["radii"], refs[1]["proj"]["radii"]))
        rgb, depth, T = eng.render()
        last = eng.cache("last_ids").reshape(2, h, w)
        for k in range(2):
            assert np.abs(rgb[k] - refs[k]["fwd"]["rgb"]).max() <= 1e-4
            assert np.abs(depth[k] - refs[k]["fwd"]["depth"]).max() <= 1e-4 * max(1.0, np.abs(refs[k]["fwd"]["depth"]).max())
            assert np.abs(T[k] - refs[k]["fwd"]["T"]).max() <= 1e-4
            # last_ids are positions in the whole sorted list (image 1's run starts at n0); a pixel no
            # fragment reached keeps 0 and T = 1
            reached = refs[k]["fwd"]["T"] < 1.0
            assert np.array_equal(last[k], np.where(reached, refs[k]["fwd"]["last_ids"] + (n0 if k else 0), 0))
            print(f"  pose gradient {k}: max err / max {np.abs(got_pose[k] - poses[k]).max() / np.abs(poses[k]).max():.3e}", flush=True)
            assert np.abs(got_pose[k] - poses[k]).max() <= 1e-3 * np.abs(poses[k]).max(), (k, got_pose[k], poses[k])
        g = eng.grads()
        for key, v in g.items():
            r = sum(ref["grads"][key].astype(np.float64) for ref in refs).reshape(n, -1)
            scale = sum(np.abs(ref["grads"][key].astype(np.float64)).reshape(n, -1).max(axis=1, keepdims=True) for ref in refs)
            world_grad_check(v, r, n, f"two-cameras/{key}", scale=scale)


def _two_camera_scene(pkg, n=3000, seed=71, cull_every=0):
    """A scene, two cameras that see different subsets of it, per-camera cotangents, and the scene with both."""
    import copy
    S = pkg.scenes
    base = S.tiny_scene(n=n, width=250, height=180, seed=seed)
    if cull_every:
        base.means[::cull_every, 2] = -10.0
    cams = []
    # the second camera looks past the scene's edge, so that each camera sees splats the other does not
    for k, (ang, t) in enumerate([(0.2, (0.9, -0.2, 2.2)), (-0.35, (-1.1, 0.1, 2.4))]):
        c, s_ = np.cos(ang), np.sin(ang)
        vm = np.array([[c, 0, s_, t[0]], [0, 1, 0, t[1]], [-s_, 0, c, t[2]], [0, 0, 0, 1]], np.float32)
        it = np.array([150.0 + 20 * k, 155.0 - 10 * k, 125.0, 90.0 + 5 * k], np.float32)
        cams.append((vm, it))
    rng = np.random.default_rng(5)
    h, w = base.height, base.width
    v_rgb = rng.standard_normal((2, h, w, 3)).astype(np.float32)
    v_depth = rng.standard_normal((2, h, w)).astype(np.float32)
    v_T = rng.standard_normal((2, h, w)).astype(np.float32)
    singles = []
    for k, (vm, it) in enumerate(cams):
        sc = copy.deepcopy(base)
        sc.viewmat, sc.intrins = vm, it
        sc.v_rgb, sc.v_depth, sc.v_T = v_rgb[k], v_depth[k], v_T[k]
        singles.append(sc)
    both = copy.deepcopy(base)
    both.viewmat = np.stack([c[0] for c in cams])
    both.intrins = np.stack([c[1] for c in cams])
    both.v_rgb, both.v_depth, both.v_T = v_rgb, v_depth, v_T
    return base, singles, both


@pytest.mark.parametrize("native", [False, True, "world-rows"])
def test_engine_two_cameras_packed_projection(pkg, oracle, H, native):
    """The packed projection over a camera batch (ProjectionPackedFwd_kernel.cuh:37-47,119-135: one scan over C * N):
    rows ordered by (camera, splat), camera_ids saying which image a row belongs to, and every later stage on
    those rows; against the oracle's packed chain run once per camera."""
    host, lib = H
    base, singles, both = _two_camera_scene(pkg, cull_every=4)
    n, h, w = base.n, base.height, base.width
    refs = [oracle.pipeline_packed(sc) for sc in singles]
    m = [r["proj"]["visible"] for r in refs]
    assert min(m) > 100 and m[0] != m[1]
    world_rows = native == "world-rows"   # the parameter rows of both cameras, one run behind the other
    native = bool(native)
    eng = host.Engine(both, packed_projection=True, fuse_tile_count=native, packed_rows=native, overwrite_world_grads=native,
                      packed_vscreen=native, tile_sort=native, packed_world_rows=world_rows)
    tiles = ((w + 15) // 16) * ((h + 15) // 16)
    for rep in range(2):
        eng.forward()
        eng.backward()
        assert np.array_equal(eng.cache("gaussian_ids"), np.concatenate([r["proj"]["gaussian_ids"] for r in refs]))
        assert np.array_equal(eng.cache("camera_ids"), np.repeat([0, 1], m).astype(np.int32))
        assert np.array_equal(eng.cache("aabb").reshape(-1, 4), np.concatenate([r["proj"]["aabb"] for r in refs]))
        n0 = refs[0]["sorted_ids"].size
        assert eng.n_isects == n0 + refs[1]["sorted_ids"].size
        assert np.array_equal(eng.cache("sorted_ids"),
                              np.concatenate([refs[0]["sorted_ids"], refs[1]["sorted_ids"] + (np.int64(tiles) << 32)]))
        assert np.array_equal(eng.cache("sorted_flat"), np.concatenate([refs[0]["sorted_flat"], refs[1]["sorted_flat"] + m[0]]))
        rgb, depth, T = eng.render()
        for k in range(2):
            assert np.abs(rgb[k] - refs[k]["fwd"]["rgb"]).max() <= 1e-4
            assert np.abs(T[k] - refs[k]["fwd"]["T"]).max() <= 1e-4
        g = eng.grads()
        for key, v in g.items():
            r = sum(ref["grads"][key].astype(np.float64) for ref in refs).reshape(n, -1)
            scale = sum(np.abs(ref["grads"][key].astype(np.float64)).reshape(n, -1).max(axis=1, keepdims=True) for ref in refs)
            world_grad_check(v, r, n, f"two-cameras-packed/{key}", scale=scale)


def test_engine_two_cameras_tile_mask(pkg, oracle, H):
    """compute_tile_active on an [I = 2, H_mask, W_mask] mask (IntersectTile.cuh:18-22) and both tile passes with one
    [tile_h, tile_w] block of the map per image: each image's keys are its own camera's masked keys."""
    host, lib = H
    base, singles, both = _two_camera_scene(pkg)
    h, w = base.height, base.width
    tiles = ((w + 15) // 16) * ((h + 15) // 16)
    rng = np.random.default_rng(9)
    masks = (rng.uniform(size=(2, 23, 31)) > 0.55).astype(np.uint8)
    refs = []
    for k, sc in enumerate(singles):
        live = oracle.compute_tile_active(masks[k], w, h)
        assert 0 < live.sum() < live.size
        refs.append(oracle.pipeline(sc, tile_active=live))
    eng = host.Engine(both)
    eng.set_tile_mask(masks)
    eng.forward()
    n0 = refs[0]["sorted_ids"].size
    assert eng.n_isects == n0 + refs[1]["sorted_ids"].size
    assert np.array_equal(eng.cache("sorted_ids"),
                          np.concatenate([refs[0]["sorted_ids"], refs[1]["sorted_ids"] + (np.int64(tiles) << 32)]))
    assert np.array_equal(eng.cache("sorted_flat"), np.concatenate([refs[0]["sorted_flat"], refs[1]["sorted_flat"] + base.n]))
    rgb, depth, T = eng.render()
    for k in range(2):
        assert np.abs(rgb[k] - refs[k]["fwd"]["rgb"]).max() <= 1e-4


@pytest.mark.parametrize("packed", [False, True])
def test_engine_two_cameras_fused_optimizer(pkg, oracle, H, packed):
    """The fused optimizer over a camera batch: one Adam step on the SUM of both cameras' gradients
    (FusedProjectionBwdOptim.cu:160-212 gathers every camera's row of a splat; FusedProjectionBwdOptim_kernel.cuh:262-330
    sums them). Oracle: camera 1's projection backward as incoming gradients (SH included) of the fused step of
    camera 0."""
    host, lib = H
    base, singles, both = _two_camera_scene(pkg, n=4000, seed=72, cull_every=5 if packed else 0)
    n = base.n
    hy = dict(lr_means=1.6e-4, lr_quats=1e-3, lr_scales=5e-3, lr_opacs=5e-2, lr_features_dc=2.5e-3, lr_features_sh=1.25e-3,
              max_gauss_ratio=6.0, scale_regularization_weight=0.01, mcmc_opacity_reg_weight=0.01, mcmc_scale_reg_weight=0.01,
              quat_norm_reg_weight=0.02, sh_reg_weight=0.05)
    eng = host.Engine(both, packed_projection=packed)
    eng.forward()
    eng.backward_fused_optimizer(hy, 3)
    got = eng.params()
    refs = [oracle.pipeline(sc) for sc in singles]
    P = {k: np.ascontiguousarray(getattr(base, k), np.float32).copy() for k in oracle.WORLD_KEYS}
    g1 = {k: np.zeros_like(v) for k, v in P.items()}
    g2 = {k: np.zeros_like(v) for k, v in P.items()}
    other = refs[1]["grads"]
    v_in = dict(means=other["v_means"], quats=other["v_quats"], log_scales=other["v_scales"], opacity_logits=other["v_opacities"],
                features_dc=other["v_dc"], features_sh=other["v_sh"])
    v_in = {k: np.ascontiguousarray(v, np.float32) for k, v in v_in.items()}
    oracle.fused_projection_bwd_optimizer(singles[0], refs[0]["proj"]["aabb"], refs[0]["vscreen"], P, g1, g2,
                                          dict(hy, v_in_sh=1.0), step=3, v_in=v_in)
    lrs = dict(means="lr_means", quats="lr_quats", log_scales="lr_scales", opacity_logits="lr_opacs",
               features_dc="lr_features_dc", features_sh="lr_features_sh")
    vis1_only = (refs[1]["proj"]["aabb"][:, 2] > refs[1]["proj"]["aabb"][:, 0]) & ~(refs[0]["proj"]["aabb"][:, 2] > refs[0]["proj"]["aabb"][:, 0])
    assert vis1_only.sum() > 20       # splats only the second camera sees: their step comes from its gradients alone
    for k in oracle.WORLD_KEYS:
        step_got = got[k].astype(np.float64) - getattr(base, k)
        step_want = P[k].astype(np.float64) - getattr(base, k)
        # a first Adam step moves every parameter by about lr whatever the gradient's size, so a wrong gradient SIGN
        # or a missing camera shows as a difference of the order of lr
        far = np.abs(step_got - step_want) > 0.02 * hy[lrs[k]] + 1e-7
        assert far.mean() < 2e-3, (k, float(far.mean()))
        moved = np.abs(step_want.reshape(n, -1)[vis1_only]).max(axis=1) > 0.5 * hy[lrs[k]]
        assert moved.mean() > 0.5, k      # (a visible splat that no pixel composites has no gradient and stays)


@pytest.mark.parametrize("accum_mode", [1, 3])
def test_engine_two_cameras_variants(pkg, oracle, H, accum_mode):
    """Two cameras with the distortion images, median depth and accumulation weights: per-pixel outputs are
    each camera's own, the weights of both cameras land in the splat's one world row
    (RasterizationEval3DBwd_kernel.cuh:368: row % N) -- summed for SUM/AVG, the larger for MAX."""
    import copy
    host, lib = H
    S = pkg.scenes
    base = S.tiny_scene(n=2500, width=200, height=150, seed=77)
    h, w, n = base.height, base.width, base.n
    rng = np.random.default_rng(9)
    vms, its = [], []
    for k, ang in enumerate([0.15, -0.3]):
        c, s_ = np.cos(ang), np.sin(ang)
        vms.append(np.array([[c, 0, s_, 0.2 - 0.5 * k], [0, 1, 0, 0.1 * k], [-s_, 0, c, 3.0 + 0.3 * k], [0, 0, 0, 1]], np.float32))
        its.append(np.array([140.0 + 15 * k, 145.0, 100.0, 75.0 - 4 * k], np.float32))
    cot = dict(v_rgb=rng.standard_normal((2, h, w, 3)), v_depth=rng.standard_normal((2, h, w)), v_T=rng.standard_normal((2, h, w)),
               v_dist_rgb=rng.uniform(-1, 1, (2, h, w, 3)), v_dist_depth=rng.uniform(-1, 1, (2, h, w)),
               accum_map=rng.uniform(0, 1, (2, h, w)))
    cot = {k: v.astype(np.float32) for k, v in cot.items()}
    refs, meds = [], []
    for k in range(2):
        sc = copy.deepcopy(base)
        sc.viewmat, sc.intrins = vms[k], its[k]
        sc.v_rgb, sc.v_depth, sc.v_T = cot["v_rgb"][k], cot["v_depth"][k], cot["v_T"][k]
        va = dict(dist_type=2, median=False, accum_mode=accum_mode, v_dist_rgb=cot["v_dist_rgb"][k],
                  v_dist_depth=cot["v_dist_depth"][k], accum_map=cot["accum_map"][k])
        refs.append(oracle.pipeline(sc, variant=va))
        meds.append(oracle.pipeline(sc, backward=False, variant=dict(median=True))["fwd"]["median"])
        assert refs[-1]["proj"]["visible"] > 100
    both = copy.deepcopy(base)
    both.viewmat, both.intrins = np.stack(vms), np.stack(its)
    both.v_rgb, both.v_depth, both.v_T = cot["v_rgb"], cot["v_depth"], cot["v_T"]
    eng = host.Engine(both)
    eng.set_variants(dist_type=2, median=True)
    eng.forward()
    eng.backward_with_variants(cot["v_dist_rgb"], cot["v_dist_depth"], None, cot["accum_map"], accum_mode=accum_mode)
    dist_rgb, dist_depth = eng.cache("dist_rgb").reshape(2, h, w, 3), eng.cache("dist_depth").reshape(2, h, w)
    median = eng.cache("median").reshape(2, h, w)
    for k in range(2):
        assert np.abs(dist_rgb[k] - refs[k]["fwd"]["dist_rgb"]).max() <= 1e-4
        assert np.abs(dist_depth[k] - refs[k]["fwd"]["dist_depth"]).max() <= 1e-4
        assert (np.abs(median[k] - meds[k]) <= 1e-4 * np.maximum(1, np.abs(meds[k]))).all()
    aw = eng.cache("accum_weight")
    a0, a1 = (r["vscreen"]["accum_weight"] for r in refs)
    want = np.maximum(a0, a1) if accum_mode == 1 else a0 + a1
    assert aw.size == want.size == (2 * n if accum_mode == 3 else n)
    assert (a0[:n] > 0).sum() > 100 and (a1[:n] > 0).sum() > 100 and ((a0[:n] > 0) != (a1[:n] > 0)).sum() > 10
    assert np.allclose(aw, want, rtol=1e-3, atol=1e-6)
    g = eng.grads()
    for key, v in g.items():
        r = sum(ref["grads"][key].astype(np.float64) for ref in refs).reshape(n, -1)
        scale = sum(np.abs(ref["grads"][key].astype(np.float64)).reshape(n, -1).max(axis=1, keepdims=True) for ref in refs)
        world_grad_check(v, r, n, f"two-cameras-variants/{key}", scale=scale)


def test_forward_only_caller_learns_of_a_short_frame(pkg, oracle, H):
    """A render loop never runs a backward and never asks for the counts. With the counts left on the device, a frame
    whose intersection outgrew its arrays is counted, left in the backend's sticky error, and its image is refused
    when it is fetched; the next frame reads its count again and is whole."""
    host, lib = H
    sc = pkg.scenes.make_scene(1, n=20000, width=320, height=240, parity_variant=True)
    plain = host.Engine(sc)
    plain.forward()
    want = plain.render()
    K = plain.n_isects
    eng = host.Engine(sc, deferred_counts=True)
    eng.forward()
    assert eng.n_isects == K
    base = eng.short_frames
    eng.set_deferred_counts(True, capacity=K // 3)
    eng.forward()                       # short: nobody asks
    eng.forward()                       # settles the abandoned counts; this one reads its count and is whole
    assert eng.short_frames == base + 1
    got = eng.render()
    for a, b in zip(got, want):
        assert np.array_equal(a, b)
    eng.set_deferred_counts(True, capacity=K // 3)
    eng.forward()                       # short again, and this time the image is fetched
    with pytest.raises(lib.SsrError, match="did not fit"):
        eng.render()
    assert eng.short_frames == base + 2
    eng.forward()
    got = eng.render()
    for a, b in zip(got, want):
        assert np.array_equal(a, b)
    eng.set_deferred_counts(False, 0)
