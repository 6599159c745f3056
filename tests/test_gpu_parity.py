"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle on the same seeded
inputs. Bars: tile keys / sorted ids / tile ranges bit-exact; images max-abs 1e-4 per channel;
gradients 1e-3 relative (with a floor proportional to the sum of |terms|, since float atomics add
in a different order)."""
import ctypes as C
import dataclasses
import math

import numpy as np
import pytest

from gpu_pipeline import GpuRun, world_grad_check

pytestmark = pytest.mark.gpu

IMG_TOL = 1e-4
GRAD_RTOL = 1e-3


@pytest.fixture(scope="module")
def gpu(pkg):
    from spirula_studio_amd import lib
    pkg.lib = lib
    lib.check(lib.load().ssr_init(0))
    return pkg


def _grad_close(got, ref, abs_scale, name, max_bad=0, rtol=GRAD_RTOL, afrac=2e-6):
    got, ref = got.astype(np.float64), ref.astype(np.float64)
    tol = rtol * np.abs(ref) + afrac * abs_scale + 1e-9
    bad = np.abs(got - ref) > tol
    assert bad.sum() <= max_bad, (name, int(bad.sum()), float(np.abs(got - ref).max()),
                                  got[bad][:4], ref[bad][:4])


def _compare(gpu, oracle, sc, label, fused_count=False, use_list=False, use_packed=False, mask=None, variant=None,
             use_vrows=False, tile_sort=False, spare=None, bwd_lanes=False, block_masks=False):
    """spare: run K4-K6 without reading the counts back, in arrays of K + spare entries (spare >= 0). bwd_lanes: the
    compositing backward with one lane per fragment (SSR_BWD_SCHEDULE_LANES). block_masks: the forward records the
    block mask of every staged entry and the backward reads them instead of repeating the tests."""
    live = None if mask is None else oracle.compute_tile_active(mask, sc.width, sc.height)
    r = oracle.pipeline(sc, tile_active=live, variant=variant)
    print(f"[{label}] N={sc.n} {sc.width}x{sc.height} visible={r['proj']['visible']} K={r['isect_ids'].size}", flush=True)
    K = r["isect_ids"].size
    g = GpuRun(gpu, sc, use_list=use_list, use_packed=use_packed, use_vrows=use_vrows, tile_sort=tile_sort,
               capacity=None if spare is None else K + spare, bwd_lanes=bwd_lanes, block_masks=block_masks)
    if mask is not None:
        g.set_tile_mask(mask)
        assert np.array_equal(g.host("tile_active"), live)
    g.variant = variant or {}
    g.run_all(fused_count=fused_count)
    if use_list:
        assert g.V == r['proj']['visible']
        assert np.array_equal(np.sort(g.host('vis_ids')[:g.V]), np.nonzero(r['proj']['aabb'][:, 2] > r['proj']['aabb'][:, 0])[0])
    vis = r["proj"]["aabb"][:, 2] > r["proj"]["aabb"][:, 0]
    # K1: bit-exact on every compared array (culled screen rows are not written by either side)
    p = g.proj_host()
    for k in ["aabb", "sort_depth", "radii"]:
        assert np.array_equal(p[k].view(np.uint32), r["proj"][k].view(np.uint32)), k
    for k in ["xy", "depth", "conic", "opac", "rgb"]:
        assert np.array_equal(p[k][vis].view(np.uint32), r["proj"][k][vis].view(np.uint32)), k
    # K2..K6: bit-exact
    assert np.array_equal(g.host("counts"), r["counts"])
    assert np.array_equal(g.host("cum"), r["cum"])
    if spare is None:
        assert g.K == K
        assert np.array_equal(g.unsorted_keys, r["isect_ids"])
        assert np.array_equal(g.unsorted_vals, r["flatten_ids"])
        assert np.array_equal(g.host(g.keys), r["sorted_ids"])
        assert np.array_equal(g.host(g.vals), r["sorted_flat"])
        assert np.array_equal(g.host("offsets"), r["offsets"])
    else:   # the keys in front, one more offset
        n_tiles = sc.tile_w * sc.tile_h
        assert g.K_real == K and g.K == K + spare
        assert np.array_equal(g.host(g.keys)[:K], r["sorted_ids"])
        assert np.array_equal(g.host(g.vals)[:K], r["sorted_flat"])
        assert np.array_equal(g.host("offsets")[:n_tiles], r["offsets"].ravel())
        assert g.host("offsets")[n_tiles] == K
    # K7
    f = r["fwd"]
    assert np.abs(g.host("r_rgb") - f["rgb"]).max() <= IMG_TOL
    assert np.abs(g.host("r_T") - f["T"]).max() <= IMG_TOL
    dd = np.abs(g.host("r_depth") - f["depth"])
    assert (dd <= IMG_TOL * np.maximum(1.0, np.abs(f["depth"]))).all()
    assert np.array_equal(g.host("r_last"), f["last_ids"])
    va = variant or {}
    if va.get("dist_type"):
        assert np.abs(g.host("r_dist_depth") - f["dist_depth"]).max() <= IMG_TOL
        if va["dist_type"] == 2:
            assert np.abs(g.host("r_dist_rgb") - f["dist_rgb"]).max() <= IMG_TOL
    if va.get("median"):
        assert (np.abs(g.host("r_median") - f["median"]) <= IMG_TOL * np.maximum(1.0, np.abs(f["median"]))).all()
    # K8
    vs = r["vscreen"]
    if va.get("accum_mode"):
        aw = g.host("accum_weight")
        assert np.allclose(aw, vs["accum_weight"], rtol=1e-3, atol=1e-6)
        assert (aw[:sc.n] > 0).sum() > 10
    ab = vs["abs_terms"]
    # The median's backward finds the crossing of T = 1/2 on the transmittance it reconstructs by undoing the
    # recursion; a pixel whose T sits within rounding of 1/2 can attribute it to the neighbouring splat on either
    # side (the reference's own backward has the same property against its forward), so two elements may disagree.
    # The median's terms are not part of the |term| sums that set the floor, and its interpolation weight divides
    # by ln(1 - alpha) >= 0.004, so the floor is raised to 1e-4 of those sums; the relative bar stays at 1e-3.
    # (Measured on the MI355X: nothing beyond 1e-3 relative + 3e-5 of the sums except two elements in one case.)
    mb = 2 if va.get("median") else 0
    kw = dict(rtol=GRAD_RTOL, afrac=1e-4) if mb else {}
    if va.get("dist_type") and not mb:
        # the distortion terms contain (c W - C), a difference of nearly equal numbers whose rounding is
        # not part of the |term| sums that set the floor: widen the floor for these runs
        kw = dict(afrac=3e-5)
    _grad_close(g.host("v_xy"), vs["v_xy"], ab[:, 0:2], "v_xy", 2 * mb, **kw)
    _grad_close(g.host("v_depth"), vs["v_depth"], ab[:, 2], "v_depth", mb, **kw)
    _grad_close(g.host("v_conic"), vs["v_conic"], ab[:, 3:6], "v_conic", 3 * mb, **kw)
    _grad_close(g.host("v_opac"), vs["v_opac"], ab[:, 6], "v_opac", mb, **kw)
    _grad_close(g.host("v_rgb"), vs["v_rgb"], ab[:, 7:10], "v_rgb", 3 * mb, **kw)
    if mb:   # K9 below would inherit those few rows
        return g, r
    # K9, fed its own K8 output, against the oracle chain: 1e-3 relative per element, each element's floor being
    # what the floors of the ten screen gradients become through the projection VJP
    gr = r["grads"]
    floors = oracle.world_grad_floors(sc, r, afrac=kw.get("afrac", 2e-6))
    for k, o in [("w_means", "v_means"), ("w_quats", "v_quats"), ("w_log_scales", "v_scales"),
                 ("w_opacity_logits", "v_opacities"), ("w_features_dc", "v_dc"), ("w_features_sh", "v_sh")]:
        got = g.host(k)
        world_grad_check(got, gr[o], sc.n, f"{label}/{k}", elem_floor=floors[o])
        assert not np.any(got[~vis]), k
    return g, r


def test_counts_stay_on_the_device(gpu, oracle):
    """K4-K8 in arrays sized without the counts (ssr_tile_write_capped, ssr_sort_tile_pairs_capped, closed offsets):
    same keys, ranges, images and gradients as with the readback, whatever the spare room."""
    _compare(gpu, oracle, gpu.scenes.tiny_scene(n=400, width=72, height=56, seed=3), "tiny-cap", tile_sort=True, spare=300)
    _compare(gpu, oracle, gpu.scenes.tiny_scene(n=300, width=16, height=16, seed=6), "one-tile-cap", tile_sort=True, spare=1)
    _compare(gpu, oracle, gpu.scenes.tiny_scene(n=400, width=72, height=56, seed=3), "exact-cap", tile_sort=True, spare=0)
    # 128 x 128 tiles: a power of two
    _compare(gpu, oracle, gpu.scenes.tiny_scene(n=60, width=2048, height=2048, seed=12), "pow2-cap", tile_sort=True, spare=5000)
    sc = gpu.scenes.make_scene(2, n=30000, width=480, height=270)
    _compare(gpu, oracle, sc, "cfg2-cap", fused_count=True, use_list=True, use_packed=True, use_vrows=True, tile_sort=True,
             spare=70000)
    huge = gpu.scenes.tiny_scene(n=600, width=640, height=400, seed=13)
    huge.log_scales[::7] += 2.5          # splats that cover hundreds of tiles (the cooperative write)
    huge.means[::50, 2] = -3.6
    _compare(gpu, oracle, huge, "huge-cap", fused_count=True, use_list=True, tile_sort=True, spare=100)
    none = gpu.scenes.tiny_scene(n=64, width=40, height=24, seed=1)
    none.means[:, 2] = -10.0   # nothing in view: a count of zero that only the device knows
    g, r = _compare(gpu, oracle, none, "all-culled-cap", tile_sort=True, spare=128)
    assert g.K_real == 0 and not np.any(g.host("offsets")) and np.all(g.host("r_T") == 1.0)
    g, r = _compare(gpu, oracle, none, "all-culled-cap-list", fused_count=True, use_list=True, tile_sort=True, spare=128)
    assert g.K_real == 0 and g.V == 0 and np.all(g.host("r_T") == 1.0)


def test_counts_beyond_the_capacity_lose_keys_only(gpu, oracle):
    """More keys than the arrays hold: nothing outside the arrays is touched, every later stage runs on what fitted,
    and the count that comes back says so."""
    sc = gpu.scenes.tiny_scene(n=400, width=72, height=56, seed=3)
    r = oracle.pipeline(sc)
    K = r["isect_ids"].size
    cap = K - K // 3
    g = GpuRun(gpu, sc, tile_sort=True, capacity=cap)
    g.run_all()
    assert g.K_real == K and g.K == cap
    n_tiles = sc.tile_w * sc.tile_h
    keys, vals, offs = g.host(g.keys), g.host(g.vals), g.host("offsets")
    assert offs[n_tiles] == cap and np.all(np.diff(offs) >= 0)
    assert np.all((keys >> 32) < n_tiles) and np.all(np.diff(keys) >= 0)   # real keys only, sorted
    # what fitted is what the key write puts below `cap`
    keep = np.sort(r["isect_ids"][:cap], kind="stable")
    assert np.array_equal(keys, keep)
    assert vals.min() >= 0 and vals.max() < sc.n
    assert np.isfinite(g.host("r_rgb")).all() and np.isfinite(g.host("w_means")).all()


def _compare_packed(gpu, oracle, sc, label, fused_count=False, use_packed=False, read_nnz=True, variant=None):
    """Packed projection outputs (nnz compacted rows) through every later stage."""
    r = oracle.pipeline_packed(sc, variant=variant)
    q = r["proj"]
    m = q["visible"]
    print(f"[{label}] N={sc.n} {sc.width}x{sc.height} nnz={m} K={r['isect_ids'].size}", flush=True)
    g = GpuRun(gpu, sc, use_packed=use_packed, packed_projection=True, read_nnz=read_nnz)
    g.variant = variant or {}
    g.run_all(fused_count=fused_count)
    assert g.nnz == m
    # K1 packed: ids exact and ascending, rows bit-exact, rows past nnz untouched
    assert np.array_equal(g.host("gaussian_ids")[:m], q["gaussian_ids"])
    assert not np.any(g.host("camera_ids")[:m])
    assert np.array_equal(g.host("radii").view(np.uint32), q["radii"].view(np.uint32))
    for k in ["aabb", "sort_depth", "xy", "depth", "conic", "opac", "rgb"]:
        got = g.host(k)
        assert np.array_equal(got[:m].view(np.uint32), q[k].view(np.uint32)), k
        assert np.all(got[m:].view(np.uint32) == 0x7fc12345), k
    # K2..K6: bit-exact, flatten ids are packed row numbers
    assert np.array_equal(g.host("counts")[:m], r["counts"])
    assert np.array_equal(g.host("cum")[:m], r["cum"])
    assert g.K == r["isect_ids"].size
    assert np.array_equal(g.unsorted_keys, r["isect_ids"])
    assert np.array_equal(g.unsorted_vals, r["flatten_ids"])
    assert np.array_equal(g.host(g.keys), r["sorted_ids"])
    assert np.array_equal(g.host(g.vals), r["sorted_flat"])
    assert np.array_equal(g.host("offsets"), r["offsets"])
    f = r["fwd"]
    assert np.abs(g.host("r_rgb") - f["rgb"]).max() <= IMG_TOL
    assert np.abs(g.host("r_T") - f["T"]).max() <= IMG_TOL
    dd = np.abs(g.host("r_depth") - f["depth"])
    assert (dd <= IMG_TOL * np.maximum(1.0, np.abs(f["depth"]))).all()
    assert np.array_equal(g.host("r_last"), f["last_ids"])
    va = variant or {}
    if va.get("dist_type"):
        assert np.abs(g.host("r_dist_depth") - f["dist_depth"]).max() <= IMG_TOL
        if va["dist_type"] == 2:
            assert np.abs(g.host("r_dist_rgb") - f["dist_rgb"]).max() <= IMG_TOL
    if va.get("median"):
        assert (np.abs(g.host("r_median") - f["median"]) <= IMG_TOL * np.maximum(1.0, np.abs(f["median"]))).all()
    vs = r["vscreen"]
    if va.get("accum_mode"):   # indexed by world splat through gaussian_ids
        assert np.allclose(g.host("accum_weight"), vs["accum_weight"], rtol=1e-3, atol=1e-6)
    ab = vs["abs_terms"]
    kw = dict(afrac=3e-5) if va.get("dist_type") else {}   # see _compare
    assert not va.get("median"), "median rows: use _compare's tolerance handling"
    for k, cols in [("v_xy", slice(0, 2)), ("v_depth", 2), ("v_conic", slice(3, 6)), ("v_opac", 6), ("v_rgb", slice(7, 10))]:
        _grad_close(g.host(k)[:m], vs[k], ab[:, cols], k, **kw)
    gr = r["grads"]
    vis = np.zeros(sc.n, bool)
    vis[q["gaussian_ids"]] = True
    for k, o in [("w_means", "v_means"), ("w_quats", "v_quats"), ("w_log_scales", "v_scales"),
                 ("w_opacity_logits", "v_opacities"), ("w_features_dc", "v_dc"), ("w_features_sh", "v_sh")]:
        got = g.host(k)
        world_grad_check(got, gr[o], sc.n, f"{label}/{k}")
        assert not np.any(got[~vis]), k
    return g, r


def test_device_math_is_bit_identical_to_host(gpu, oracle):
    lib, L = gpu.lib.load(), gpu.lib
    rng = np.random.default_rng(0)
    a = np.concatenate([rng.uniform(-100, 100, 300000), rng.normal(0, 3, 300000),
                        [0.0, -0.0, 1.0, 88.7, -87.3, 1e-40, 255.0]]).astype(np.float32)
    b = rng.normal(0, 3, a.size).astype(np.float32)
    db, do = L.DeviceArray.from_host(b), L.DeviceArray(a.shape, np.float32)
    for op in range(4):
        x = np.abs(a) if op == 1 else a
        da = L.DeviceArray.from_host(x)
        L.check(lib.ssr_debug_math(op, a.size, da.ptr, db.ptr, do.ptr, None))
        got = do.to_host()
        want = oracle.math(op, x, b)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), op
    # Adam's inverse bias corrections (ops 4, 5) at integer steps
    t = np.concatenate([np.arange(1, 20000), [50000, 1000000]]).astype(np.float32)
    dt, dr = L.DeviceArray.from_host(t), L.DeviceArray(t.shape, np.float32)
    for op in (4, 5):
        L.check(lib.ssr_debug_math(op, t.size, dt.ptr, dt.ptr, dr.ptr, None))
        assert np.array_equal(dr.to_host().view(np.uint32), oracle.math(op, t).view(np.uint32)), op


def test_tiny_pinhole(gpu, oracle):
    _compare(gpu, oracle, gpu.scenes.tiny_scene(n=400, width=72, height=56, seed=3), "tiny")


def test_tiny_fused_count(gpu, oracle):
    _compare(gpu, oracle, gpu.scenes.tiny_scene(n=500, width=64, height=64, seed=5), "tiny-fused", fused_count=True)


def test_visible_work_list(gpu, oracle):
    """K4 and K9 driven by the list of visible splats that K1 emits: same keys, same gradients."""
    sc = gpu.scenes.make_scene(4, n=60000, width=480, height=270, sh_codec=0)   # mostly culled
    _compare(gpu, oracle, sc, "cfg4-list", fused_count=True, use_list=True)
    _compare(gpu, oracle, gpu.scenes.tiny_scene(n=700, width=96, height=64, seed=8), "tiny-list", use_list=True)


def test_packed_fragment_rows(gpu, oracle):
    """The compositing kernels fed from K1's 48-byte packed rows: identical results."""
    _compare(gpu, oracle, gpu.scenes.tiny_scene(n=700, width=96, height=64, seed=9), "tiny-packed", use_packed=True)
    sc = gpu.scenes.make_scene(2, n=50000, width=480, height=270, parity_variant=True)
    _compare(gpu, oracle, sc, "cfg2-packed", fused_count=True, use_list=True, use_packed=True)


def test_huge_splats_cooperative_key_write(gpu, oracle):
    """Splats that cover hundreds of tiles take the wavefront-cooperative path of the key write."""
    sc = gpu.scenes.tiny_scene(n=600, width=640, height=400, seed=13)
    sc.log_scales[::7] += 2.5          # every 7th splat becomes very large
    sc.means[::50, 2] = -3.6           # a few right in front of the camera (camera at z = -4)
    g, r = _compare(gpu, oracle, sc, "huge", fused_count=True, use_list=True)
    assert r["counts"].max() > 500
    _compare(gpu, oracle, sc, "huge-nolist")


def test_tile_segmented_sort(gpu, oracle):
    """ssr_sort_tile_pairs in place of the whole-key sort and the offsets kernel: the same sorted keys,
    values and tile ranges, and so the same images and gradients."""
    _compare(gpu, oracle, gpu.scenes.tiny_scene(n=400, width=72, height=56, seed=3), "tiny-seg", tile_sort=True)
    _compare(gpu, oracle, gpu.scenes.tiny_scene(n=300, width=16, height=16, seed=6), "one-tile-seg", tile_sort=True)
    sc = gpu.scenes.tiny_scene(n=600, width=640, height=400, seed=13)
    sc.log_scales[::7] += 2.5          # tiles with thousands of entries: the larger segment classes
    sc.means[::50, 2] = -3.6
    _compare(gpu, oracle, sc, "huge-seg", fused_count=True, use_list=True, tile_sort=True)
    _compare(gpu, oracle, gpu.scenes.make_scene(1), "cfg1-seg", fused_count=True, use_list=True, use_packed=True,
             use_vrows=True, tile_sort=True)
    _compare(gpu, oracle, gpu.scenes.make_scene(5, n=40000, width=1024, height=512), "cfg5/eq-seg", tile_sort=True)
    mask = np.zeros((30, 50), np.uint8)
    mask[4:20, 8:30] = 1
    _compare(gpu, oracle, gpu.scenes.tiny_scene(n=900, width=160, height=96, seed=41), "mask-seg", mask=mask, tile_sort=True)


CAMERA_PAIRS = [(0, 1), (0, 2), (0, 3), (1, 0), (1, 1), (1, 2), (2, 0), (2, 1), (2, 2)]


def _lens_scene(gpu, model, tier, n=1500, seed=31, width=200, height=144):
    S = gpu.scenes
    sc = S.tiny_scene(n=n, width=width, height=height, seed=seed, camera_model=model)
    if model == S.CAM_PINHOLE:   # a wide field of view, where the lens terms are not small
        sc.intrins = np.array([0.6 * width, 0.62 * width, 0.5 * width, 0.5 * height], np.float32)
        sc.viewmat[2, 3] = 2.6
    return S.with_lens(sc, tier)


@pytest.mark.parametrize("model,tier", CAMERA_PAIRS)
def test_camera_variants(gpu, oracle, model, tier):
    """FISHEYE / EQUISOLID and the lens-distortion tiers (every pair of
    src/kernels/projection/CameraVariants.cuh:11-22 beyond the two hand-written ones): K1 bit-exact, and
    through the whole path to the gradients."""
    sc = _lens_scene(gpu, model, tier)
    g, r = _compare(gpu, oracle, sc, f"model{model}-lens{tier}")
    assert r["proj"]["visible"] > 100
    _compare(gpu, oracle, sc, f"model{model}-lens{tier}-native", fused_count=True, use_list=True, use_packed=True,
             use_vrows=True, tile_sort=True)


def test_camera_variants_strong_lens_and_packed(gpu, oracle):
    """A lens strong enough that is_valid_distortion drops part of the field; the packed projection on a
    wide lens; a larger fisheye frame."""
    sc = _lens_scene(gpu, 1, 2, n=2500, seed=37)
    sc.dist_coeffs = (sc.dist_coeffs * np.float32(8.0)).astype(np.float32)
    _compare(gpu, oracle, sc, "fisheye-strong-prism")
    sc = _lens_scene(gpu, 0, 3, n=2500, seed=38)
    sc.dist_coeffs = (sc.dist_coeffs * np.float32(-8.0)).astype(np.float32)
    _compare(gpu, oracle, sc, "pinhole-strong-rational", fused_count=True, use_list=True)
    _compare_packed(gpu, oracle, _lens_scene(gpu, 2, 1, n=2000, seed=39), "equisolid-opencv-packed", fused_count=True)
    _compare_packed(gpu, oracle, _lens_scene(gpu, 0, 2, n=2000, seed=40), "pinhole-prism-packed", use_packed=True)
    sc = gpu.scenes.make_scene(5, n=40000, width=768, height=768)
    sc.camera_model = gpu.scenes.CAM_FISHEYE
    sc.intrins = np.array([768 / math.pi, 768 / math.pi, 384, 384], np.float32)
    _compare(gpu, oracle, gpu.scenes.with_lens(sc, 1), "cfg5-as-fisheye", fused_count=True, use_list=True, use_packed=True,
             use_vrows=True, tile_sort=True)


@pytest.mark.parametrize("model,tier,packed", [(0, 0, False), (0, 0, True), (0, 1, False), (1, 2, False), (3, 0, True)])
def test_antialiased_variant(gpu, oracle, model, tier, packed):
    """The antialiased ("mip") variant of the primitive through the whole iteration: blur 0.1 and the opacity
    compensation in the projection, its gradient in the projection backward."""
    sc = _lens_scene(gpu, model, tier, n=2500, seed=35)
    sc.log_scales -= 2.2          # a pixel or two on screen: the blur and its compensation matter
    sc.antialiased = True
    plain = oracle.projection_fwd(dataclasses.replace(sc, antialiased=False))
    if packed:
        g, r = _compare_packed(gpu, oracle, sc, f"mip-{model}-{tier}-packed", fused_count=True, use_packed=True)
        opac = r["full_proj"]["opac"]
    else:
        g, r = _compare(gpu, oracle, sc, f"mip-{model}-{tier}", fused_count=True, use_list=True, use_packed=True, use_vrows=True)
        opac = r["proj"]["opac"]
    both = (plain["aabb"][:, 2] > plain["aabb"][:, 0]) & (r["full_proj" if packed else "proj"]["aabb"][:, 2] > 0)
    assert both.sum() > 100 and (opac[both] < 0.9 * plain["opac"][both]).mean() > 0.1     # the compensation is at work


def test_tiny_equirect(gpu, oracle):
    _compare(gpu, oracle, gpu.scenes.tiny_scene(n=600, width=128, height=64, seed=4, camera_model=3), "tiny-eq")


def test_config1_reduced(gpu, oracle):
    _compare(gpu, oracle, gpu.scenes.make_scene(1, n=20000, width=400, height=400, parity_variant=True), "cfg1/5")


def test_config1_full(gpu, oracle):
    _compare(gpu, oracle, gpu.scenes.make_scene(1), "cfg1")
    _compare(gpu, oracle, gpu.scenes.make_scene(1), "cfg1-lanes", use_packed=True, use_vrows=True, tile_sort=True, bwd_lanes=True)


@pytest.mark.parametrize("lanes", [False, True])
def test_backward_schedules(gpu, oracle, lanes):
    """Both cuts of the compositing backward (a row per fragment, a lane per fragment) against the oracle on scenes
    that stress what differs between them: large overlapping splats with early termination, an image that is no
    multiple of the tile, opacities at the 0.999 cap (alpha capped, the exponent's gradient gated), one splat,
    lists of exactly 16 / 17 / 128 / 129 fragments in a block, the equirectangular camera's small footprints."""
    S = gpu.scenes
    kw = dict(bwd_lanes=lanes)
    _compare(gpu, oracle, S.tiny_scene(n=300, width=64, height=48, seed=11), f"sched{int(lanes)}-tiny", **kw)
    _compare(gpu, oracle, S.tiny_scene(n=300, width=64, height=48, seed=11), f"sched{int(lanes)}-tiny-masks", block_masks=True, **kw)
    kw["block_masks"] = True   # the rest with the forward's block masks handed to the backward, as the engine runs
    _compare(gpu, oracle, S.tiny_scene(n=700, width=70, height=37, seed=12), f"sched{int(lanes)}-ragged", use_packed=True, use_vrows=True, **kw)
    sc = S.tiny_scene(n=400, width=80, height=64, seed=13)
    sc.opacity_logits[::3] = 9.0          # sigmoid 0.99988: the pixel under the centre saturates at 0.999
    sc.opacity_logits[1::7] = 6.9         # 0.99899: inside the band around the cap
    _compare(gpu, oracle, sc, f"sched{int(lanes)}-opaque", use_list=True, use_packed=True, use_vrows=True, tile_sort=True, **kw)
    # the loss-map weight sums (sum, avg) ride in the gradient rows' spare floats under either cut; batches of 112
    for accum in (2, 3):
        sc = S.tiny_scene(n=700, width=70, height=37, seed=14 + accum)
        va = dict(dist_type=0, median=False, accum_mode=accum, **_variant_cotangents(sc, accum))
        _compare(gpu, oracle, sc, f"sched{int(lanes)}-sums{accum}", use_packed=True, use_vrows=True, variant=va, **kw)
    sc = S.make_scene(2, n=50000, width=480, height=270, parity_variant=True)
    va = dict(dist_type=0, median=False, accum_mode=3, **_variant_cotangents(sc, 5))
    _compare(gpu, oracle, sc, f"sched{int(lanes)}-sums-cfg2", fused_count=True, use_list=True, use_packed=True, use_vrows=True, tile_sort=True, variant=va, **kw)
    for n in (1, 16, 17, 112, 113, 128, 129, 257):  # every splat covers the one tile's every block: block lists of exactly n
        sc = S.tiny_scene(n=n, width=16, height=16, seed=100 + n)
        sc.means[:, :2] *= 0.02
        sc.log_scales[:] = -1.0 + 0.2 * (sc.log_scales - sc.log_scales.mean())   # large, and not isotropic (an isotropic
        # splat's quaternion gradient is zero but for rounding, which no relative bar can hold)
        sc.opacity_logits[:] = -3.0       # faint: no pixel terminates, every fragment composites
        _compare(gpu, oracle, sc, f"sched{int(lanes)}-list{n}", use_packed=True, use_vrows=True, **kw)
    _compare(gpu, oracle, S.make_scene(5, n=20000, width=256, height=128, parity_variant=True), f"sched{int(lanes)}-equirect",
             use_list=True, use_packed=True, use_vrows=True, tile_sort=True, **kw)


@pytest.mark.parametrize("cfg", [2, 3, 4, 5])
def test_bench_configs_full_against_the_oracle(gpu, oracle, cfg):
    """Configs 2 (the headline, 1M splats at 1080p), 3 (3M, int8 SH), 4 (10M, camera inside the scene, 4K) and 5 (6M,
    equirectangular 4096x2048) whole and at full size against the oracle, on the stage order the benchmark runs: every key, id, range and last id bit for bit, every pixel to 1e-4, every
    gradient row to 1e-3."""
    _compare(gpu, oracle, gpu.scenes.make_scene(cfg), f"cfg{cfg}-full", fused_count=True, use_list=True, use_packed=True,
             use_vrows=True, tile_sort=True, bwd_lanes=cfg in (2, 4), block_masks=True)   # the cut the engine picks for each (tiles per visible splat)


@pytest.mark.parametrize("codec,stride", [(1, 256), (1, 0), (2, 256), (3, 0)])
def test_quantized_sh(gpu, oracle, codec, stride):
    sc = gpu.scenes.make_scene(3, n=30000, width=480, height=270, sh_codec=0)
    gpu.scenes.apply_sh_codec(sc, codec, bounds_stride=stride)
    _compare(gpu, oracle, sc, f"cfg3-codec{codec}-stride{stride}")


def test_config5_reduced_equirect(gpu, oracle):
    _compare(gpu, oracle, gpu.scenes.make_scene(5, n=40000, width=512, height=256, parity_variant=True), "cfg5/150")


def test_empty_and_culled(gpu, oracle):
    sc = gpu.scenes.tiny_scene(n=64, width=40, height=24, seed=1)
    sc.means[:, 2] = -10.0
    g, r = _compare(gpu, oracle, sc, "all-culled")
    assert g.K == 0 and not np.any(g.host("offsets"))
    assert np.all(g.host("r_T") == 1.0)


@pytest.mark.parametrize("use_list,accumulate", [(False, False), (True, False), (False, True), (True, True)])
def test_projection_backward_staged_rows_equal_plain_rows(gpu, oracle, use_list, accumulate):
    """The projection backward that moves its SH gradient rows through LDS (16-byte aligned rows of 45 floats,
    degree 3) and the one-thread-per-row kernel it stands in for give the same rows bit for bit: stored or added,
    with and without a work list, culled rows zeroed or left alone alike."""
    sc = gpu.scenes.make_scene(2, n=20011, width=480, height=270)   # the last wavefront is short
    sc.means[::5, 2] = -20.0                                         # culled rows among the visible ones
    g = GpuRun(gpu, sc, use_list=use_list, use_vrows=True)
    g.run_all(backward=False, fused_count=True)
    g.raster_bwd()
    g.projection_bwd(accumulate=accumulate, poison=not accumulate)
    staged = g.host("w_features_sh").copy()
    others = {k: g.host(k).copy() for k in ["w_means", "w_quats", "w_log_scales", "w_opacity_logits", "w_features_dc"]}
    g.projection_bwd(accumulate=accumulate, poison=not accumulate, misalign_sh_rows=True)
    plain = g.sh_rows_misaligned()
    assert np.array_equal(staged.view(np.uint32), plain.view(np.uint32))
    aabb = g.host("aabb")
    vis = aabb[:, 2] > aabb[:, 0]
    assert 1000 < vis.sum() < sc.n - 1000 and np.any(staged[vis] != 0) and np.isfinite(staged[vis]).all()
    for k, v in others.items():
        assert np.array_equal(g.host(k).view(np.uint32), v.view(np.uint32)), k


def test_packed_projection_tiny(gpu, oracle):
    """projection_3dgs_packed_forward: compacted rows in ascending splat order, then the whole chain."""
    _compare_packed(gpu, oracle, gpu.scenes.tiny_scene(n=700, width=96, height=64, seed=21), "pk-tiny")
    _compare_packed(gpu, oracle, gpu.scenes.tiny_scene(n=900, width=80, height=48, seed=22), "pk-tiny-fused",
                    fused_count=True, use_packed=True)


def test_packed_backward_adds_repeated_ids(gpu, oracle):
    """A packed id list that names splats twice (the rows of two cameras in one list): the accumulating
    projection backward adds atomically by default, so both rows of a splat reach its world row; with
    ids declared unique the plain read-add-write is used and gives the single-camera result."""
    D = gpu.lib.DeviceArray
    g, r = _compare_packed(gpu, oracle, gpu.scenes.tiny_scene(n=900, width=96, height=64, seed=29), "pk-repeat")
    m = g.rows // 3
    assert m > 50
    once = {k: g.host(k).copy() for k in ["w_means", "w_quats", "w_log_scales", "w_opacity_logits", "w_features_dc", "w_features_sh"]}
    ids = g.host("gaussian_ids")[:m]
    keep = np.zeros(g.n, bool)
    keep[ids] = True
    for k in ["gaussian_ids", "v_xy", "v_depth", "v_conic", "v_opac", "v_rgb"]:
        a = g.host(k)[:m]
        g.d[k] = D.from_host(np.concatenate([a, a]))
    g.rows = 2 * m
    g.use_vrows = False
    g.projection_bwd(accumulate=True)
    for k, v in once.items():
        got = g.host(k)
        assert np.array_equal(got[keep], 2.0 * v[keep]), k      # x + x is exact, whichever row lands first
        assert not np.any(got[~keep]), k
    assert np.abs(once["w_means"][keep]).max() > 0


def test_zero_world_rows_skip_lists(gpu):
    """ssr_zero_world_rows zeroes exactly the listed rows, minus the rows its skip lists name (non-empty aabb rows,
    members of an ascending id list): checked against numpy on random lists, with an empty skip list, a skip list
    that covers everything, and ids at both ends of the range."""
    L = gpu.lib
    lib = L.load()
    rng = np.random.default_rng(77)
    n, S = 5000, 45
    shapes = dict(means=(n, 3), quats=(n, 4), log_scales=(n, 3), opacity_logits=(n,), features_dc=(n, 3), features_sh=(n, S))
    for case in range(5):
        host = {k: rng.uniform(1, 2, sh).astype(np.float32) for k, sh in shapes.items()}
        dev = {k: L.DeviceArray.from_host(v) for k, v in host.items()}
        w = L.World()
        for k in shapes:
            setattr(w, k, dev[k].ptr)
        w.sh_stride = S
        ids = np.unique(np.concatenate([rng.choice(n, 900, replace=False), [0, n - 1]])).astype(np.int32)
        rng.shuffle(ids)
        keep = {0: np.zeros(0, np.int32), 1: np.arange(n, dtype=np.int32), 2: np.array([0, n - 1], np.int32)}.get(
            case, np.sort(rng.choice(n, 1500, replace=False)).astype(np.int32))
        aabb = np.zeros((n, 4), np.float32)
        if case == 4:
            vis = rng.random(n) < 0.3
            aabb[vis] = [1.0, 2.0, 5.0, 7.0]
        d_ids, d_keep, d_aabb = L.DeviceArray.from_host(ids), L.DeviceArray.from_host(np.concatenate([keep, [0]]).astype(np.int32)), L.DeviceArray.from_host(aabb)
        L.check(lib.ssr_zero_world_rows(C.byref(w), d_ids.ptr, ids.size, d_aabb.ptr if case == 4 else None,
                                        d_keep.ptr if keep.size else None, keep.size, None))
        L.check(lib.ssr_device_synchronize())
        gone = np.zeros(n, bool)
        gone[ids] = True
        gone[keep] = False
        if case == 4:
            gone &= ~vis
        assert gone.any() or case == 1
        for k in shapes:
            want = host[k].copy()
            want[gone] = 0.0
            assert np.array_equal(dev[k].to_host(), want), (case, k)
    e = lib.ssr_zero_world_rows(C.byref(w), d_ids.ptr, ids.size, None, None, 5, None)
    assert e != 0 and b"skip list" in lib.ssr_last_error()


def test_packed_projection_without_readback(gpu, oracle):
    """Outputs sized for all N splats, nnz read only afterwards: rows past nnz stay untouched."""
    _compare_packed(gpu, oracle, gpu.scenes.tiny_scene(n=1300, width=96, height=64, seed=23), "pk-noread",
                    fused_count=True, read_nnz=False)


def test_packed_projection_sparse_and_dense(gpu, oracle):
    sc = gpu.scenes.make_scene(4, n=80000, width=480, height=270, sh_codec=3)     # mostly culled, int8 SH
    g, r = _compare_packed(gpu, oracle, sc, "pk-cfg4", fused_count=True, use_packed=True)
    assert 0 < g.nnz < sc.n // 2
    sc = gpu.scenes.make_scene(2, n=50000, width=480, height=270, parity_variant=True)   # mostly visible
    _compare_packed(gpu, oracle, sc, "pk-cfg2", fused_count=True)
    sc = gpu.scenes.make_scene(5, n=40000, width=512, height=256)                 # equirect
    _compare_packed(gpu, oracle, sc, "pk-cfg5")


def test_packed_projection_first_pass_cull(gpu, oracle):
    """The packed mask kernel first rejects splats from the mean and the scales alone and lists the rest: it may
    only reject what the projection rejects. Splats straddling every image edge with centres far off the image,
    very large splats, splats just in front of and just behind the camera plane, 256-splat slices with every
    share of candidates: rows, ids and the whole chain as the oracle's."""
    S = gpu.scenes
    sc = S.tiny_scene(n=3000, width=96, height=64, seed=31)
    sc.means[:, :2] *= 8.0                      # most centres off the image, many footprints reaching back in
    sc.log_scales[::5] += 2.0                   # some very large ones
    g, r = _compare_packed(gpu, oracle, sc, "pk-cull-edges", fused_count=True)
    assert 0 < g.nnz < 0.8 * sc.n
    sc = S.tiny_scene(n=2048, width=96, height=64, seed=32)
    cam_z = (sc.means @ sc.viewmat[2, :3]) + sc.viewmat[2, 3]
    sc.means -= np.outer(cam_z - np.where(np.arange(sc.n) % 2, 2e-2, -2e-2) * (1 + np.arange(sc.n) % 7), sc.viewmat[2, :3]) * (np.arange(sc.n) % 3 == 0)[:, None]
    _compare_packed(gpu, oracle, sc, "pk-cull-camera-plane")
    sc = S.tiny_scene(n=256 * 6, width=96, height=64, seed=33)
    blk = np.arange(sc.n) // 256
    for b, share in enumerate([0.0, 0.3, 0.6, 0.65, 0.9, 1.0]):   # share of a workgroup's splats in front of the camera
        idx = np.where(blk == b)[0]
        sc.means[idx[int(share * idx.size):], 2] = -10.0
    _compare_packed(gpu, oracle, sc, "pk-cull-threshold", fused_count=True)


def test_packed_projection_world_rows(gpu, oracle):
    """The optional parameter planes of the packed projection: entry i of the four planes holds the parameters of
    splat gaussian_ids[i] bit for bit, entries past nnz stay untouched, every other output is what it is without them, and a
    projection backward that reads the rows gives the same bits as one that gathers from the five arrays (store
    and add mode, fp32 and int8 SH, with and without the gradient rows of the compositing backward)."""
    S = gpu.scenes
    cases = [("wr-tiny", S.tiny_scene(n=2500, width=96, height=64, seed=41), dict()),
             ("wr-cfg4", S.make_scene(4, n=80000, width=480, height=270, sh_codec=3), dict(use_packed=True, use_vrows=True)),
             ("wr-cfg2", S.make_scene(2, n=30000, width=480, height=270, parity_variant=True), dict(read_nnz=False))]
    cases[0][1].means[::3, 2] = -10.0   # a third behind the camera
    keys = ["w_means", "w_quats", "w_log_scales", "w_opacity_logits", "w_features_dc", "w_features_sh"]
    for label, sc, kw in cases:
        print(f"[{label}] N={sc.n}", flush=True)
        runs = []
        for wr in (False, True):
            g = GpuRun(gpu, sc, packed_projection=True, world_rows=wr, **kw)
            g.run_all(fused_count=True)
            runs.append(g)
        a, b = runs
        m = b.nnz
        assert a.nnz == m and 0 < m < sc.n
        ids = b.host("gaussian_ids")[:m]
        rows = b.host("world_rows")
        want = np.zeros((m, 16), np.float32)
        want[:, 0:3] = sc.means[ids]; want[:, 3] = np.ravel(sc.opacity_logits)[ids]
        want[:, 4:8] = sc.quats[ids]; want[:, 8:11] = sc.log_scales[ids]; want[:, 11:14] = sc.features_dc[ids]
        assert np.array_equal(rows[:, :m].view(np.uint32), want.reshape(m, 4, 4).transpose(1, 0, 2).view(np.uint32))
        assert np.all(rows[:, m:].view(np.uint32) == 0x7fc12345)
        for k in ["gaussian_ids", "aabb", "sort_depth", "xy", "depth", "conic", "opac", "rgb", "radii", "r_rgb", "r_last"]:
            assert np.array_equal(a.host(k).view(np.uint32), b.host(k).view(np.uint32)), k
        # the projection backward on ONE set of screen gradients (the compositing backward's atomics differ in the
        # last bits from run to run), with and without the rows
        vis = np.zeros(sc.n, bool); vis[ids] = True
        for accumulate in (True, False):   # atomic adds into zeros (the plain kernel); stores over poison (the staged one)
            got = []
            for use in (True, False):
                b.projection_bwd(accumulate=accumulate, poison=not accumulate, use_world_rows=use)
                b.check(b.lib.ssr_device_synchronize())
                got.append({k: b.host(k) for k in keys})
            for k in keys:
                assert np.array_equal(got[0][k][vis].view(np.uint32), got[1][k][vis].view(np.uint32)), (k, accumulate)
                assert np.isfinite(got[0][k][vis]).all() and np.any(got[0][k][vis] != 0), k


def test_packed_projection_all_culled_and_empty(gpu, oracle):
    sc = gpu.scenes.tiny_scene(n=300, width=40, height=24, seed=1)
    sc.means[:, 2] = -10.0
    g, r = _compare_packed(gpu, oracle, sc, "pk-all-culled")
    assert g.nnz == 0 and g.K == 0 and np.all(g.host("r_T") == 1.0)


def test_packed_projection_block_boundaries(gpu, oracle):
    """Visibility patterns that leave whole wavefront slices (256 splats) and whole workgroup segments (1024 splats)
    of the mask kernel empty or full."""
    sc = gpu.scenes.tiny_scene(n=256 * 9 + 17, width=96, height=64, seed=24)
    blk = np.arange(sc.n) // 256
    sc.means[(blk == 0) | (blk == 3) | (blk == 4) | (blk == 9), 2] = -10.0   # culled blocks, incl. first and last
    g, r = _compare_packed(gpu, oracle, sc, "pk-blocks", fused_count=True)
    assert 0 < g.nnz < sc.n
    sc = gpu.scenes.tiny_scene(n=1024 * 5 + 300, width=96, height=64, seed=25)
    seg = np.arange(sc.n) // 1024
    sc.means[(seg == 0) | (seg == 2) | (seg == 5), 2] = -10.0   # culled segments: the first, one inside, the short last one
    g, r = _compare_packed(gpu, oracle, sc, "pk-segments", fused_count=True)
    assert 0 < g.nnz < sc.n
    sc = gpu.scenes.tiny_scene(n=1024 * 3, width=96, height=64, seed=26)
    seg = np.arange(sc.n) // 1024
    sc.means[(seg == 1) & (np.arange(sc.n) % 1024 < 1023), 2] = -10.0   # one survivor at the end of a segment
    g, r = _compare_packed(gpu, oracle, sc, "pk-segment-last-row")
    assert 0 < g.nnz < sc.n


def test_tile_skip_mask(gpu, oracle):
    """compute_tile_active + the tile_active argument of both tile passes: skipped tiles get an empty
    range, everything else is unchanged (src/kernels/tile/IntersectTile.cu:309-368)."""
    rng = np.random.default_rng(3)
    sc = gpu.scenes.tiny_scene(n=900, width=160, height=96, seed=41)
    sc.log_scales[::9] += 1.5
    mask = np.zeros((40, 67), np.uint8)          # a mask at another resolution than the image
    mask[5:30, 10:50] = rng.random((25, 40)) < 0.02
    g, r = _compare(gpu, oracle, sc, "mask-tiny", mask=mask)
    live = g.host("tile_active")
    assert 0 < live.sum() < live.size
    _compare(gpu, oracle, sc, "mask-tiny-list", fused_count=True, use_list=True, use_packed=True, mask=mask)
    _compare(gpu, oracle, sc, "mask-none-live", mask=np.zeros((8, 8), np.uint8))
    # huge splats: the wavefront-cooperative key write under a mask
    sc = gpu.scenes.tiny_scene(n=600, width=640, height=400, seed=13)
    sc.log_scales[::7] += 2.5
    sc.means[::50, 2] = -3.6
    mask = (rng.random((400, 640)) < 0.0005).astype(np.uint8)
    g, r = _compare(gpu, oracle, sc, "mask-huge", fused_count=True, use_list=True, mask=mask)
    assert r["counts"].max() > 96


@pytest.mark.parametrize("cfg", ["tiny", "cfg2", "equirect-steps", "fisheye-prism", "tiny-packed", "cfg4-packed", "tiny-ctl", "cfg2-ctl", "tiny-mip"])
def test_fused_projection_bwd_optimizer(gpu, oracle, cfg):
    """K9 fused with Adam (fused_projection_bwd_optimizer_3dgs, fp32 state): both sides are fed the
    SAME screen gradients (the device's), so only the arithmetic of the fused kernel is compared."""
    rng = np.random.default_rng(11)
    if cfg in ("tiny", "tiny-ctl", "tiny-mip"):
        sc = gpu.scenes.tiny_scene(n=900, width=96, height=64, seed=61)
        if cfg == "tiny-mip":      # the antialiased primitive (fused_projection_bwd_optimizer_mip)
            sc.log_scales -= 1.5
            sc.antialiased = True
        sc.means[::4, 2] = -10.0
        sc.log_scales[5] = [-2.0, -4.5, -3.0]
        sc.features_dc[7] = [2.5, -2.2, 0.1]
        sc.quats *= np.linspace(0.5, 2.0, sc.n)[:, None].astype(np.float32)
    elif cfg in ("cfg2", "cfg2-ctl"):
        sc = gpu.scenes.make_scene(2, n=40000, width=480, height=270, parity_variant=True)
    elif cfg == "fisheye-prism":
        sc = _lens_scene(gpu, 1, 2, n=3000, seed=43)
    elif cfg == "tiny-packed":
        sc = gpu.scenes.tiny_scene(n=900, width=96, height=64, seed=61)
        sc.means[::4, 2] = -10.0
    elif cfg == "cfg4-packed":
        sc = gpu.scenes.make_scene(4, n=60000, width=480, height=270, sh_codec=0)   # mostly culled
    else:
        sc = gpu.scenes.make_scene(5, n=30000, width=512, height=256)
    sc.log_scales[11] = [-2.5, -6.5, -6.6]                 # a needle
    sc.log_scales[12] = [-3.0, -3.0, -3.0]                 # ties in the max and min of the scales
    packed = cfg.endswith("packed")
    g = GpuRun(gpu, sc, packed_projection=packed)
    g.projection_fwd(); g.tiles(); g.raster_fwd(); g.raster_bwd()
    vs = {k: g.host(k) for k in ["v_xy", "v_depth", "v_conic", "v_opac", "v_rgb"]}
    aabb = g.host("aabb")
    if packed:   # the packed mode is the plain one renumbered: give the oracle the rows scattered back to splats
        ids = g.host("gaussian_ids")[:g.rows]
        assert 0 < g.rows < sc.n and np.all(np.diff(ids) > 0)
        row_of = np.full(sc.n, -1, np.int32)
        row_of[ids] = np.arange(g.rows, dtype=np.int32)
        full = np.zeros((sc.n, 4), np.float32)
        full[ids] = aabb[:g.rows]
        aabb = full
        for k in vs:
            full = np.zeros((sc.n,) + vs[k].shape[1:], np.float32)
            full[ids] = vs[k][:g.rows]
            vs[k] = full
    P = {k: np.ascontiguousarray(getattr(sc, k), np.float32).copy() for k in oracle.WORLD_KEYS}
    g1 = {k: rng.normal(0, 1e-3, P[k].shape).astype(np.float32) for k in oracle.WORLD_KEYS}
    g2 = {k: rng.uniform(1e-7, 1e-5, P[k].shape).astype(np.float32) for k in oracle.WORLD_KEYS}
    v_in = {"means": rng.normal(0, 1e-3, (sc.n, 3)).astype(np.float32)}
    h = dict(lr_means=1.6e-4, lr_quats=1e-3, lr_scales=5e-3, lr_opacs=5e-2, lr_features_dc=2.5e-3,
             lr_features_sh=1.25e-4, max_gauss_ratio=6.0, scale_regularization_weight=0.01,
             mcmc_opacity_reg_weight=0.01, mcmc_scale_reg_weight=0.01, quat_norm_reg_weight=0.02, sh_reg_weight=0.05)
    if cfg in ("tiny", "cfg4-packed", "fisheye-prism"):   # with the effective-rank regularizer (needles and blobs both occur)
        h.update(erank_reg_weight=0.1, erank_reg_weight_s3=0.01)
    if cfg.endswith("ctl"):   # the colour trust region, with rates at which its clips bind
        h.update(color_trust_linear=1, eps_tr=1e-4, lr_features_dc=2.5e-2, lr_features_sh=1.25e-2)
    steps = rng.integers(1, 400, sc.n).astype(np.int32) if cfg == "equirect-steps" else None
    sa = cfg in ("tiny", "cfg4-packed", "cfg2")   # the scale-agnostic step of the means (the reference's default)
    dP, d1, d2, dscore = g.fused_optimizer(g1, g2, h, step=37, steps=steps, v_in=v_in, scale_agnostic=sa)
    score = oracle.fused_projection_bwd_optimizer(sc, aabb, vs, P, g1, g2, h, step=37, steps=steps, v_in=v_in,
                                                  radii=g.host("radii") if sa else None)
    lrs = dict(means="lr_means", quats="lr_quats", log_scales="lr_scales", opacity_logits="lr_opacs",
               features_dc="lr_features_dc", features_sh="lr_features_sh")
    for k in oracle.WORLD_KEYS:
        # moments: relative to the row's gradient scale; parameters: a fraction of one learning-rate step
        a, b = d1[k].reshape(sc.n, -1).astype(np.float64), g1[k].reshape(sc.n, -1).astype(np.float64)
        assert (np.abs(a - b) <= 1e-3 * np.abs(b) + 1e-4 * (np.abs(b).max(axis=1, keepdims=True) + 1e-12)).all(), ("g1", k)
        a, b = d2[k].reshape(sc.n, -1).astype(np.float64), g2[k].reshape(sc.n, -1).astype(np.float64)
        assert (np.abs(a - b) <= 2e-3 * np.abs(b) + 1e-12).all(), ("g2", k)
        a, b = dP[k].astype(np.float64), P[k].astype(np.float64)
        assert np.abs(a - b).max() <= 0.02 * h[lrs[k]] * 40 + 1e-6, (k, float(np.abs(a - b).max()))
    assert np.allclose(dscore, score, rtol=1e-3, atol=1e-9)
    if cfg.endswith("ctl"):   # the clipped steps themselves: both sides land on the same values, and the clips did bind
        k0 = 0.28209479177387814
        for k in ("features_dc", "features_sh"):
            assert np.abs(dP[k].astype(np.float64) - P[k]).max() <= 3e-5, (k, float(np.abs(dP[k].astype(np.float64) - P[k]).max()))
        opac = 1 / (1 + np.exp(-sc.opacity_logits.astype(np.float64)))
        c_dc = np.maximum(k0 * sc.features_dc.astype(np.float64) + 0.5, (1 / 255.0) ** 2)
        clip = k0 * np.sqrt(4e-4 * c_dc / np.maximum(opac, 1e-12)[:, None])
        moved = np.abs(dP["features_sh"].astype(np.float64) - sc.features_sh)
        assert (moved <= clip[:, None, :] * (1 + 1e-4) + 1e-7).all()
        assert (moved >= clip[:, None, :] * (1 - 1e-3)).mean() > 0.02
    if packed:
        assert np.array_equal(g.host("row_of"), row_of)


@pytest.mark.parametrize("cfg", ["tiny", "tiny-deg1-packed-steps", "cfg3", "tiny-nonsh", "cfg3-nonsh-packed-steps", "tiny-nonsh-ctl"])
def test_fused_optimizer_quantized_sh_state(gpu, oracle, cfg):
    """The fused optimizer at the reference's quantization level 1: SH values as 16-bit codes and their Adam
    moments as 8-bit (u, log_s) cells, both against per-256-splat bounds that are recomputed every step
    (FusedProjectionBwdOptim_kernel.cuh:709-1030). Two consecutive steps against the oracle, both sides fed the
    device's screen gradients; the second step starts from non-zero moments. Codes may differ by one where the
    two sides' gradients differ in the last bit."""
    rng = np.random.default_rng(17)
    S = gpu.scenes
    deg, packed = 3, False
    # "nonsh": also the moments of the five non-SH tensors quantized (16-bit cells), as the reference runs at this level
    ns = oracle.zero_non_sh_state(1) if "nonsh" in cfg else None
    if cfg.startswith("tiny") and "deg1" not in cfg:
        sc = S.tiny_scene(n=700, width=96, height=64, seed=83)        # two full blocks and a partial one
        sc.means[::4, 2] = -10.0
    elif cfg == "tiny-deg1-packed-steps":
        sc = S.tiny_scene(n=1100, width=96, height=64, seed=84)
        sc.means[::3, 2] = -10.0
        deg, packed = 1, True                                          # coefficients above degree 1 are re-encoded as zeros
    else:
        sc = S.make_scene(3, n=30000, width=320, height=192, sh_codec=0)
        packed = "packed" in cfg
    S.apply_sh_codec(sc, 2, bounds_stride=256 * 45)
    h = dict(lr_means=1.6e-4, lr_quats=1e-3, lr_scales=5e-3, lr_opacs=5e-2, lr_features_dc=2.5e-3, lr_features_sh=2.5e-3,
             max_gauss_ratio=6.0, scale_regularization_weight=0.01, mcmc_opacity_reg_weight=0.01, mcmc_scale_reg_weight=0.01,
             quat_norm_reg_weight=0.02, sh_reg_weight=0.05)
    if cfg.endswith("ctl"):
        h.update(color_trust_linear=1, eps_tr=1e-4, lr_features_dc=2.5e-2, lr_features_sh=1.25e-2)
    n, R = sc.n, 45
    nb = (n + 255) // 256
    steps = rng.integers(1, 60, n).astype(np.int32) if "steps" in cfg else None
    q = dict(state_packed=np.zeros(n * R, np.uint16), state_bounds=np.zeros((nb, 4), np.float32),
             value_packed=np.ascontiguousarray(sc.sh_packed).view(np.uint16).copy(),
             value_bounds=np.ascontiguousarray(sc.sh_bounds, np.float32).reshape(nb, 2).copy(), num_sh_buffer=15)
    P = {k: np.ascontiguousarray(getattr(sc, k), np.float32).copy() for k in oracle.WORLD_KEYS[:5]}
    g1 = {k: np.zeros_like(v) for k, v in P.items()}
    g2 = {k: np.zeros_like(v) for k, v in P.items()}
    if ns is not None:
        ns, g1, g2 = oracle.zero_non_sh_state(n), None, None
    sa = "nonsh" in cfg and "cfg3" in cfg    # with the scale-agnostic step of the means
    for t in (1, 2):
        # the scene both sides start this step from
        for k in P:
            setattr(sc, k, P[k].copy())
        sc.sh_packed, sc.sh_bounds = q["value_packed"].copy(), q["value_bounds"].copy()
        g = GpuRun(gpu, sc, sh_degree=deg, packed_projection=packed)
        g.projection_fwd(); g.tiles(); g.raster_fwd(); g.raster_bwd()
        vs = {k: g.host(k) for k in ["v_xy", "v_depth", "v_conic", "v_opac", "v_rgb"]}
        aabb = g.host("aabb")
        if packed:
            ids = g.host("gaussian_ids")[:g.rows]
            full = np.zeros((n, 4), np.float32); full[ids] = aabb[:g.rows]; aabb = full
            for k in vs:
                full = np.zeros((n,) + vs[k].shape[1:], np.float32); full[ids] = vs[k][:g.rows]; vs[k] = full
        dP, d1, d2, dscore, dq = g.fused_optimizer(g1, g2, h, step=t, steps=steps, quant_state=q, non_sh=ns, scale_agnostic=sa)
        oq = {k: (v.copy() if isinstance(v, np.ndarray) else v) for k, v in q.items()}
        oP = {k: v.copy() for k, v in P.items()}
        o1 = None if ns is not None else {k: v.copy() for k, v in g1.items()}
        o2 = None if ns is not None else {k: v.copy() for k, v in g2.items()}
        ons = None if ns is None else dict(packed=[a.copy() for a in ns["packed"]], bounds=[a.copy() for a in ns["bounds"]])
        oracle.fused_projection_bwd_optimizer_q(sc, aabb, vs, oP, oq, o1, o2, h, step=t, steps=steps, sh_degree=deg, non_sh=ons,
                                                radii=g.host("radii") if sa else None)
        if ns is not None:
            dns = g.non_sh_out
            for ti, k in enumerate(oracle.NON_SH_KEYS):
                assert np.allclose(dns["bounds"][ti], ons["bounds"][ti], rtol=1e-4, atol=1e-6), (k, t)
                a, b = dns["packed"][ti].astype(np.int64), ons["packed"][ti].astype(np.int64)
                du, ds = np.abs((a & 65535) - (b & 65535)), np.abs((a >> 16) - (b >> 16))
                # the two sides' gradients agree to rounding, which a 16-bit code resolves: a few steps at most
                assert max(du.max(), ds.max()) <= 24 and max((du > 2).mean(), (ds > 2).mean()) < 0.02, (k, t, int(du.max()), int(ds.max()))
                assert a.any()
            ns = dns
        assert np.allclose(dq["value_bounds"], oq["value_bounds"], rtol=1e-5, atol=1e-8)
        assert np.allclose(dq["state_bounds"], oq["state_bounds"], rtol=1e-4, atol=1e-6)
        for key, width in [("value_packed", 16), ("state_packed", 8)]:
            a, b = dq[key].astype(np.int64), oq[key].astype(np.int64)
            if width == 16:
                d = np.abs(a - b)
                assert d.max() <= 2 and (d > 0).mean() < 0.02, (key, int(d.max()), float((d > 0).mean()))
            else:
                du, ds = np.abs((a & 255) - (b & 255)), np.abs((a >> 8) - (b >> 8))
                assert max(du.max(), ds.max()) <= 1 and max((du > 0).mean(), (ds > 0).mean()) < 0.01, (key, t)
        for k in P:   # the non-SH parameters take the fp32 path
            assert np.abs(dP[k].astype(np.float64) - oP[k]).max() <= 0.02 * 5e-2 * 40 + 1e-6, k
        if deg < 3:   # coefficients above the active degree: zero values, zero moments
            vals = oracle.decode_sh_values(dq, n).reshape(n, 15, 3)
            m1, m2 = oracle.decode_sh_moments(dq, n)
            step = (dq["value_bounds"][:, 1] - dq["value_bounds"][:, 0]).max() / 65535
            assert np.abs(vals[:, deg * (deg + 2):]).max() <= step
            assert not np.any(m2.reshape(n, 15, 3)[:, deg * (deg + 2):])
        # carry the DEVICE's state into the next step
        P, g1, g2, q = dP, d1, d2, dq
    vals0 = oracle.decode_sh_values(dict(q, value_packed=np.ascontiguousarray(sc.sh_packed).view(np.uint16), value_bounds=sc.sh_bounds), n)
    assert np.abs(oracle.decode_sh_values(q, n) - vals0).max() > 1e-4    # the coefficients did move


def _variant_cotangents(sc, seed=1):
    rng = np.random.default_rng(seed)
    h, w = sc.height, sc.width
    return dict(v_dist_rgb=rng.uniform(-1, 1, (h, w, 3)).astype(np.float32),
                v_dist_depth=rng.uniform(-1, 1, (h, w)).astype(np.float32),
                v_median=rng.uniform(-1, 1, (h, w)).astype(np.float32),
                accum_map=rng.uniform(0, 1, (h, w)).astype(np.float32))


@pytest.mark.parametrize("dist_type,median,accum", [(1, False, 0), (2, False, 0), (0, True, 0), (0, False, 1), (0, False, 2),
                                                    (0, False, 3), (2, True, 3), (1, True, 1)])
def test_compositing_variants(gpu, oracle, dist_type, median, accum):
    """Depth distortion (D, RGB_D), median depth and pixel-weight accumulation (max, sum, avg) of the
    compositing forward and backward, alone and combined."""
    sc = gpu.scenes.make_scene(1, n=20000, width=240, height=160, parity_variant=True)
    va = dict(dist_type=dist_type, median=median, accum_mode=accum, **_variant_cotangents(sc))
    _compare(gpu, oracle, sc, f"variant-{dist_type}-{int(median)}-{accum}", fused_count=True, use_list=True, use_packed=True, variant=va)
    sc = gpu.scenes.tiny_scene(n=700, width=96, height=64, seed=9)
    va = dict(dist_type=dist_type, median=median, accum_mode=accum, **_variant_cotangents(sc, 2))
    _compare(gpu, oracle, sc, "variant-tiny", variant=va)


def test_packed_gradient_rows(gpu, oracle):
    """K8 writing one 12-float gradient row per splat and K9 reading it: same gradients, the five
    v_screen arrays untouched."""
    _compare(gpu, oracle, gpu.scenes.tiny_scene(n=700, width=96, height=64, seed=9), "vrows-tiny", use_vrows=True)
    sc = gpu.scenes.make_scene(2, n=50000, width=480, height=270, parity_variant=True)
    _compare(gpu, oracle, sc, "vrows-cfg2", fused_count=True, use_list=True, use_packed=True, use_vrows=True)
    va = dict(dist_type=2, median=False, accum_mode=3, **_variant_cotangents(sc))
    _compare(gpu, oracle, sc, "vrows-variants", fused_count=True, use_list=True, use_packed=True, use_vrows=True, variant=va)
    sc = gpu.scenes.tiny_scene(n=64, width=40, height=24, seed=1)
    sc.means[:, 2] = -10.0
    _compare(gpu, oracle, sc, "vrows-culled", use_vrows=True)
