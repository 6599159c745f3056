"""Variants of the compositing kernels (depth distortion, median depth, per-splat accumulation of a
pixel weight map; src/kernels/raster/RasterizationEval3DFwd_kernel.cuh:143-148,245-307 and
RasterizationEval3DBwd_kernel.cuh:150-172,207-279,433-585), oracle side, pinned against definitions
evaluated in float64 and their finite differences."""
import numpy as np
import pytest

import ref64
from test_oracle_raster import _tile_frags


def _scene(pkg, n=80, w=32, h=32, seed=9):
    sc = pkg.scenes.tiny_scene(n=n, width=w, height=h, seed=seed, big=True)
    return sc


def _cot(sc, seed=1):
    rng = np.random.default_rng(seed)
    h, w = sc.height, sc.width
    return dict(v_dist_rgb=rng.uniform(-1, 1, (h, w, 3)).astype(np.float32),
                v_dist_depth=rng.uniform(-1, 1, (h, w)).astype(np.float32),
                v_median=rng.uniform(-1, 1, (h, w)).astype(np.float32),
                accum_map=rng.uniform(0, 1, (h, w)).astype(np.float32))


@pytest.mark.parametrize("dist_type", [1, 2])
def test_forward_distortion_and_median(pkg, oracle, dist_type):
    sc = _scene(pkg, n=250, w=48, h=40, seed=3)
    r = oracle.pipeline(sc, backward=False, variant=dict(dist_type=dist_type, median=True))
    plain = oracle.pipeline(sc, backward=False)
    f = r["fwd"]
    assert np.array_equal(f["rgb"], plain["fwd"]["rgb"]) and np.array_equal(f["T"], plain["fwd"]["T"])
    assert np.array_equal(f["last_ids"], plain["fwd"]["last_ids"])
    assert (f["median"] > 0).sum() > 100 and (f["median"] == 0).sum() > 10
    bad = 0
    for py in range(sc.height):
        for px in range(sc.width):
            tile = (py // 16) * sc.tile_w + px // 16
            s, fr, _ = _tile_frags(r, sc, tile)
            e = ref64.composite_ex(px + 0.5, py + 0.5, fr, dist_type)
            ok = abs(e["depth"] - f["depth"][py, px]) < 2e-4 * max(1, e["depth"])
            ok &= abs(e["dist_depth"] - f["dist_depth"][py, px]) < 2e-5 + 1e-3 * abs(e["dist_depth"])
            ok &= abs(e["median"] - f["median"][py, px]) < 2e-4 * max(1, e["median"])
            if dist_type == 2:
                ok &= np.abs(e["dist_rgb"] - f["dist_rgb"][py, px]).max() < 2e-5
            bad += not ok
    assert bad <= 2, bad


def _total(sc, r, tiles, cot, dist_type, use_median, override=None):
    v_rgb, v_d, v_T = sc.v_rgb.astype(np.float64), sc.v_depth.astype(np.float64), sc.v_T.astype(np.float64)
    tot = 0.0
    for t, s, fr, g in tiles:
        if override is not None:
            gi, key, k, val = override
            fr = {kk: vv.copy() for kk, vv in fr.items()}
            for j in np.nonzero(g == gi)[0]:
                fr[key].reshape(len(g), -1)[j, k] = val
        ty, tx = divmod(t, sc.tile_w)
        for py in range(ty * 16, min(ty * 16 + 16, sc.height)):
            for px in range(tx * 16, min(tx * 16 + 16, sc.width)):
                e = ref64.composite_ex(px + 0.5, py + 0.5, fr, dist_type)
                tot += float(v_rgb[py, px] @ e["rgb"] + v_d[py, px] * e["depth"] + v_T[py, px] * e["T"])
                if dist_type:
                    tot += float(cot["v_dist_depth"][py, px]) * e["dist_depth"]
                    if dist_type == 2:
                        tot += float(cot["v_dist_rgb"][py, px].astype(np.float64) @ e["dist_rgb"])
                if use_median:
                    tot += float(cot["v_median"][py, px]) * e["median"]
    return tot


@pytest.mark.parametrize("dist_type", [1, 2])
def test_backward_with_distortion_matches_finite_differences(pkg, oracle, dist_type):
    sc = _scene(pkg, n=60, w=32, h=32, seed=9)
    cot = _cot(sc)
    r = oracle.pipeline(sc, variant=dict(dist_type=dist_type, **cot))
    vs, p = r["vscreen"], r["proj"]
    tiles = [(t, *_tile_frags(r, sc, t)) for t in range(sc.tile_w * sc.tile_h)]
    names = [("xy", "v_xy"), ("depth", "v_depth"), ("conic", "v_conic"), ("opac", "v_opac"), ("rgb", "v_rgb")]
    used = np.unique(r["sorted_flat"])
    rng = np.random.default_rng(0)
    for gi in rng.choice(used, size=min(4, used.size), replace=False):
        for key, vname in names:
            base = p[key][gi].astype(np.float64).reshape(-1)
            got = np.asarray(vs[vname][gi], np.float64).reshape(-1)
            fd = np.zeros_like(base)
            for k in range(base.size):
                h = 1e-5 * max(1.0, abs(base[k]))
                fd[k] = (_total(sc, r, tiles, cot, dist_type, False, (gi, key, k, base[k] + h)) -
                         _total(sc, r, tiles, cot, dist_type, False, (gi, key, k, base[k] - h))) / (2 * h)
            scale = vs["abs_terms"][gi].max() + 1e-6
            assert np.abs(got - fd).max() <= 4e-3 * max(np.abs(fd).max(), 1e-3 * scale), (gi, key, got, fd)


def test_median_backward_depth_gradient(pkg, oracle):
    """The depth part of the median gradient is exact (weights f and 1 - f on the two bracketing
    splats). Its opacity part is, by the reference's own statement, partial (the far splat's own
    opacity term is omitted, RasterizationEval3DBwd_kernel.cuh:433-440), so only v_depth is compared with
    finite differences; that the opacity-side gradients change at all is checked separately."""
    sc = _scene(pkg, n=60, w=32, h=32, seed=9)
    sc.v_rgb[:] = 0; sc.v_depth[:] = 0; sc.v_T[:] = 0      # median cotangent only
    cot = _cot(sc)
    r = oracle.pipeline(sc, variant=dict(median=True, **cot))
    vs, p = r["vscreen"], r["proj"]
    tiles = [(t, *_tile_frags(r, sc, t)) for t in range(sc.tile_w * sc.tile_h)]
    used = np.unique(r["sorted_flat"])
    nz = 0
    for gi in used[:12]:
        base = float(p["depth"][gi])
        h = 1e-4 * max(1.0, abs(base))
        fd = (_total(sc, r, tiles, cot, 0, True, (gi, "depth", 0, base + h)) -
              _total(sc, r, tiles, cot, 0, True, (gi, "depth", 0, base - h))) / (2 * h)
        assert abs(vs["v_depth"][gi] - fd) <= 2e-3 * max(abs(fd), 1e-3), (gi, vs["v_depth"][gi], fd)
        nz += abs(fd) > 1e-6
    assert nz >= 3
    assert np.abs(vs["v_opac"]).max() > 0 and not np.any(vs["v_rgb"])


def test_median_backward_is_the_gradient_of_its_surrogate(pkg, oracle):
    """Every part of the median gradient, opacity side included. The reference's backward leaves out the far splat's
    own opacity term on purpose (RasterizationEval3DBwd_kernel.cuh:433-440), so it is not the gradient of the forward;
    it IS the gradient of the forward with d0 = ln(1 - alpha_far) held fixed: z_near + (z_far - z_near)(ln 1/2 - a)/d0,
    a = ln T before the far splat. That surrogate is written out independently in float64 (ref64.median_surrogate) and
    differentiated by central differences with respect to every screen attribute of sampled splats; the oracle's
    v_xy, v_conic, v_opac and v_depth must equal it."""
    sc = _scene(pkg, n=60, w=32, h=32, seed=9)
    sc.v_rgb[:] = 0; sc.v_depth[:] = 0; sc.v_T[:] = 0      # median cotangent only
    cot = _cot(sc)
    r = oracle.pipeline(sc, variant=dict(median=True, **cot))
    vs, p = r["vscreen"], r["proj"]
    tiles = [(t, *_tile_frags(r, sc, t)) for t in range(sc.tile_w * sc.tile_h)]
    plans, n_plans = {}, 0
    for t, s, fr, g in tiles:
        ty, tx = divmod(t, sc.tile_w)
        for py in range(ty * 16, min(ty * 16 + 16, sc.height)):
            for px in range(tx * 16, min(tx * 16 + 16, sc.width)):
                plans[(py, px)] = ref64.median_plan(px + 0.5, py + 0.5, fr)
                n_plans += plans[(py, px)] is not None
    assert n_plans > 100

    def total(override=None):
        tot = 0.0
        for t, s, fr, g in tiles:
            if override is not None:
                gi, key, k, val = override
                if not np.any(g == gi):
                    continue
                fr = {kk: vv.copy() for kk, vv in fr.items()}
                for j in np.nonzero(g == gi)[0]:
                    fr[key].reshape(len(g), -1)[j, k] = val
            ty, tx = divmod(t, sc.tile_w)
            for py in range(ty * 16, min(ty * 16 + 16, sc.height)):
                for px in range(tx * 16, min(tx * 16 + 16, sc.width)):
                    pl = plans[(py, px)]
                    if pl is not None:
                        tot += float(cot["v_median"][py, px]) * ref64.median_surrogate(px + 0.5, py + 0.5, fr, pl)
        return tot

    used = np.unique(r["sorted_flat"])
    rng = np.random.default_rng(2)
    names = [("xy", "v_xy"), ("depth", "v_depth"), ("conic", "v_conic"), ("opac", "v_opac")]
    checked = dict(v_xy=0, v_depth=0, v_conic=0, v_opac=0)
    for gi in rng.choice(used, size=min(8, used.size), replace=False):
        for key, vname in names:
            base = p[key][gi].astype(np.float64).reshape(-1)
            got = np.asarray(vs[vname][gi], np.float64).reshape(-1)
            fd = np.zeros_like(base)
            for k in range(base.size):
                h = 1e-5 * max(1.0, abs(base[k]))
                fd[k] = (total((gi, key, k, base[k] + h)) - total((gi, key, k, base[k] - h))) / (2 * h)
            # float32 kernel arithmetic against float64 differences; terms of both signs add up per splat
            scale = max(np.abs(fd).max(), np.abs(got).max())
            assert np.abs(got - fd).max() <= 3e-3 * scale + 1e-7, (gi, key, got, fd)
            checked[vname] += int(np.abs(fd).max() > 1e-6)
    assert min(checked.values()) >= 2, checked     # every kind of gradient was really exercised
    assert not np.any(vs["v_rgb"])
    # and the surrogate is not the forward: differences of the forward's own median disagree with the oracle on the
    # opacity of some sampled splat (the omitted term), so a backward that "fixed" the omission would fail above
    differs = 0
    for gi in rng.choice(used, size=min(8, used.size), replace=False):
        base = float(p["opac"][gi])
        h = 1e-5
        fd_true = (_total(sc, r, tiles, cot, 0, True, (gi, "opac", 0, base + h)) -
                   _total(sc, r, tiles, cot, 0, True, (gi, "opac", 0, base - h))) / (2 * h)
        differs += abs(fd_true - float(vs["v_opac"][gi])) > 0.05 * max(abs(fd_true), abs(float(vs["v_opac"][gi])), 1e-6)
    assert differs >= 2, differs


@pytest.mark.parametrize("mode", [1, 2, 3])
def test_accumulated_pixel_weights(pkg, oracle, mode):
    """accum_weight[splat] = max / sum over pixels of map[pixel] * alpha * T_before (Avg: also the
    sum of alpha * T_before as denominator)."""
    sc = _scene(pkg, n=120, w=48, h=32, seed=4)
    cot = _cot(sc)
    r = oracle.pipeline(sc, variant=dict(accum_mode=mode, accum_map=cot["accum_map"]))
    got = r["vscreen"]["accum_weight"]
    num, den = np.zeros(sc.n), np.zeros(sc.n)
    for py in range(sc.height):
        for px in range(sc.width):
            tile = (py // 16) * sc.tile_w + px // 16
            s, fr, g = _tile_frags(r, sc, tile)
            e = ref64.composite_ex(px + 0.5, py + 0.5, fr)
            for w, k in zip(e["w"], e["ks"]):
                v = float(cot["accum_map"][py, px]) * w
                if mode == 1:
                    num[g[k]] = max(num[g[k]], v)
                else:
                    num[g[k]] += v
                    den[g[k]] += w
    assert np.allclose(got[:sc.n], num, rtol=2e-4, atol=1e-6)
    if mode == 3:
        assert np.allclose(got[sc.n:], den, rtol=2e-4, atol=1e-6)
    assert (num > 0).sum() > 20
