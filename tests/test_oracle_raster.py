"""Pins the oracle's compositing forward (K7) and backward (K8) against a brute-force float64
per-pixel restatement and its finite differences."""
import numpy as np
import pytest

import ref64


def _run(pkg, oracle, n=250, w=48, h=40, seed=3, big=True):
    sc = pkg.scenes.tiny_scene(n=n, width=w, height=h, seed=seed, big=big)
    return sc, oracle.pipeline(sc, backward=True)


def _tile_frags(r, sc, tile):
    offs, flat = r["offsets"], r["sorted_flat"]
    s = offs[tile]
    e = flat.size if tile == sc.tile_w * sc.tile_h - 1 else offs[tile + 1]
    g = flat[s:e]
    p = r["proj"]
    return s, dict(xy=p["xy"][g].astype(np.float64), conic=p["conic"][g].astype(np.float64),
                   opac=p["opac"][g].astype(np.float64), rgb=p["rgb"][g].astype(np.float64),
                   depth=p["depth"][g].astype(np.float64)), g


def test_forward_matches_bruteforce(pkg, oracle):
    """Untiled float64 compositing over each tile's sorted list equals the tiled result. The 8x8
    footprint cull only drops splats whose alpha is below 1/255 anyway, so no cull is applied in
    the brute force; pixels where the two differ by rounding of that boundary are counted."""
    sc, r = _run(pkg, oracle)
    f = r["fwd"]
    assert 0.02 < f["T"].mean() < 0.9 and (f["T"] < 1e-3).sum() > 10   # both regimes present
    bad = 0
    for py in range(sc.height):
        for px in range(sc.width):
            tile = (py // 16) * sc.tile_w + px // 16
            s, fr, _ = _tile_frags(r, sc, tile)
            rgb, d, T, last = ref64.composite(px + 0.5, py + 0.5, fr)
            ok = (np.abs(rgb - f["rgb"][py, px]).max() < 2e-5 and abs(T - f["T"][py, px]) < 2e-6
                  and abs(d - f["depth"][py, px]) < 1e-4 * max(1, d))
            if T < 1.0:
                ok = ok and (s + last == f["last_ids"][py, px])
            bad += not ok
    assert bad <= 2, bad
    assert np.all((f["T"] >= 0) & (f["T"] <= 1))
    empty = f["T"] == 1.0
    assert not np.any(f["rgb"][empty]) and not np.any(f["last_ids"][empty])


def test_forward_no_splats(pkg, oracle):
    sc = pkg.scenes.tiny_scene(n=5, width=40, height=24, seed=1)
    sc.means[:, 2] = -10   # all behind the camera
    r = oracle.pipeline(sc, backward=True)
    assert r["isect_ids"].size == 0 and not np.any(r["offsets"])
    assert np.all(r["fwd"]["T"] == 1) and not np.any(r["fwd"]["rgb"]) and not np.any(r["fwd"]["depth"])
    for k, v in r["grads"].items():
        assert not np.any(v), k


def test_done_pixel_drops_the_crossing_splat(pkg, oracle):
    """When T(1-alpha) <= 1e-4 the pixel stops WITHOUT adding that splat
    (src/kernels/raster/RasterizationEval3DFwd_kernel.cuh:264-282); alpha is capped at 0.999."""
    S = pkg.scenes
    sc = S.tiny_scene(n=3, width=16, height=16, seed=1)
    sc.viewmat = np.eye(4, dtype=np.float32)
    sc.means[:] = [[0, 0, 1.0], [0, 0, 2.0], [0, 0, 3.0]]
    sc.log_scales[:] = 4.0             # huge: alpha ~ opacity everywhere
    sc.opacity_logits[:] = 20.0        # opacity 1 -> alpha capped at 0.999
    sc.features_sh[:] = 0
    sc.features_dc[:] = [[1, 0, 0], [0, 1, 0], [0, 0, 1]]
    r = oracle.pipeline(sc, backward=False)
    f = r["fwd"]
    # T: 1 -> 1e-3 -> (1e-6 <= 1e-4: stop). Only the first splat is composited.
    np.testing.assert_allclose(f["T"], 1 - 0.999, rtol=1e-3)
    assert np.all(f["last_ids"] == 0)
    c0 = 0.5 + 0.28209479
    np.testing.assert_allclose(f["rgb"][8, 8], [0.999 * c0, 0.999 * 0.5, 0.999 * 0.5], rtol=1e-5)
    np.testing.assert_allclose(f["depth"], 1.0, rtol=1e-5)


def _loss(fr, px, py, vr, vd, vT):
    rgb, d, T, _ = ref64.composite(px, py, fr)
    return float(vr @ rgb + vd * d + vT * T)


def test_backward_matches_finite_differences(pkg, oracle):
    sc, r = _run(pkg, oracle, n=60, w=32, h=32, seed=9)
    vs = r["vscreen"]
    p = r["proj"]
    names = [("xy", "v_xy"), ("depth", "v_depth"), ("conic", "v_conic"), ("opac", "v_opac"), ("rgb", "v_rgb")]
    # total loss = sum over pixels; differentiate w.r.t. the screen rows of a few splats
    tiles = [(t, *_tile_frags(r, sc, t)) for t in range(sc.tile_w * sc.tile_h)]
    v_rgb, v_d, v_T = sc.v_rgb.astype(np.float64), sc.v_depth.astype(np.float64), sc.v_T.astype(np.float64)

    def total(override=None):
        tot = 0.0
        for t, s, fr, g in tiles:
            if override is not None:
                gi, key, k, val = override
                hit = np.nonzero(g == gi)[0]
                if hit.size == 0 and key is not None:
                    pass
                fr = {kk: vv.copy() for kk, vv in fr.items()}
                for j in hit:
                    fr[key].reshape(len(g), -1)[j, k] = val
            ty, tx = divmod(t, sc.tile_w)
            for py in range(ty * 16, min(ty * 16 + 16, sc.height)):
                for px in range(tx * 16, min(tx * 16 + 16, sc.width)):
                    tot += _loss(fr, px + 0.5, py + 0.5, v_rgb[py, px], v_d[py, px], v_T[py, px])
        return tot

    used = np.unique(r["sorted_flat"])
    rng = np.random.default_rng(0)
    checked = 0
    for gi in rng.choice(used, size=min(6, used.size), replace=False):
        for key, vname in names:
            base = p[key][gi].astype(np.float64).reshape(-1)
            got = np.asarray(vs[vname][gi], np.float64).reshape(-1)
            fd = np.zeros_like(base)
            for k in range(base.size):
                h = 1e-5 * max(1.0, abs(base[k]))
                fd[k] = (total((gi, key, k, base[k] + h)) - total((gi, key, k, base[k] - h))) / (2 * h)
            scale = r["vscreen"]["abs_terms"][gi].max() + 1e-6
            assert np.abs(got - fd).max() <= 3e-3 * max(np.abs(fd).max(), 1e-3 * scale), (gi, key, got, fd)
            checked += 1
    assert checked >= 20


def test_backward_undo_recovers_unit_transmittance(pkg, oracle):
    """Undoing every contributing splat from T_final returns to T = 1: replay the recursion."""
    sc, r = _run(pkg, oracle, n=200, w=32, h=32, seed=2)
    f, p = r["fwd"], r["proj"]
    for (py, px) in [(3, 4), (17, 20), (30, 9), (12, 12)]:
        tile = (py // 16) * sc.tile_w + px // 16
        s, fr, g = _tile_frags(r, sc, tile)
        T = float(f["T"][py, px])
        last = int(f["last_ids"][py, px])
        for k in range(last - s, -1, -1):
            dx, dy = fr["xy"][k, 0] - (px + 0.5), fr["xy"][k, 1] - (py + 0.5)
            a, b, c = fr["conic"][k]
            sig = 0.5 * (a * dx * dx + c * dy * dy) + b * dx * dy
            al = min(0.999, fr["opac"][k] * np.exp(-sig))
            if sig < 0 or al <= 1 / 255:
                continue
            T = T / (1 - al)
        assert abs(T - 1.0) < 1e-4


def test_backward_is_idempotent_and_accumulates(pkg, oracle):
    sc, r = _run(pkg, oracle, n=150, w=32, h=32, seed=6)
    p, f = r["proj"], r["fwd"]
    a = oracle.raster_bwd(sc.n, p, sc.width, sc.height, r["offsets"], r["sorted_flat"], f,
                          sc.v_rgb, sc.v_depth, sc.v_T)
    for k in ["v_xy", "v_depth", "v_conic", "v_opac", "v_rgb"]:
        assert np.array_equal(a[k], r["vscreen"][k])
