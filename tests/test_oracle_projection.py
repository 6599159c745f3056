"""Pins the oracle's projection + SH forward (K1) and backward (K9) against independent float64
restatements, closed forms and finite differences."""
import math

import numpy as np
import pytest

import ref64


def _scene(pkg, model, n=400, seed=11):
    S = pkg.scenes
    sc = S.tiny_scene(n=n, width=256, height=192, seed=seed, camera_model=model, big=False)
    if model == S.CAM_PINHOLE:
        # a rotated, translated camera (0.2 rad about y, as src/backend/tests/render_parity.cpp:113-118)
        c, s = math.cos(0.2), math.sin(0.2)
        sc.viewmat = np.array([[c, 0, s, 0.1], [0, 1, 0, -0.05], [-s, 0, c, 4], [0, 0, 0, 1]], np.float32)
    else:
        c, s = math.cos(0.3), math.sin(0.3)
        sc.viewmat = np.array([[c, 0, s, 0.2], [0, 1, 0, 0.1], [-s, 0, c, -0.1], [0, 0, 0, 1]], np.float32)
    return sc


@pytest.mark.parametrize("model", [0, 3])
def test_forward_matches_float64_matrix_form(pkg, oracle, model):
    sc = _scene(pkg, model)
    o = oracle.projection_fwd(sc)
    vis = o["aabb"][:, 2] > o["aabb"][:, 0]
    assert vis.sum() > 50
    for g in np.nonzero(vis)[0][:200]:
        r = ref64.project(sc.means[g].astype(np.float64), sc.quats[g].astype(np.float64),
                          sc.log_scales[g].astype(np.float64), float(sc.opacity_logits[g]),
                          sc.viewmat, sc.intrins, sc.width, model)
        np.testing.assert_allclose(o["xy"][g], r["xy"], rtol=2e-5, atol=2e-3)
        np.testing.assert_allclose(o["depth"][g], r["depth"], rtol=2e-6)
        np.testing.assert_allclose(o["conic"][g], r["conic"], rtol=3e-4, atol=1e-6)
        np.testing.assert_allclose(o["opac"][g], r["opac"], rtol=1e-6)
        col = ref64.sh_color(sc.means[g].astype(np.float64), sc.viewmat,
                             sc.features_dc[g].astype(np.float64), sc.features_sh[g].astype(np.float64))
        np.testing.assert_allclose(o["rgb"][g], col, rtol=1e-5, atol=2e-6)
        # extents: 3.33 sigma or the opacity-aware bound, whichever is smaller
        ext = min(3.33, math.sqrt(2 * math.log(r["opac"] * 255)))
        rx, ry = ext * math.sqrt(r["cov2d"][0, 0]), ext * math.sqrt(r["cov2d"][1, 1])
        want = np.clip([r["xy"][0] - rx, r["xy"][1] - ry, r["xy"][0] + rx, r["xy"][1] + ry],
                       0, [sc.width - 1, sc.height - 1, sc.width - 1, sc.height - 1])
        np.testing.assert_allclose(o["aabb"][g], want, rtol=1e-4, atol=5e-3)
        sd = r["pc"][2] if model == 0 else float(r["pc"] @ r["pc"])
        np.testing.assert_allclose(o["sort_depth"][g], sd, rtol=1e-5)


def test_closed_form_on_axis_isotropic(pkg, oracle):
    """An isotropic splat on the optical axis: mean2d = (cx, cy), cov2d = (f s / z)^2 I + 0.3 I."""
    S = pkg.scenes
    sc = S.tiny_scene(n=4, width=200, height=100, seed=3)
    sc.viewmat = np.eye(4, dtype=np.float32)
    sc.means[:] = [[0, 0, 5], [0, 0, 2], [0, 0, 9], [0, 0, -1]]
    sc.log_scales[:] = math.log(0.05)
    sc.quats[:] = [0.5, 0.5, -0.5, 0.5]
    sc.opacity_logits[:] = 2.0
    sc.features_sh[:] = 0
    sc.features_dc[:] = [[1.0, -0.5, 0.0]]
    o = oracle.projection_fwd(sc)
    f = float(sc.intrins[0])
    for g, z in enumerate([5.0, 2.0, 9.0]):
        var = (f * 0.05 / z) ** 2 + 0.3
        np.testing.assert_allclose(o["xy"][g], [100, 50], atol=1e-4)
        np.testing.assert_allclose(o["conic"][g], [1 / var, 0, 1 / var], rtol=1e-5, atol=1e-7)
        np.testing.assert_allclose(o["depth"][g], z, rtol=1e-6)
        np.testing.assert_allclose(o["sort_depth"][g], z, rtol=1e-6)
        # degree-0 colour: 0.5 + 0.2820948 dc, clamped at 0
        np.testing.assert_allclose(o["rgb"][g], np.maximum(0.5 + 0.28209479 * sc.features_dc[g], 0), rtol=1e-6)
    assert np.all(o["aabb"][3] == 0) and o["sort_depth"][3] == 0   # behind the camera: culled
    assert o["visible"] == 3


def test_culls(pkg, oracle):
    S = pkg.scenes
    sc = S.tiny_scene(n=5, width=128, height=128, seed=5)
    sc.viewmat = np.eye(4, dtype=np.float32)
    sc.means[:] = [[0, 0, 3], [0, 0, 3], [40, 0, 3], [0, 0, 3], [0, 0, 3]]
    sc.log_scales[:] = math.log(0.1)
    sc.opacity_logits[:] = [3.0, -6.0, 3.0, 3.0, 3.0]   # #1: opacity < 1/255
    sc.log_scales[3] = math.log(1e-6)                    # tiny but blurred: still visible
    o = oracle.projection_fwd(sc)
    vis = o["aabb"][:, 2] > o["aabb"][:, 0]
    assert vis.tolist() == [True, False, False, True, True]
    # radii receive the angular radius of visible splats only
    assert (o["radii"] > 0).tolist() == vis.tolist()


def test_sh_basis_vs_textbook(pkg, oracle):
    """Feed one-hot coefficients: the colour is 0.5 + Y_j(dir), Y_j from the textbook forms."""
    S = pkg.scenes
    rng = np.random.default_rng(4)
    n = 15 * 6
    sc = S.tiny_scene(n=n, width=128, height=128, seed=2)
    sc.viewmat = np.eye(4, dtype=np.float32)
    sc.viewmat[:3, 3] = [0.3, -0.2, 6.0]
    sc.means[:] = rng.uniform(-1, 1, (n, 3))
    sc.log_scales[:] = math.log(0.05)
    sc.opacity_logits[:] = 3
    sc.features_dc[:] = 0
    sc.features_sh[:] = 0
    for g in range(n):
        sc.features_sh[g, g % 15, :] = [1.0, 0.5, -0.25]
    o = oracle.projection_fwd(sc)
    for g in range(n):
        d = sc.means[g].astype(np.float64) + sc.viewmat[:3, :3].astype(np.float64).T @ sc.viewmat[:3, 3]
        Y = ref64.real_sh_deg3(d)[g % 15]
        np.testing.assert_allclose(o["rgb"][g], np.maximum(0.5 + Y * np.array([1.0, 0.5, -0.25]), 0),
                                   atol=3e-6)


@pytest.mark.parametrize("codec", [1, 2, 3])
@pytest.mark.parametrize("stride", [256, 0])
def test_quantized_sh_equals_fp32_on_decoded(pkg, oracle, codec, stride):
    """Quantized path == fp32 path fed the dequantized coefficients, bit for bit; endpoints exact."""
    S = pkg.scenes
    if codec == 3 and stride == 0:
        pytest.skip("the int8 codec has no bounds table")
    sc = S.tiny_scene(n=700, width=128, height=96, seed=9, big=False)
    a = oracle.projection_fwd(sc)
    S.apply_sh_codec(sc, codec, bounds_stride=stride)
    q = oracle.projection_fwd(sc)            # decodes inside
    codec_saved = sc.sh_codec
    sc.sh_codec = S.SH_F32                    # same scene, fp32 path on the decoded values
    f = oracle.projection_fwd(sc)
    sc.sh_codec = codec_saved
    assert np.array_equal(q["rgb"], f["rgb"])
    assert np.abs(q["rgb"] - a["rgb"]).max() < (0.02 if codec != 2 else 2e-4)
    if codec in (1, 2):
        qmax = 255 if codec == 1 else 65535
        flat = sc.features_sh.reshape(-1)
        st = stride if stride else 256 * 45
        lo_idx = np.nonzero(sc.sh_packed == 0)[0]
        hi_idx = np.nonzero(sc.sh_packed == qmax)[0]
        assert np.array_equal(flat[lo_idx], sc.sh_bounds[lo_idx // st, 0])
        # lo + (hi - lo) * (qmax * (1/qmax)) reproduces hi only up to float rounding
        np.testing.assert_allclose(flat[hi_idx], sc.sh_bounds[hi_idx // st, 1], rtol=3e-7, atol=1e-9)


def _loss64(sc, g, model, v, mean, quat, ls, logit, dc, sh):
    r = ref64.project(mean, quat, ls, logit, sc.viewmat, sc.intrins, sc.width, model)
    col = ref64.sh_color(mean, sc.viewmat, dc, sh)
    f64 = lambda a: np.asarray(a, np.float64)   # keep the whole loss in float64
    return float(f64(v["v_xy"][g]) @ r["xy"] + f64(v["v_depth"][g]) * r["depth"]
                 + f64(v["v_conic"][g]) @ r["conic"] + f64(v["v_opac"][g]) * r["opac"]
                 + f64(v["v_rgb"][g]) @ col)


@pytest.mark.parametrize("model", [0, 3])
def test_backward_matches_finite_differences(pkg, oracle, model):
    sc = _scene(pkg, model, n=120, seed=21)
    rng = np.random.default_rng(7)
    o = oracle.projection_fwd(sc)
    n = sc.n
    v = dict(v_xy=rng.normal(0, 1, (n, 2)).astype(np.float32), v_depth=rng.normal(0, 1, n).astype(np.float32),
             v_conic=rng.normal(0, 1, (n, 3)).astype(np.float32), v_opac=rng.normal(0, 1, n).astype(np.float32),
             v_rgb=rng.normal(0, 1, (n, 3)).astype(np.float32))
    g_or = oracle.projection_bwd(sc, o["aabb"], v)
    vis = np.nonzero(o["aabb"][:, 2] > o["aabb"][:, 0])[0]
    assert len(vis) > 30
    checked = 0
    for g in vis[:40]:
        args = [sc.means[g].astype(np.float64), sc.quats[g].astype(np.float64),
                sc.log_scales[g].astype(np.float64), np.array([float(sc.opacity_logits[g])]),
                sc.features_dc[g].astype(np.float64), sc.features_sh[g].astype(np.float64)]
        names = ["v_means", "v_quats", "v_scales", "v_opacities", "v_dc", "v_sh"]

        def L(a):
            return _loss64(sc, g, model, v, a[0], a[1], a[2], float(a[3][0]), a[4], a[5])
        for ai, name in enumerate(names):
            got = np.asarray(g_or[name][g], np.float64).reshape(-1)
            fd = np.zeros_like(got)
            base = args[ai].reshape(-1)
            for k in range(base.size):
                h = 1e-6 * max(1.0, abs(base[k]))
                ap = [x.copy() for x in args]
                am = [x.copy() for x in args]
                ap[ai].reshape(-1)[k] += h
                am[ai].reshape(-1)[k] -= h
                fd[k] = (L(ap) - L(am)) / (2 * h)
            scale = np.abs(fd).max() + 1e-6
            assert np.abs(got - fd).max() <= 2e-3 * scale, (g, name, got, fd)
        checked += 1
    assert checked >= 30
    # culled splats receive nothing
    cull = np.nonzero(~(o["aabb"][:, 2] > o["aabb"][:, 0]))[0]
    for name in ["v_means", "v_quats", "v_scales", "v_opacities", "v_dc", "v_sh"]:
        assert not np.any(g_or[name][cull])


def test_backward_jacobian_clamp_routes_to_bound(pkg, oracle):
    """A splat far off-axis has its J[.,2] entries clamped (src/shaders/primitive_3dgs.slang:89-95);
    the clamp bound depends on z, and finite differences of the clamped forward see that."""
    S = pkg.scenes
    sc = S.tiny_scene(n=2, width=64, height=64, seed=1)
    sc.viewmat = np.eye(4, dtype=np.float32)
    sc.means[:] = [[1.05, 0.9, 1.0], [-1.0, -0.95, 1.0]]    # projects at the image border region
    sc.log_scales[:] = math.log(0.3)
    sc.opacity_logits[:] = 2.0
    o = oracle.projection_fwd(sc)
    assert np.all(o["aabb"][:, 2] > o["aabb"][:, 0])
    # confirm the clamp is active for these inputs
    for g in range(2):
        x, y, z = sc.means[g]
        f, cx = float(sc.intrins[0]), float(sc.intrins[2])
        lim_pos, lim_neg = 64 + 0.3 * 32, 0.3 * 32
        j02 = -f * x / z ** 2
        assert j02 < -(lim_pos - cx) / z or j02 > (lim_neg + cx) / z
    rng = np.random.default_rng(3)
    n = 2
    v = dict(v_xy=rng.normal(0, 1, (n, 2)).astype(np.float32), v_depth=rng.normal(0, 1, n).astype(np.float32),
             v_conic=rng.normal(0, 1, (n, 3)).astype(np.float32), v_opac=rng.normal(0, 1, n).astype(np.float32),
             v_rgb=np.zeros((n, 3), np.float32))
    g_or = oracle.projection_bwd(sc, o["aabb"], v)
    for g in range(2):
        base = sc.means[g].astype(np.float64)
        fd = np.zeros(3)
        for k in range(3):
            h = 1e-6
            p, m = base.copy(), base.copy()
            p[k] += h
            m[k] -= h
            a = [sc.quats[g].astype(np.float64), sc.log_scales[g].astype(np.float64), float(sc.opacity_logits[g]),
                 sc.features_dc[g].astype(np.float64), sc.features_sh[g].astype(np.float64)]
            fd[k] = (_loss64(sc, g, 0, v, p, *a) - _loss64(sc, g, 0, v, m, *a)) / (2 * h)
        assert np.abs(g_or["v_means"][g] - fd).max() <= 2e-3 * (np.abs(fd).max() + 1e-6)


def test_sh_clamp_mask_and_filters(pkg, oracle):
    """Colour channels clamped at zero pass no gradient (src/shaders/harmonics.slang:1103)."""
    S = pkg.scenes
    sc = S.tiny_scene(n=3, width=64, height=64, seed=1)
    sc.viewmat = np.eye(4, dtype=np.float32)
    sc.viewmat[2, 3] = 4
    sc.means[:] = 0
    sc.log_scales[:] = math.log(0.1)
    sc.opacity_logits[:] = 2
    sc.features_sh[:] = 0
    sc.features_dc[:] = [[-5, 1, 1], [1, -5, 1], [1, 1, 1]]
    o = oracle.projection_fwd(sc)
    assert o["rgb"][0, 0] == 0 and o["rgb"][1, 1] == 0
    v = dict(v_xy=np.zeros((3, 2), np.float32), v_depth=np.zeros(3, np.float32),
             v_conic=np.zeros((3, 3), np.float32), v_opac=np.zeros(3, np.float32),
             v_rgb=np.ones((3, 3), np.float32))
    g = oracle.projection_bwd(sc, o["aabb"], v)
    c0 = np.float32(0.2820947917738781)
    np.testing.assert_allclose(g["v_dc"], [[0, c0, c0], [c0, 0, c0], [c0, c0, c0]], rtol=1e-7)
    assert np.all(g["v_sh"][0, :, 0] == 0) and np.any(g["v_sh"][0, :, 1] != 0)
