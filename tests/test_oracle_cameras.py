"""Pins the oracle's FISHEYE / EQUISOLID cameras and the lens-distortion tiers (every pair of
src/kernels/projection/CameraVariants.cuh:11-22 beyond PINHOLE/None and EQUIRECTANGULAR) against
closed forms and an independent float64 restatement whose Jacobian comes from complex-step
differentiation, and the backward against finite differences of that restatement."""
import dataclasses
import math

import numpy as np
import pytest

import ref64

PAIRS = [(0, 1), (0, 2), (0, 3), (1, 0), (1, 1), (1, 2), (2, 0), (2, 1), (2, 2)]


def _scene(pkg, model, tier, n=500, seed=17):
    S = pkg.scenes
    sc = S.tiny_scene(n=n, width=256, height=192, seed=seed, camera_model=model, big=False)
    if model == S.CAM_PINHOLE:
        c, s = math.cos(0.2), math.sin(0.2)
        sc.viewmat = np.array([[c, 0, s, 0.1], [0, 1, 0, -0.05], [-s, 0, c, 3.0], [0, 0, 0, 1]], np.float32)
        sc.intrins = np.array([150.0, 160.0, 128.0, 96.0], np.float32)    # wide: |x/z| up to ~0.6
    else:
        c, s = math.cos(0.3), math.sin(0.3)
        sc.viewmat = np.array([[c, 0, s, 0.2], [0, 1, 0, 0.1], [-s, 0, c, -0.1], [0, 0, 0, 1]], np.float32)
        sc.intrins = np.array([256 / math.pi, 250 / math.pi, 130.0, 94.0], np.float32)
    return S.with_lens(sc, tier)


def _ref(sc, g):
    return ref64.project(sc.means[g].astype(np.float64), sc.quats[g].astype(np.float64),
                         sc.log_scales[g].astype(np.float64), float(sc.opacity_logits[g]), sc.viewmat, sc.intrins,
                         sc.width, sc.camera_model, tier=sc.distortion, coeffs=sc.dist_coeffs)


@pytest.mark.parametrize("model,tier", PAIRS)
def test_forward_matches_float64(pkg, oracle, model, tier):
    sc = _scene(pkg, model, tier)
    o = oracle.projection_fwd(sc)
    vis = o["aabb"][:, 2] > o["aabb"][:, 0]
    assert vis.sum() > 60
    for g in np.nonzero(vis)[0][:150]:
        r = _ref(sc, g)
        np.testing.assert_allclose(o["xy"][g], r["xy"], rtol=2e-5, atol=3e-3)
        np.testing.assert_allclose(o["depth"][g], r["depth"], rtol=2e-6)
        np.testing.assert_allclose(o["conic"][g], r["conic"], rtol=1e-3, atol=2e-6)
        ext = min(3.33, math.sqrt(2 * math.log(r["opac"] * 255)))
        rx, ry = ext * math.sqrt(r["cov2d"][0, 0]), ext * math.sqrt(r["cov2d"][1, 1])
        want = np.clip([r["xy"][0] - rx, r["xy"][1] - ry, r["xy"][0] + rx, r["xy"][1] + ry],
                       0, [sc.width - 1, sc.height - 1, sc.width - 1, sc.height - 1])
        np.testing.assert_allclose(o["aabb"][g], want, rtol=2e-4, atol=1e-2)
        x, y, z = r["pc"]
        sd = z if model == 0 else z ** 4 + (x * x + y * y) ** 2 / 512.0    # get_sorting_depth, projection_utils.slang:1012-1029
        np.testing.assert_allclose(o["sort_depth"][g], sd, rtol=2e-5)
        assert r.get("lens_valid", True)
        if model != 0 and z < 0:
            assert r["centre_weight"] <= 1 / 255 + 1e-6


@pytest.mark.parametrize("model,tier", PAIRS)
def test_visibility_follows_the_lens_checks(pkg, oracle, model, tier):
    """A splat is dropped exactly when one of the reference's tests says so: behind the pinhole, the lens map
    not locally invertible (is_valid_distortion), behind a wide lens yet visible at the centre, too faint,
    or outside the image. Cases within a hair of a threshold are left out."""
    sc = _scene(pkg, model, tier, n=700, seed=23)
    if tier:   # stronger lens, so that the validity test bites inside the field of view
        sc.dist_coeffs = (sc.dist_coeffs * np.float32(-10.0 if model == 0 else 8.0)).astype(np.float32)
    if model == 0:
        sc.viewmat[2, 3] = 2.2   # closer: |x/z| up to about 0.8
    o = oracle.projection_fwd(sc)
    vis = o["aabb"][:, 2] > o["aabb"][:, 0]
    n_lens_culled = n_checked = 0
    for g in range(sc.n):
        pc = sc.viewmat[:3, :3].astype(np.float64) @ sc.means[g] + sc.viewmat[:3, 3]
        if model == 0 and pc[2] <= 0:
            assert not vis[g]
            continue
        r = _ref(sc, g)
        jd = r.get("lens_jdet", 1.0)
        if min(abs(jd - 0.25), abs(jd - 4.0)) < 1e-3:
            continue
        if not r.get("lens_valid", True):
            assert not vis[g]
            n_lens_culled += 1
            continue
        if model != 0 and pc[2] < 0:
            if abs(r["centre_weight"] - 1 / 255) < 1e-5:
                continue
            if r["centre_weight"] > 1 / 255:
                assert not vis[g]
                continue
        ext = min(3.33, math.sqrt(2 * math.log(max(r["opac"] * 255, 1.0))))
        rx, ry = ext * math.sqrt(r["cov2d"][0, 0]), ext * math.sqrt(r["cov2d"][1, 1])
        lo = [r["xy"][0] - rx, r["xy"][1] - ry]
        hi = [r["xy"][0] + rx, r["xy"][1] + ry]
        margins = [hi[0], hi[1], sc.width - lo[0], sc.height - lo[1]]
        if min(abs(m) for m in margins) < 1e-2 or abs(r["opac"] - 1 / 255) < 1e-6:
            continue
        # the kernel also wants the extents, clamped to the pixel grid, to keep some area
        # (src/kernels/projection/ProjectionFwd_kernel.cuh:102)
        ex = np.clip(hi[0], 0, sc.width - 1) - np.clip(lo[0], 0, sc.width - 1)
        ey = np.clip(hi[1], 0, sc.height - 1) - np.clip(lo[1], 0, sc.height - 1)
        if min(abs(ex - 1e-3), abs(ey - 1e-3)) < 1e-2:
            continue
        inside = min(margins) > 0 and r["opac"] >= 1 / 255 and ex > 1e-3 and ey > 1e-3
        assert bool(vis[g]) == inside, (g, margins, r["opac"])
        n_checked += 1
    assert n_checked > 120
    if tier:
        assert n_lens_culled > 0


def test_closed_forms(pkg, oracle):
    """Equidistant: pixel radius = f * theta. Equisolid: f * 2 sin(theta / 2). On the axis both act as a
    perspective camera of focal length f / z. Radial OpenCV distortion on a pinhole: u (1 + k1 u^2)."""
    S = pkg.scenes
    for model in (1, 2):
        sc = S.tiny_scene(n=4, width=400, height=300, seed=3, camera_model=model)
        sc.viewmat = np.eye(4, dtype=np.float32)
        sc.intrins = np.array([100.0, 100.0, 200.0, 150.0], np.float32)
        th = math.radians(60.0)
        sc.means[:] = [[0, 0, 5], [3 * math.sin(th), 0, 3 * math.cos(th)], [0, -2 * math.sin(th), 2 * math.cos(th)], [0, 0, 2]]
        sc.log_scales[:] = math.log(0.05)
        sc.quats[:] = [0.5, 0.5, -0.5, 0.5]
        sc.opacity_logits[:] = 2.0
        o = oracle.projection_fwd(sc)
        rad = th if model == 1 else 2 * math.sin(th / 2)
        np.testing.assert_allclose(o["xy"][0], [200, 150], atol=1e-4)
        np.testing.assert_allclose(o["xy"][1], [200 + 100 * rad, 150], rtol=2e-6)
        np.testing.assert_allclose(o["xy"][2], [200, 150 - 100 * rad], rtol=2e-6)
        for g, z in [(0, 5.0), (3, 2.0)]:
            var = (100 * 0.05 / z) ** 2 + 0.3
            np.testing.assert_allclose(o["conic"][g], [1 / var, 0, 1 / var], rtol=1e-5, atol=1e-7)
        # off axis the radial and tangential magnifications are d(rad)/d(theta) / |p| and rad / (|p| sin theta)
        m_rad = (1.0 if model == 1 else math.cos(th / 2)) / 3.0
        m_tan = rad / (3.0 * math.sin(th))
        vx, vy = (100 * 0.05 * m_rad) ** 2 + 0.3, (100 * 0.05 * m_tan) ** 2 + 0.3
        np.testing.assert_allclose(o["conic"][1], [1 / vx, 0, 1 / vy], rtol=2e-5, atol=1e-7)
    sc = S.tiny_scene(n=3, width=400, height=300, seed=3)
    sc.viewmat = np.eye(4, dtype=np.float32)
    sc.intrins = np.array([200.0, 200.0, 200.0, 150.0], np.float32)
    sc.means[:] = [[1.0, 0, 2.0], [0, 0.6, 2.0], [1.6, 0, 2.0]]
    sc.log_scales[:] = math.log(0.02)
    sc.opacity_logits[:] = 2.0
    sc = S.with_lens(sc, S.LENS_OPENCV)
    sc.dist_coeffs = np.array([-0.5, 0, 0, 0, 0, 0, 0, 0], np.float32)
    o = oracle.projection_fwd(sc)
    np.testing.assert_allclose(o["xy"][0], [200 + 200 * 0.5 * (1 - 0.5 * 0.25), 150], rtol=2e-6)
    np.testing.assert_allclose(o["xy"][1], [200, 150 + 200 * 0.3 * (1 - 0.5 * 0.09)], rtol=2e-6)
    # at u = 0.8 the radial map folds: d/du [u (1 - u^2 / 2)] = 1 - 1.5 u^2 = 0.04 < 0.25 -> dropped
    assert o["aabb"][2, 2] == 0 and o["aabb"][0, 2] > 0


def _loss64(sc, g, v, mean, quat, ls, logit, dc, sh):
    r = ref64.project(mean, quat, ls, logit, sc.viewmat, sc.intrins, sc.width, sc.camera_model, tier=sc.distortion,
                      coeffs=sc.dist_coeffs)
    col = ref64.sh_color(mean, sc.viewmat, dc, sh)
    f64 = lambda a: np.asarray(a, np.float64)
    return float(f64(v["v_xy"][g]) @ r["xy"] + f64(v["v_depth"][g]) * r["depth"] + f64(v["v_conic"][g]) @ r["conic"]
                 + f64(v["v_opac"][g]) * r["opac"] + f64(v["v_rgb"][g]) @ col)


@pytest.mark.parametrize("model,tier", PAIRS)
def test_backward_matches_finite_differences(pkg, oracle, model, tier):
    sc = _scene(pkg, model, tier, n=160, seed=29)
    rng = np.random.default_rng(7)
    o = oracle.projection_fwd(sc)
    n = sc.n
    v = dict(v_xy=rng.normal(0, 1, (n, 2)).astype(np.float32), v_depth=rng.normal(0, 1, n).astype(np.float32),
             v_conic=rng.normal(0, 1, (n, 3)).astype(np.float32), v_opac=rng.normal(0, 1, n).astype(np.float32),
             v_rgb=rng.normal(0, 1, (n, 3)).astype(np.float32))
    g_or = oracle.projection_bwd(sc, o["aabb"], v)
    vis = np.nonzero(o["aabb"][:, 2] > o["aabb"][:, 0])[0]
    assert len(vis) > 20
    for g in vis[:25]:
        args = [sc.means[g].astype(np.float64), sc.quats[g].astype(np.float64), sc.log_scales[g].astype(np.float64),
                np.array([float(sc.opacity_logits[g])]), sc.features_dc[g].astype(np.float64),
                sc.features_sh[g].astype(np.float64)]
        names = ["v_means", "v_quats", "v_scales", "v_opacities"]

        def L(a):
            return _loss64(sc, g, v, a[0], a[1], a[2], float(a[3][0]), a[4], a[5])
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
    cull = np.nonzero(~(o["aabb"][:, 2] > o["aabb"][:, 0]))[0]
    for name in ["v_means", "v_quats", "v_scales", "v_opacities", "v_dc", "v_sh"]:
        assert not np.any(g_or[name][cull])


def test_pinhole_clamp_with_a_lens_routes_to_the_bound(pkg, oracle):
    """As for the undistorted pinhole: a clamped J[.,2] follows its bound, which depends on z alone
    (src/shaders/primitive_3dgs.slang:84-95); the finite differences of the clamped forward see that."""
    S = pkg.scenes
    sc = S.tiny_scene(n=2, width=64, height=64, seed=1)
    sc.viewmat = np.eye(4, dtype=np.float32)
    sc.means[:] = [[1.05, 0.9, 1.0], [-1.0, -0.95, 1.0]]
    sc.log_scales[:] = math.log(0.3)
    sc.opacity_logits[:] = 2.0
    sc = S.with_lens(sc, S.LENS_OPENCV)
    sc.dist_coeffs = np.array([0.01, 0.0, 0.001, -0.001, 0, 0, 0, 0], np.float32)
    o = oracle.projection_fwd(sc)
    assert np.all(o["aabb"][:, 2] > o["aabb"][:, 0])
    rng = np.random.default_rng(5)
    v = dict(v_xy=rng.normal(0, 1, (2, 2)).astype(np.float32), v_depth=np.zeros(2, np.float32),
             v_conic=rng.normal(0, 1, (2, 3)).astype(np.float32), v_opac=np.zeros(2, np.float32),
             v_rgb=np.zeros((2, 3), np.float32))
    g_or = oracle.projection_bwd(sc, o["aabb"], v)
    for g in range(2):
        r = _ref(sc, g)
        J_free = ref64.model_jacobian(0, sc.distortion, sc.dist_coeffs, sc.intrins, r["pc"])
        lim = 64 + 0.3 * 32
        assert J_free[0, 2] < -(lim - 32) / r["pc"][2] or J_free[0, 2] > (0.3 * 32 + 32) / r["pc"][2]   # clamped
        mean = sc.means[g].astype(np.float64)
        fd = np.zeros(3)
        for k in range(3):
            h = 1e-6
            mp, mm = mean.copy(), mean.copy()
            mp[k] += h; mm[k] -= h
            a = [sc.quats[g].astype(np.float64), sc.log_scales[g].astype(np.float64), float(sc.opacity_logits[g]),
                 sc.features_dc[g].astype(np.float64), sc.features_sh[g].astype(np.float64)]
            fd[k] = (_loss64(sc, g, v, mp, *a) - _loss64(sc, g, v, mm, *a)) / (2 * h)
        np.testing.assert_allclose(g_or["v_means"][g], fd, rtol=2e-3, atol=2e-3 * np.abs(fd).max())


@pytest.mark.parametrize("model,tier", [(0, 0), (0, 1), (0, 3), (1, 2), (2, 0), (3, 0)])
def test_camera_pose_gradient_matches_finite_differences(pkg, oracle, model, tier):
    """dL/dR and dL/dt of the view matrix (the reference's v_viewmats: the projection through mean_c = R mean + t and
    cov_c = R cov R^T, the colour through the view direction mean + R^T t), summed over the splats, against central
    differences of the float64 loss in each of the twelve entries (R perturbed entry by entry, not kept orthonormal:
    that is the derivative the reference's autodiff forms)."""
    sc = _scene(pkg, model, tier, n=120, seed=37)
    rng = np.random.default_rng(9)
    o = oracle.projection_fwd(sc)
    n = sc.n
    v = dict(v_xy=rng.normal(0, 1, (n, 2)).astype(np.float32), v_depth=rng.normal(0, 1, n).astype(np.float32),
             v_conic=rng.normal(0, 1, (n, 3)).astype(np.float32), v_opac=rng.normal(0, 1, n).astype(np.float32),
             v_rgb=rng.normal(0, 1, (n, 3)).astype(np.float32))
    vis = np.nonzero(o["aabb"][:, 2] > o["aabb"][:, 0])[0]
    assert len(vis) > 20
    got = oracle.projection_bwd(sc, o["aabb"], v, pose=True)["v_viewmat"].astype(np.float64)
    assert not np.any(got[3])
    # the same world gradients with and without the pose output
    plain = oracle.projection_bwd(sc, o["aabb"], v)
    with_pose = oracle.projection_bwd(sc, o["aabb"], v, pose=True)
    for k in plain:
        assert np.array_equal(plain[k], with_pose[k]), k

    def total(vm):
        import dataclasses
        s2 = dataclasses.replace(sc, viewmat=vm)
        return sum(_loss64(s2, g, v, sc.means[g].astype(np.float64), sc.quats[g].astype(np.float64), sc.log_scales[g].astype(np.float64),
                           float(sc.opacity_logits[g]), sc.features_dc[g].astype(np.float64), sc.features_sh[g].astype(np.float64))
                   for g in vis)
    fd = np.zeros((4, 4))
    base = sc.viewmat.astype(np.float64)
    for i in range(3):
        for j in range(4):
            h = 1e-6 * max(1.0, abs(base[i, j]))
            vp, vm_ = base.copy(), base.copy()
            vp[i, j] += h
            vm_[i, j] -= h
            fd[i, j] = (total(vp) - total(vm_)) / (2 * h)
    scale = np.abs(fd).max()
    assert scale > 1e-3
    assert np.abs(got - fd).max() <= 3e-3 * scale, (got, fd)


# ---- the antialiased ("mip") variant of the primitive: same projection function, runtime flag ----

def _aa_scene(pkg, model, tier, n=300, seed=41):
    sc = _scene(pkg, model, tier, n=n, seed=seed)
    sc.log_scales -= 1.2          # small on screen: the blur matters, compensation well below 1
    sc.antialiased = True
    return sc


@pytest.mark.parametrize("model,tier", [(0, 0), (0, 2), (1, 1), (3, 0)])
def test_antialiased_forward_matches_float64(pkg, oracle, model, tier):
    sc = _aa_scene(pkg, model, tier)
    o = oracle.projection_fwd(sc)
    plain = oracle.projection_fwd(dataclasses.replace(sc, antialiased=False))
    vis = o["aabb"][:, 2] > o["aabb"][:, 0]
    assert vis.sum() > 40
    comps = []
    for g in np.nonzero(vis)[0][:120]:
        r = ref64.project(sc.means[g].astype(np.float64), sc.quats[g].astype(np.float64), sc.log_scales[g].astype(np.float64),
                          float(sc.opacity_logits[g]), sc.viewmat, sc.intrins, sc.width, sc.camera_model, tier=sc.distortion,
                          coeffs=sc.dist_coeffs, antialiased=True)
        np.testing.assert_allclose(o["xy"][g], r["xy"], rtol=2e-5, atol=3e-3)
        np.testing.assert_allclose(o["conic"][g], r["conic"], rtol=1e-3, atol=2e-6)
        np.testing.assert_allclose(o["opac"][g], r["opac"], rtol=2e-4, atol=1e-7)
        # closed form of the compensation: the blurred splat keeps the integrated weight of the unblurred one,
        # opacity * 2 pi sqrt(det) is the same before and after
        c2 = r["cov2d"]
        before = c2 - np.float32(0.1) * np.eye(2)
        sig = 1 / (1 + math.exp(-float(sc.opacity_logits[g])))
        assert abs(o["opac"][g] * math.sqrt(np.linalg.det(c2)) - sig * math.sqrt(max(np.linalg.det(before), 0))) <= 2e-4 * sig * math.sqrt(np.linalg.det(c2))
        comps.append(o["opac"][g] / sig)
        if plain["aabb"][g, 2] > plain["aabb"][g, 0]:
            assert o["opac"][g] <= plain["opac"][g] * (1 + 1e-6)          # never brighter than the plain variant
            assert o["conic"][g, 0] >= plain["conic"][g, 0] * (1 - 1e-6)   # and sharper (blur 0.1 instead of 0.3)
    assert min(comps) < 0.7 and max(comps) > 0.8      # the compensation spans a wide range in the scene


@pytest.mark.parametrize("model,tier", [(0, 0), (0, 1), (2, 2), (3, 0)])
def test_antialiased_backward_matches_finite_differences(pkg, oracle, model, tier):
    sc = _aa_scene(pkg, model, tier, n=160, seed=43)
    rng = np.random.default_rng(11)
    o = oracle.projection_fwd(sc)
    n = sc.n
    v = dict(v_xy=rng.normal(0, 1, (n, 2)).astype(np.float32), v_depth=rng.normal(0, 1, n).astype(np.float32),
             v_conic=rng.normal(0, 1, (n, 3)).astype(np.float32), v_opac=rng.normal(0, 3, n).astype(np.float32),
             v_rgb=rng.normal(0, 1, (n, 3)).astype(np.float32))
    g_or = oracle.projection_bwd(sc, o["aabb"], v, pose=True)
    vis = np.nonzero(o["aabb"][:, 2] > o["aabb"][:, 0])[0]
    assert len(vis) > 20

    def loss(g, mean, quat, ls, logit, viewmat=None):
        r = ref64.project(mean, quat, ls, logit, sc.viewmat if viewmat is None else viewmat, sc.intrins, sc.width, sc.camera_model,
                          tier=sc.distortion, coeffs=sc.dist_coeffs, antialiased=True)
        col = ref64.sh_color(mean, sc.viewmat if viewmat is None else viewmat, sc.features_dc[g].astype(np.float64),
                             sc.features_sh[g].astype(np.float64))
        f64 = lambda a: np.asarray(a, np.float64)
        return float(f64(v["v_xy"][g]) @ r["xy"] + f64(v["v_depth"][g]) * r["depth"] + f64(v["v_conic"][g]) @ r["conic"]
                     + f64(v["v_opac"][g]) * r["opac"] + f64(v["v_rgb"][g]) @ col)
    for g in vis[:20]:
        args = [sc.means[g].astype(np.float64), sc.quats[g].astype(np.float64), sc.log_scales[g].astype(np.float64),
                np.array([float(sc.opacity_logits[g])])]
        for ai, name in enumerate(["v_means", "v_quats", "v_scales", "v_opacities"]):
            got = np.asarray(g_or[name][g], np.float64).reshape(-1)
            fd = np.zeros_like(got)
            for k in range(args[ai].size):
                h = 1e-6 * max(1.0, abs(args[ai][k]))
                ap, am = [x.copy() for x in args], [x.copy() for x in args]
                ap[ai][k] += h
                am[ai][k] -= h
                fd[k] = (loss(g, ap[0], ap[1], ap[2], float(ap[3][0])) - loss(g, am[0], am[1], am[2], float(am[3][0]))) / (2 * h)
            assert np.abs(got - fd).max() <= 2e-3 * (np.abs(fd).max() + 1e-6), (g, name, got, fd)
    # the opacity gradient reaches the scales through the compensation: with only v_opac set the scale gradient is not zero
    v0 = {k: np.zeros_like(a) for k, a in v.items()}
    v0["v_opac"] = v["v_opac"]
    assert np.abs(oracle.projection_bwd(sc, o["aabb"], v0)["v_scales"][vis]).max() > 1e-3
    assert not np.any(oracle.projection_bwd(dataclasses.replace(sc, antialiased=False), o["aabb"], v0)["v_scales"])
    # and the camera pose
    fd = np.zeros((4, 4))
    base = sc.viewmat.astype(np.float64)
    tot = lambda vm: sum(loss(g, sc.means[g].astype(np.float64), sc.quats[g].astype(np.float64), sc.log_scales[g].astype(np.float64),
                              float(sc.opacity_logits[g]), vm) for g in vis)
    for i in range(3):
        for j in range(4):
            h = 1e-6 * max(1.0, abs(base[i, j]))
            vp, vm_ = base.copy(), base.copy()
            vp[i, j] += h
            vm_[i, j] -= h
            fd[i, j] = (tot(vp) - tot(vm_)) / (2 * h)
    assert np.abs(g_or["v_viewmat"].astype(np.float64) - fd).max() <= 3e-3 * np.abs(fd).max()
