"""Projection backward fused with Adam (oracle restatement of the fp32-state branch of
src/kernels/optim/FusedProjectionBwdOptim_kernel.cuh:232-710), pinned against a float64 numpy Adam fed
the (separately pinned) projection gradient, with the regularizer gradients taken by central finite
differences of the loss definitions of src/shaders/per_splat_losses.slang:30-81."""
import numpy as np
import pytest

B1, B2, EPS = float(np.float32(0.9)), float(np.float32(0.999)), 1e-15   # the reference's float constants
KSH0 = 0.28209479177387814


def _erank64(ls, w, w3):
    """erank_reg_3dgs, src/shaders/per_splat_losses.slang:3-15, in float64."""
    x = np.exp(2.0 * np.asarray(ls, np.float64))
    s = np.sort(x / x.sum())
    s3, s1 = s[0], s[2]
    s2 = 1.0 - s1 - s3
    r = np.exp(-s1 * np.log(s1) - s2 * np.log(s2) - s3 * np.log(s3))
    return w * max(-np.log(r - 0.99999), 0.0) + w3 * s3


def _losses64(ls, logit, quat, dc, sh, h, n_coef):
    """Sum of the per-splat regularizers with v_loss = 1, in float64."""
    e = np.exp(ls)
    ratio = e.max() / e.min()
    loss = h["mcmc_opacity_reg_weight"] / (1 + np.exp(-logit))
    loss += h["mcmc_scale_reg_weight"] * 1e-2 * ls.sum() / 3.0
    loss += h["scale_regularization_weight"] * (max(ratio, h["max_gauss_ratio"]) - h["max_gauss_ratio"])
    qn = np.linalg.norm(quat)
    loss += h["quat_norm_reg_weight"] * (qn - 1 - np.log(qn))
    # dc / sh magnitude: the kernel adds w (relu(dc - lim) + min(dc + lim, 0)) and (w / n_coef) sh to the gradients,
    # i.e. the losses w/2 (relu(|dc| - lim))^2 and w / (2 n_coef) |sh|^2
    lim = 0.5 / KSH0
    loss += 0.5 * h["sh_reg_weight"] * (np.maximum(np.abs(dc) - lim, 0) ** 2).sum()
    loss += 0.5 * h["sh_reg_weight"] / max(n_coef, 1) * (sh ** 2).sum()
    if h.get("erank_reg_weight", 0.0) or h.get("erank_reg_weight_s3", 0.0):
        loss += _erank64(ls, h.get("erank_reg_weight", 0.0), h.get("erank_reg_weight_s3", 0.0))
    return loss


def _fd(f, x, eps=1e-6):
    g = np.zeros_like(x)
    for i in range(x.size):
        d = np.zeros_like(x)
        d.flat[i] = eps
        g.flat[i] = (f(x + d) - f(x - d)) / (2 * eps)
    return g


def _rot_raw(q):
    """normalized_quat_to_rotmat (src/shaders/projection_utils.slang:69-88) applied to the quaternion as stored."""
    w, x, y, z = q
    return np.array([[1 - 2 * (y * y + z * z), 2 * (x * y - w * z), 2 * (x * z + w * y)],
                     [2 * (x * y + w * z), 1 - 2 * (x * x + z * z), 2 * (y * z - w * x)],
                     [2 * (x * z - w * y), 2 * (y * z + w * x), 1 - 2 * (x * x + y * y)]])


@pytest.mark.parametrize("per_splat_steps,scale_agnostic", [(False, False), (True, False), (False, True)])
def test_fused_optimizer_against_float64_adam(pkg, oracle, per_splat_steps, scale_agnostic):
    sc = pkg.scenes.tiny_scene(n=120, width=96, height=64, seed=51)
    sc.means[::4, 2] = -10.0                     # culled splats still decay their moments
    sc.log_scales[5] = [-2.0, -4.5, -3.0]        # ratio e^2.5 > max_gauss_ratio
    sc.features_dc[7] = [2.5, -2.2, 0.1]         # beyond +-0.5/kSh0
    sc.quats *= np.linspace(0.5, 2.0, sc.n)[:, None].astype(np.float32)   # non-unit quaternions
    r = oracle.pipeline(sc)
    rng = np.random.default_rng(2)
    P = {k: np.ascontiguousarray(getattr(sc, k), np.float32).copy() for k in oracle.WORLD_KEYS}
    g1 = {k: (rng.normal(0, 1e-3, P[k].shape)).astype(np.float32) for k in oracle.WORLD_KEYS}
    g2 = {k: (rng.uniform(1e-7, 1e-5, P[k].shape)).astype(np.float32) for k in oracle.WORLD_KEYS}
    v_in = {"means": rng.normal(0, 1e-3, (sc.n, 3)).astype(np.float32), "opacity_logits": None}
    h = dict(lr_means=1.6e-4, lr_quats=1e-3, lr_scales=5e-3, lr_opacs=5e-2, lr_features_dc=2.5e-3,
             lr_features_sh=1.25e-4, max_gauss_ratio=6.0, scale_regularization_weight=0.01,
             mcmc_opacity_reg_weight=0.01, mcmc_scale_reg_weight=0.01, quat_norm_reg_weight=0.02, sh_reg_weight=0.05,
             erank_reg_weight=0.1, erank_reg_weight_s3=0.01)
    sc.log_scales[9] = [-3.0, -3.0 - 1e-3, -7.0]   # nearly a needle... a disc: effective rank close to 2
    sc.log_scales[11] = [-2.5, -6.5, -6.6]         # a needle: effective rank close to 1, the log term is large
    steps = rng.integers(1, 400, sc.n).astype(np.int32) if per_splat_steps else None
    step = 37
    P0 = {k: v.astype(np.float64) for k, v in P.items()}
    G1 = {k: v.astype(np.float64) for k, v in g1.items()}
    G2 = {k: v.astype(np.float64) for k, v in g2.items()}
    radii = r["proj"]["radii"] if scale_agnostic else None
    score = oracle.fused_projection_bwd_optimizer(sc, r["proj"]["aabb"], r["vscreen"], P, g1, g2, h, step=step,
                                                  steps=steps, v_in=v_in, radii=radii)
    # ---- float64 expectation ----
    gr = r["grads"]
    data = dict(means=gr["v_means"] + v_in["means"], quats=gr["v_quats"], log_scales=gr["v_scales"],
                opacity_logits=gr["v_opacities"], features_dc=gr["v_dc"], features_sh=gr["v_sh"])
    data = {k: v.astype(np.float64) for k, v in data.items()}
    t = (steps if per_splat_steps else np.full(sc.n, step)).astype(np.float64)
    c1, c2 = 1 / (1 - B1 ** t), 1 / (1 - B2 ** t)
    exp_score = np.exp(P0["log_scales"].max(axis=1)) * np.linalg.norm(data["means"], axis=1)
    assert np.allclose(score, exp_score, rtol=1e-5, atol=1e-12)
    for g in range(sc.n):
        ls, lo, q, dc, sh = (P0["log_scales"][g], P0["opacity_logits"][g], P0["quats"][g], P0["features_dc"][g],
                             P0["features_sh"][g])
        reg = dict(
            log_scales=_fd(lambda x: _losses64(x, lo, q, dc, sh, h, 15), ls),
            opacity_logits=_fd(lambda x: _losses64(ls, x[0], q, dc, sh, h, 15), np.array([lo]))[0],
            quats=_fd(lambda x: _losses64(ls, lo, x, dc, sh, h, 15), q),
            features_dc=_fd(lambda x: _losses64(ls, lo, q, x, sh, h, 15), dc),
            features_sh=_fd(lambda x: _losses64(ls, lo, q, dc, x, h, 15), sh), means=0.0)
        for k in oracle.WORLD_KEYS:
            v = data[k][g] + reg[k]
            x = P0[k][g]
            if k == "quats":
                x = x / np.linalg.norm(x)
                v = v - np.dot(x, v) * x
            m1 = B1 * G1[k][g] + (1 - B1) * v
            m2 = B2 * G2[k][g] + (1 - B2) * v * v
            if k == "means" and scale_agnostic:
                # use_scale_agnostic_mean, FusedProjectionBwdOptim_kernel.cuh:519-534
                Rm = _rot_raw(q)
                cov = Rm @ np.diag(np.exp(ls)) @ Rm.T
                extent = np.sqrt(2 * np.log(max(255.0 / (1 + np.exp(-lo)), 1.00001)))
                m1 = B1 * G1[k][g] + (1 - B1) * (cov @ v) * extent
                m2 = B2 * G2[k][g] + (1 - B2) * v * v * (0.6 * float(radii[g])) ** 2
            lr = h["lr_" + {"log_scales": "scales", "opacity_logits": "opacs"}.get(k, k)]
            new = x - lr * c1[g] * m1 / (np.sqrt(m2 * c2[g]) + EPS)
            if k == "quats":
                new = new / np.linalg.norm(new)
            scale = np.abs(v).max() + 1e-12
            assert np.allclose(g1[k][g], m1, rtol=2e-5, atol=2e-6 * scale), (k, g)
            assert np.allclose(g2[k][g], m2, rtol=5e-5, atol=1e-12), (k, g)
            assert np.allclose(P[k][g], new, rtol=1e-5, atol=2e-5 * lr * 50 + 1e-7), (k, g, P[k][g], new)


def test_zero_learning_rates_and_weights_leave_parameters_alone(pkg, oracle):
    sc = pkg.scenes.tiny_scene(n=60, width=64, height=48, seed=52)
    r = oracle.pipeline(sc)
    P = {k: np.ascontiguousarray(getattr(sc, k), np.float32).copy() for k in oracle.WORLD_KEYS}
    keep = {k: v.copy() for k, v in P.items()}
    g1 = {k: np.zeros_like(v) for k, v in P.items()}
    g2 = {k: np.zeros_like(v) for k, v in P.items()}
    oracle.fused_projection_bwd_optimizer(sc, r["proj"]["aabb"], r["vscreen"], P, g1, g2, {}, step=1)
    for k in P:
        if k == "quats":   # re-normalised
            assert np.allclose(P[k], keep[k] / np.linalg.norm(keep[k], axis=1, keepdims=True), atol=1e-6)
        else:
            assert np.array_equal(P[k], keep[k]), k
    # moments took the gradient: g1 = 0.1 v
    assert np.allclose(g1["means"], 0.1 * r["grads"]["v_means"], rtol=1e-5, atol=1e-12)
    assert np.allclose(g2["features_sh"], 0.001 * r["grads"]["v_sh"] ** 2, rtol=1e-4, atol=1e-20)


def test_effective_rank_regularizer(oracle):
    """Loss and gradient of erank_reg_3dgs against its float64 definition and central differences; the
    -log term switches off once exp(entropy) - 0.99999 reaches 1; on ties the derivative of max / min is
    shared between the tied operands, as the reference's differentiated max does
    (src/generated/per_splat_losses.cuh:19-45)."""
    rng = np.random.default_rng(4)
    n_on = n_off = 0
    for _ in range(300):
        ls = rng.uniform(-7, -1, 3)
        u = rng.random()
        if u < 0.35:
            ls[1:] = ls[0] - rng.uniform(2.0, 5.0, 2)    # needle-like: rank near 1, the log term is active
        elif u < 0.7:
            ls = ls[0] + rng.uniform(-0.4, 0.4, 3)       # blob-like: rank well above 2, the log term is off
        w, w3 = float(rng.uniform(0, 0.2)), float(rng.uniform(0, 0.05))
        ls32 = ls.astype(np.float32).astype(np.float64)
        loss, g = oracle.erank_reg(ls32, w, w3)
        want = _erank64(ls32, w, w3)
        x = np.exp(2 * ls32); s = np.sort(x / x.sum())
        r = np.exp(-(s * np.log(s)).sum())
        if abs(r - 1.99999) < 1e-3:
            continue                                    # at the switch
        n_on += r < 1.99999
        n_off += r > 1.99999
        assert np.isclose(loss, want, rtol=2e-4, atol=1e-6)
        fd = _fd(lambda v: _erank64(v, w, w3), ls32, eps=1e-5)
        assert np.allclose(g, fd, rtol=2e-3, atol=2e-4 * (np.abs(fd).max() + 1e-3)), (ls32, g, fd)
    assert n_on > 50 and n_off > 50
    # isotropic: entropy is stationary, and d s_min / d l = 2 s_min (weights - s) with the tie weights (1/4, 1/4, 1/2)
    loss, g = oracle.erank_reg(np.array([-3.0, -3.0, -3.0]), 0.0, 1.0)
    assert np.isclose(loss, 1 / 3, rtol=1e-6)
    assert np.allclose(g, 2 / 3 * (np.array([0.25, 0.25, 0.5]) - 1 / 3), atol=1e-6)
    loss, g = oracle.erank_reg(np.array([-3.0, -3.0, -3.0]), 1.0, 0.0)
    assert loss == 0.0 and not np.any(g)               # rank 3: the log term is off


def test_colour_maps_of_the_trust_region(oracle):
    """ssr_srgb_slope against central differences of the sRGB transfer curve in float64; splat_dc_decode inverts
    splat_dc_encode, the map has slope 1 at colour 0.5 and continues linearly below colour 0
    (src/shaders/pixel_wise.slang:60-115)."""
    x = np.concatenate([np.linspace(-0.2, 0.0031, 40), np.linspace(0.0032, 2.0, 400)]).astype(np.float32)
    curve = lambda v: np.where(v < 0.0031308, 12.92 * v, 1.055 * np.maximum(v, 1e-300) ** (1 / 2.4) - 0.055)
    h = 1e-7
    want = (curve(x.astype(np.float64) + h) - curve(x.astype(np.float64) - h)) / (2 * h)
    got = oracle.colour_map(0, x)
    keep = np.abs(x.astype(np.float64) - 0.0031308) > 1e-5      # the curve's two branches meet with different slopes
    assert np.abs(got[keep] / want[keep] - 1).max() < 2e-5
    assert np.all(got[x < 0.0031308] == np.float32(12.92))
    dc = np.linspace(-4.0, 6.0, 2001).astype(np.float32)      # colours from below 0 to above 2
    enc = oracle.colour_map(1, dc)
    back = oracle.colour_map(2, enc)
    assert np.abs(back - dc).max() < 5e-6
    assert np.all(np.diff(enc) > 0)
    k = 0.28209479177387814
    # slope 1 at colour 0.5 (dc = 0) and constant slope k / a * s / k = s / a below colour 0
    e = oracle.colour_map(1, np.array([-1e-3, 1e-3], np.float32)).astype(np.float64)
    assert abs((e[1] - e[0]) / 2e-3 - 1.0) < 2e-3
    a = 1 / 255.0
    s = np.sqrt(0.5 + a * a)
    low = oracle.colour_map(1, np.array([-3.0, -2.5], np.float32)).astype(np.float64)      # colours -0.35, -0.21
    assert abs((low[1] - low[0]) / 0.5 - s / a) < 1e-2 * s / a
    # float64 definitions
    u = k * dc.astype(np.float64) + 0.5
    w = np.where(u >= 0, 2 * np.sqrt(np.maximum(u, 0) + a * a), 2 * a + u / a)
    want_enc = (w - 2 * s) * s / k
    # below colour 0 the map multiplies the fp32 rounding of the colour by s / (a k) = 640
    assert (np.abs(enc - want_enc) <= 2e-6 * np.abs(want_enc) + 1e-4).all()


@pytest.mark.parametrize("quantized", [False, True])
def test_colour_trust_region_against_float64(pkg, oracle, quantized):
    """color_trust_linear (FusedProjectionBwdOptim_kernel.cuh:551-596,651-705,774-794): DC and SH steps of the oracle
    against a float64 restatement built from the pinned gradients, the float64 colour maps and the clip radii."""
    sc = pkg.scenes.tiny_scene(n=300, width=96, height=64, seed=57)
    sc.features_dc[3] = [-2.0, 0.4, 3.0]          # a colour below 0 (linear continuation) and one above 1
    sc.opacity_logits[5] = -9.0                   # nearly transparent: wide clip
    n = sc.n
    rng = np.random.default_rng(4)
    h = dict(lr_means=1.6e-4, lr_quats=1e-3, lr_scales=5e-3, lr_opacs=5e-2, lr_features_dc=2.5e-2, lr_features_sh=1.25e-2,
             max_gauss_ratio=6.0, scale_regularization_weight=0.01, mcmc_opacity_reg_weight=0.01, mcmc_scale_reg_weight=0.01,
             quat_norm_reg_weight=0.02, sh_reg_weight=0.05, color_trust_linear=1.0, eps_tr=1e-4)     # large rates: the clips bind
    step = 5
    k0 = 0.28209479177387814
    if quantized:
        q = oracle.quantize_sh_state(sc.features_sh)
        sc.features_sh = oracle.decode_sh_values(q, n)
    r = oracle.pipeline(sc)
    P = {k: np.ascontiguousarray(getattr(sc, k), np.float32).copy() for k in oracle.WORLD_KEYS}
    g1 = {k: rng.normal(0, 1e-3, P[k].shape).astype(np.float32) for k in oracle.WORLD_KEYS}
    g2 = {k: rng.uniform(1e-7, 1e-5, P[k].shape).astype(np.float32) for k in oracle.WORLD_KEYS}
    P0 = {k: v.astype(np.float64) for k, v in P.items()}
    G1 = {k: v.astype(np.float64) for k, v in g1.items()}
    G2 = {k: v.astype(np.float64) for k, v in g2.items()}
    if quantized:
        G1["features_sh"][:] = 0; G2["features_sh"][:] = 0        # the quantized state starts from zero moments
        oracle.fused_projection_bwd_optimizer_q(sc, r["proj"]["aabb"], r["vscreen"], P, q, g1, g2, h, step=step)
        new_sh = oracle.decode_sh_values(q, n).astype(np.float64)
        tol_sh = ((q["value_bounds"][:, 1] - q["value_bounds"][:, 0]) / 65535).repeat(256)[:n, None, None] * 0.51 + 1e-6
    else:
        oracle.fused_projection_bwd_optimizer(sc, r["proj"]["aabb"], r["vscreen"], P, g1, g2, h, step=step)
        new_sh = P["features_sh"].astype(np.float64)
        tol_sh = 1e-6
    gr = r["grads"]
    c1, c2 = 1 / (1 - B1 ** step), 1 / (1 - B2 ** step)
    a = 1 / 255.0
    s = np.sqrt(0.5 + a * a)
    enc = lambda dc: ((np.where(k0 * dc + 0.5 >= 0, 2 * np.sqrt(np.maximum(k0 * dc + 0.5, 0) + a * a), 2 * a + (k0 * dc + 0.5) / a)) - 2 * s) * s / k0
    def dec(x):
        w = x * k0 / s + 2 * s
        return (np.where(w >= 2 * a, 0.25 * w * w - a * a, (w - 2 * a) * a) - 0.5) / k0
    slope = lambda c: np.where(c < 0.0031308, 12.92, 1.055 / 2.4 * np.maximum(c, 1e-300) ** (1 / 2.4 - 1))
    n_clipped_dc = n_clipped_sh = 0
    for g in range(n):
        dc, sh, lo = P0["features_dc"][g], P0["features_sh"][g], P0["opacity_logits"][g]
        opac = 1 / (1 + np.exp(-lo))
        c_dc = k0 * dc + 0.5
        sl = slope(c_dc)
        lim = 0.5 / k0
        v = (gr["v_dc"][g].astype(np.float64) + h["sh_reg_weight"] * (np.maximum(dc - lim, 0) + np.minimum(dc + lim, 0))) / sl
        m1 = B1 * G1["features_dc"][g] + (1 - B1) * v
        m2 = B2 * G2["features_dc"][g] + (1 - B2) * v * v
        delta = -h["lr_features_dc"] * c1 * m1 / (np.sqrt(m2 * c2) + EPS)
        clip = k0 * np.sqrt(2 * h["eps_tr"] / max(opac, 1e-12))
        n_clipped_dc += int((np.abs(delta) > clip).sum())
        want = dec(enc(dc) + np.clip(delta, -clip, clip))
        assert np.allclose(P["features_dc"][g], want, rtol=2e-5, atol=2e-5), (g, P["features_dc"][g], want)
        v = (gr["v_sh"][g].astype(np.float64) + h["sh_reg_weight"] / 15 * sh) / sl[None, :]
        m1 = B1 * G1["features_sh"][g] + (1 - B1) * v
        m2 = B2 * G2["features_sh"][g] + (1 - B2) * v * v
        delta = -h["lr_features_sh"] * c1 * m1 / (np.sqrt(m2 * c2) + EPS)
        clip = k0 * np.sqrt(4 * h["eps_tr"] * np.maximum(c_dc, a * a) / max(opac, 1e-12))
        n_clipped_sh += int((np.abs(delta) > clip[None, :]).sum())
        want = sh + np.clip(delta, -clip[None, :], clip[None, :])
        t = tol_sh if np.isscalar(tol_sh) else tol_sh[g]
        assert (np.abs(new_sh[g] - want) <= t + 2e-5 * np.abs(want)).all(), (g, np.abs(new_sh[g] - want).max())
    assert n_clipped_dc > 20 and n_clipped_sh > 200        # the trust region did bind
