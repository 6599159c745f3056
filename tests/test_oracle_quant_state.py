"""The quantized SH state of the fused optimizer (the reference's quantization level 1): codecs against
their float64 definitions (src/core/Tensor.h:936-1133, 1300-1405) and their invariants; the optimizer step on
the quantized state against the fp32-state step, which is pinned separately, applied to the decoded state."""
import numpy as np
import pytest

EPS = 1e-15


def test_adam_state_codec(oracle):
    rng = np.random.default_rng(1)
    n = 20000
    g2 = (10.0 ** rng.uniform(-16, -2, n)).astype(np.float32)
    g2[::50] = 0.0
    g1 = (np.sqrt(g2) * rng.uniform(-3, 3, n)).astype(np.float32)
    # float64 definition of the two stored quantities
    sq = np.sqrt(g2.astype(np.float64))
    u = g1.astype(np.float64) / (sq + EPS)
    ls = np.log1p(sq / EPS)
    mm = np.array([u.min(), u.max(), ls.min(), ls.max()], np.float32)
    codes = oracle.quant_codec(0, g1, g2, mm)
    uq, sq_q = codes & 255, codes >> 8
    want_u = np.clip(np.floor(255 * (u - mm[0]) / (mm[1] - mm[0]) + 0.5), 0, 255)
    want_s = np.clip(np.floor(255 * (ls - mm[2]) / (mm[3] - mm[2]) + 0.5), 0, 255)
    assert np.abs(uq - want_u).max() <= 1 and (uq != want_u).mean() < 2e-3      # off by one only at a rounding tie
    assert np.abs(sq_q - want_s).max() <= 1 and (sq_q != want_s).mean() < 2e-3
    assert codes[np.argmin(u)] & 255 == 0 and codes[np.argmax(u)] & 255 == 255  # endpoint-exact
    assert codes[np.argmin(ls)] >> 8 == 0 and codes[np.argmax(ls)] >> 8 == 255
    # decode inverts encode to within half a step of each stored quantity
    d1, d2 = oracle.quant_codec(1, codes=codes, mm=mm)
    du = d1.astype(np.float64) / (np.sqrt(d2.astype(np.float64)) + EPS)
    dls = np.log1p(np.sqrt(d2.astype(np.float64)) / EPS)
    assert np.abs(du - u).max() <= 0.5001 * (mm[1] - mm[0]) / 255 + 1e-6
    assert np.abs(dls - ls).max() <= 0.5001 * (mm[3] - mm[2]) / 255 + 1e-5
    # zero is a fixed point: zero codes with zero bounds decode to zero moments, and (0, 0) encodes to them
    z1, z2 = oracle.quant_codec(1, codes=np.zeros(4, np.uint32), mm=np.zeros(4, np.float32))
    assert not np.any(z1) and not np.any(z2)
    c0 = oracle.quant_codec(0, np.zeros(3, np.float32), np.zeros(3, np.float32), np.array([0, 2, 0, 30], np.float32))
    assert not np.any(c0)
    # log1p / expm1 built on the shared exp / log: relative error against libm
    x = (10.0 ** rng.uniform(-12, 12, 4000)).astype(np.float32)
    c = oracle.quant_codec(0, np.zeros_like(x), (x * EPS).astype(np.float32) ** 2, np.array([0, 1, 0, 255], np.float32))
    # with bounds (0, 255) the second code is round(log1p(x)) clipped: compare with libm's
    want = np.clip(np.floor(np.log1p(np.sqrt(((x * EPS).astype(np.float32).astype(np.float64)) ** 2) / EPS) + 0.5), 0, 255)
    assert np.abs((c >> 8) - want).max() <= 1 and ((c >> 8) != want).mean() < 5e-3


def test_value_codec(oracle):
    rng = np.random.default_rng(2)
    v = rng.normal(0, 0.2, 30000).astype(np.float32)
    lo, hi = float(v.min()), float(v.max())
    codes = oracle.quant_codec(2, v, mm=[lo, hi])
    want = np.clip(np.floor(65535 * (v.astype(np.float64) - lo) / (hi - lo) + 0.5), 0, 65535)
    assert np.abs(codes - want).max() <= 1 and (codes != want).mean() < 2e-2
    assert codes[np.argmin(v)] == 0 and codes[np.argmax(v)] == 65535
    d = oracle.quant_codec(3, codes=codes, mm=[lo, hi])
    assert np.abs(d - v).max() <= 0.5001 * (hi - lo) / 65535 + 1e-7
    assert d[np.argmin(v)] == np.float32(lo)
    # a degenerate block (all values equal): every code decodes to that value
    c = oracle.quant_codec(2, np.full(5, 0.25, np.float32), mm=[0.25, 0.25])
    assert np.all(oracle.quant_codec(3, codes=c, mm=[0.25, 0.25]) == np.float32(0.25))


@pytest.mark.parametrize("sh_degree,steps_per_splat", [(3, False), (3, True), (1, False)])
def test_quantized_state_step_equals_fp32_step_on_the_decoded_state(pkg, oracle, sh_degree, steps_per_splat):
    """One optimizer step on the quantized state must equal: decode values and moments, take the (pinned) fp32
    step, re-encode against the block-wise min / max of the results. Also: bounds cover zero when coefficients
    above the active degree exist, and those coefficients come out as exact zeros."""
    sc = pkg.scenes.tiny_scene(n=700, width=96, height=64, seed=81)     # 2 full blocks + 188
    sc.means[::5, 2] = -10.0
    rng = np.random.default_rng(3)
    n, nc = sc.n, sh_degree * (sh_degree + 2)
    h = dict(lr_means=1.6e-4, lr_quats=1e-3, lr_scales=5e-3, lr_opacs=5e-2, lr_features_dc=2.5e-3, lr_features_sh=1.25e-4,
             max_gauss_ratio=6.0, scale_regularization_weight=0.01, mcmc_opacity_reg_weight=0.01, mcmc_scale_reg_weight=0.01,
             quat_norm_reg_weight=0.02, sh_reg_weight=0.05)
    q = oracle.quantize_sh_state(sc.features_sh)
    # a few steps so that the moments are not zero when the compared step starts
    P = {k: np.ascontiguousarray(getattr(sc, k), np.float32).copy() for k in oracle.WORLD_KEYS}
    g1 = {k: np.zeros_like(v) for k, v in P.items()}
    g2 = {k: np.zeros_like(v) for k, v in P.items()}
    steps = rng.integers(1, 50, n).astype(np.int32) if steps_per_splat else None

    def run(q_state, Pq, m1, m2, t):
        sc_q = pkg.scenes.subset(sc, np.arange(n))
        for k in oracle.WORLD_KEYS[:5]:
            setattr(sc_q, k, Pq[k])
        sc_q.features_sh = oracle.decode_sh_values(q_state, n)
        r = oracle.pipeline(sc_q, sh_degree=sh_degree)
        return sc_q, r

    for t in (1, 2):
        sc_q, r = run(q, P, g1, g2, t)
        oracle.fused_projection_bwd_optimizer_q(sc_q, r["proj"]["aabb"], r["vscreen"], P, q, g1, g2, h, step=t, steps=steps,
                                                sh_degree=sh_degree)
    # the compared step
    sc_q, r = run(q, P, g1, g2, 3)
    vals = oracle.decode_sh_values(q, n)
    m1, m2 = oracle.decode_sh_moments(q, n)
    Pf = {k: v.copy() for k, v in P.items()}
    Pf["features_sh"] = vals.copy()
    f1 = {k: v.copy() for k, v in g1.items()}
    f2 = {k: v.copy() for k, v in g2.items()}
    f1["features_sh"], f2["features_sh"] = m1.reshape(n, 15, 3).copy(), m2.reshape(n, 15, 3).copy()
    qn = {k: (v.copy() if isinstance(v, np.ndarray) else v) for k, v in q.items()}
    Pq = {k: v.copy() for k, v in P.items()}
    q1 = {k: v.copy() for k, v in g1.items()}
    q2 = {k: v.copy() for k, v in g2.items()}
    oracle.fused_projection_bwd_optimizer_q(sc_q, r["proj"]["aabb"], r["vscreen"], Pq, qn, q1, q2, h, step=3, steps=steps,
                                            sh_degree=sh_degree)
    oracle.fused_projection_bwd_optimizer(sc_q, r["proj"]["aabb"], r["vscreen"], Pf, f1, f2, h, step=3, steps=steps,
                                          sh_degree=sh_degree)
    for k in oracle.WORLD_KEYS[:5]:     # the non-SH parameters do not see the quantization
        assert np.array_equal(Pq[k], Pf[k]) and np.array_equal(q1[k], f1[k]) and np.array_equal(q2[k], f2[k]), k
    R = 45
    act = np.zeros(R, bool)
    act[:3 * nc] = True
    for blk in range((n + 255) // 256):
        rows = slice(blk * 256, min((blk + 1) * 256, n))
        x = Pf["features_sh"].reshape(n, R)[rows][:, act].astype(np.float64)
        a = f1["features_sh"].reshape(n, R)[rows][:, act].astype(np.float64)
        b = f2["features_sh"].reshape(n, R)[rows][:, act].astype(np.float64)
        sq = np.sqrt(np.maximum(b, 0))
        u, ls = a / (sq + EPS), np.log1p(sq / EPS)
        lo, hi = x.min(), x.max()
        mm = [u.min(), u.max(), ls.min(), ls.max()]
        if nc < 15:
            lo, hi = min(lo, 0), max(hi, 0)
            mm = [min(mm[0], 0), max(mm[1], 0), min(mm[2], 0), mm[3]]
        assert np.allclose(qn["value_bounds"][blk], [lo, hi], rtol=1e-6, atol=1e-9)
        assert np.allclose(qn["state_bounds"][blk], mm, rtol=2e-5, atol=1e-6)
    got_v = oracle.decode_sh_values(qn, n).reshape(n, R)
    want_v = Pf["features_sh"].reshape(n, R)
    step_v = (qn["value_bounds"][:, 1] - qn["value_bounds"][:, 0]) / 65535
    tol = np.repeat(step_v, 256)[:n, None] * 0.5001 + 1e-7
    assert (np.abs(got_v[:, act] - want_v[:, act]) <= tol).all()
    assert not np.any(got_v[:, ~act]) or np.abs(got_v[:, ~act]).max() <= tol.max()      # inactive coefficients: zero (to a step)
    gm1, gm2 = oracle.decode_sh_moments(qn, n)
    wsq = np.sqrt(f2["features_sh"].reshape(n, R).astype(np.float64))
    gsq = np.sqrt(gm2.astype(np.float64))
    wu = f1["features_sh"].reshape(n, R).astype(np.float64) / (wsq + EPS)
    gu = gm1.astype(np.float64) / (gsq + EPS)
    su = np.repeat((qn["state_bounds"][:, 1] - qn["state_bounds"][:, 0]) / 255, 256)[:n, None]
    sl = np.repeat((qn["state_bounds"][:, 3] - qn["state_bounds"][:, 2]) / 255, 256)[:n, None]
    assert (np.abs(gu[:, act] - wu[:, act]) <= 0.5001 * su + 1e-5).all()
    assert (np.abs(np.log1p(gsq[:, act] / EPS) - np.log1p(wsq[:, act] / EPS)) <= 0.5001 * sl + 1e-4).all()
    if nc < 15:
        assert not np.any(gm2[:, ~act]) and np.abs(gm1[:, ~act]).max() < 1e-12


def test_adam_state_codec_16_bit(oracle):
    """QuantizedAdamState<16, 256> (the non-SH state): same definitions at 65535 levels, one 32-bit cell."""
    rng = np.random.default_rng(2)
    n = 20000
    g2 = (10.0 ** rng.uniform(-16, -2, n)).astype(np.float32)
    g2[::50] = 0.0
    g1 = (np.sqrt(g2) * rng.uniform(-3, 3, n)).astype(np.float32)
    sq = np.sqrt(g2.astype(np.float64))
    u = g1.astype(np.float64) / (sq + EPS)
    ls = np.log1p(sq / EPS)
    mm = np.array([u.min(), u.max(), ls.min(), ls.max()], np.float32)
    codes = oracle.quant_codec(4, g1, g2, mm)
    uq, sq_q = (codes & 65535).astype(np.int64), (codes >> 16).astype(np.int64)
    want_u = np.clip(np.floor(65535 * (u - mm[0]) / (mm[1] - mm[0]) + 0.5), 0, 65535)
    want_s = np.clip(np.floor(65535 * (ls - mm[2]) / (mm[3] - mm[2]) + 0.5), 0, 65535)
    # fp32 arithmetic of the encode moves a 16-bit code by a few steps at most (2^-24 relative on a 2^16 range)
    assert np.abs(uq - want_u).max() <= 2 and np.abs(sq_q - want_s).max() <= 2
    assert (uq != want_u).mean() < 0.2 and (sq_q != want_s).mean() < 0.2
    assert uq[np.argmin(u)] == 0 and uq[np.argmax(u)] == 65535 and sq_q[np.argmin(ls)] == 0 and sq_q[np.argmax(ls)] == 65535
    d1, d2 = oracle.quant_codec(5, codes=codes, mm=mm)
    du = d1.astype(np.float64) / (np.sqrt(d2.astype(np.float64)) + EPS)
    dls = np.log1p(np.sqrt(d2.astype(np.float64)) / EPS)
    assert np.abs(du - u).max() <= 1.5 * (mm[1] - mm[0]) / 65535 + 1e-6
    assert np.abs(dls - ls).max() <= 1.5 * (mm[3] - mm[2]) / 65535 + 1e-5
    z1, z2 = oracle.quant_codec(5, codes=np.zeros(4, np.uint32), mm=np.zeros(4, np.float32))
    assert not np.any(z1) and not np.any(z2)
    assert not np.any(oracle.quant_codec(4, np.zeros(3, np.float32), np.zeros(3, np.float32), np.array([0, 2, 0, 30], np.float32)))


@pytest.mark.parametrize("scale_agnostic", [False, True])
def test_quantized_non_sh_state_step(pkg, oracle, scale_agnostic):
    """One step with the quantized non-SH state equals: decode the 16-bit cells against each block's bounds, take
    the fp32 step on those moments, encode the new moments against their block-wise min / max."""
    sc = pkg.scenes.tiny_scene(n=700, width=96, height=64, seed=83)
    sc.means[::5, 2] = -10.0
    n = sc.n
    h = dict(lr_means=1.6e-4, lr_quats=1e-3, lr_scales=5e-3, lr_opacs=5e-2, lr_features_dc=2.5e-3, lr_features_sh=1.25e-4,
             max_gauss_ratio=6.0, scale_regularization_weight=0.01, mcmc_opacity_reg_weight=0.01, mcmc_scale_reg_weight=0.01,
             quat_norm_reg_weight=0.02, sh_reg_weight=0.05, erank_reg_weight=0.1, erank_reg_weight_s3=0.02)
    q = oracle.quantize_sh_state(sc.features_sh)
    ns = oracle.zero_non_sh_state(n)
    P = {k: np.ascontiguousarray(getattr(sc, k), np.float32).copy() for k in oracle.WORLD_KEYS}

    def forward(Pq, q_state):
        sc_q = pkg.scenes.subset(sc, np.arange(n))
        for k in oracle.WORLD_KEYS[:5]:
            setattr(sc_q, k, Pq[k])
        sc_q.features_sh = oracle.decode_sh_values(q_state, n)
        return sc_q, oracle.pipeline(sc_q)

    for t in (1, 2):
        sc_q, r = forward(P, q)
        oracle.fused_projection_bwd_optimizer_q(sc_q, r["proj"]["aabb"], r["vscreen"], P, q, None, None, h, step=t, non_sh=ns,
                                                radii=r["proj"]["radii"] if scale_agnostic else None)
    assert all(a.any() for a in ns["packed"])
    sc_q, r = forward(P, q)
    radii = r["proj"]["radii"] if scale_agnostic else None
    f1, f2 = oracle.decode_non_sh_state(ns, n)
    Pf = {k: v.copy() for k, v in P.items()}
    qf = {k: (v.copy() if isinstance(v, np.ndarray) else v) for k, v in q.items()}
    oracle.fused_projection_bwd_optimizer_q(sc_q, r["proj"]["aabb"], r["vscreen"], Pf, qf, f1, f2, h, step=3, radii=radii)
    Pq = {k: v.copy() for k, v in P.items()}
    qq = {k: (v.copy() if isinstance(v, np.ndarray) else v) for k, v in q.items()}
    nq = dict(packed=[a.copy() for a in ns["packed"]], bounds=[a.copy() for a in ns["bounds"]])
    oracle.fused_projection_bwd_optimizer_q(sc_q, r["proj"]["aabb"], r["vscreen"], Pq, qq, None, None, h, step=3, non_sh=nq, radii=radii)
    for k in oracle.WORLD_KEYS[:5]:       # same decoded moments, same step: the parameters agree to the bit
        assert np.array_equal(Pq[k], Pf[k]), k
    for k in ["state_packed", "value_packed"]:
        assert np.array_equal(qq[k], qf[k]), k
    d1, d2 = oracle.decode_non_sh_state(nq, n)
    for t, (k, prims) in enumerate(zip(oracle.NON_SH_KEYS, oracle.NON_SH_PRIMS)):
        a, b = f1[k].reshape(n, -1).astype(np.float64), f2[k].reshape(n, -1).astype(np.float64)
        sq = np.sqrt(np.maximum(b, 0))
        u, ls = a / (sq + EPS), np.log1p(sq / EPS)
        ga, gb = d1[k].reshape(n, -1).astype(np.float64), d2[k].reshape(n, -1).astype(np.float64)
        gsq = np.sqrt(gb)
        gu, gls = ga / (gsq + EPS), np.log1p(gsq / EPS)
        for blk in range((n + 255) // 256):
            rows = slice(blk * 256, min((blk + 1) * 256, n))
            mm = np.array([u[rows].min(), u[rows].max(), ls[rows].min(), ls[rows].max()])
            assert np.allclose(nq["bounds"][t][blk], mm, rtol=2e-5, atol=1e-6), (k, blk)
            assert np.abs(gu[rows] - u[rows]).max() <= 1.5 * (mm[1] - mm[0]) / 65535 + 1e-5 * max(1.0, np.abs(mm[:2]).max()), k
            assert np.abs(gls[rows] - ls[rows]).max() <= 1.5 * (mm[3] - mm[2]) / 65535 + 1e-5 * max(1.0, mm[3]), k
