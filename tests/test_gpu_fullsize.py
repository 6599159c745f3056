"""GPU: the benchmark configurations at their FULL sizes, checked through properties that do not
need the whole oracle pipeline: invariants of keys / order / ranges, sampled bit-exact comparisons of
the per-splat stages against the oracle, sampled float64 brute-force compositing, agreement between
the reference stage order and the native one, and linearity / idempotence of the backward."""
import numpy as np
import pytest

import ref64
from gpu_pipeline import world_grad_check

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def H(pkg):
    from spirula_studio_amd import host, lib
    host.load()
    return host, lib


def _depth_bits(d):
    u = np.abs(d).astype(np.float32).view(np.uint32)
    return np.where(u >> 31, ~u, u ^ np.uint32(0x80000000)).astype(np.uint64)


@pytest.mark.parametrize("cfg", [2, 3, 4, 5])
def test_full_size_properties(pkg, oracle, H, cfg):
    host, lib = H
    rng = np.random.default_rng(cfg)
    sc = pkg.scenes.make_scene(cfg)
    n, w, h = sc.n, sc.width, sc.height
    n_tiles = sc.tile_w * sc.tile_h
    print(f"[full cfg{cfg}] N={n} {w}x{h}", flush=True)
    eng = host.Engine(sc)
    eng.forward()
    eng.backward()
    keys = eng.cache("sorted_ids").view(np.uint64)
    flat = eng.cache("sorted_flat").astype(np.int64)
    offs = eng.cache("offsets").astype(np.int64)
    aabb = eng.cache("aabb").reshape(-1, 4)
    sdepth = eng.cache("sort_depth")
    K = keys.size
    assert K == eng.n_isects and K > 0
    print(f"[full cfg{cfg}] K={K}", flush=True)

    # ---- keys: sorted on the masked range, stable, each one consistent with its splat ----
    bits = 32 + oracle.tile_n_bits(n_tiles)
    mk = keys & np.uint64((1 << bits) - 1)
    assert np.all(mk[1:] >= mk[:-1])
    same = mk[1:] == mk[:-1]
    assert np.all(flat[1:][same] > flat[:-1][same])          # equal keys keep the write order (ascending splat)
    tile = (keys >> np.uint64(32)).astype(np.int64)
    assert tile.min() >= 0 and tile.max() < n_tiles
    assert np.array_equal(keys & np.uint64(0xffffffff), _depth_bits(sdepth[flat]))   # no pad keys, right depth bits
    vis = aabb[:, 2] > aabb[:, 0]
    assert vis[flat].all()
    tx, ty = tile % sc.tile_w, tile // sc.tile_w
    bb = aabb[flat]
    assert np.all((tx >= np.floor((bb[:, 0] + 0.5) / 16)) & (tx < np.ceil((bb[:, 2] + 0.5) / 16)))
    assert np.all((ty >= np.floor((bb[:, 1] + 0.5) / 16)) & (ty < np.ceil((bb[:, 3] + 0.5) / 16)))
    # ---- tile ranges: first index whose tile >= t ----
    assert np.array_equal(offs, np.searchsorted(tile, np.arange(n_tiles), side="left"))

    # ---- per-splat stages against the oracle on a sample (bit-exact) ----
    S = np.sort(rng.choice(n, size=min(n, 200000), replace=False))
    sub = pkg.scenes.subset(sc, S)
    p = oracle.projection_fwd(sub)
    assert np.array_equal(p["aabb"].view(np.uint32), aabb[S].view(np.uint32))
    assert np.array_equal(p["sort_depth"].view(np.uint32), sdepth[S].view(np.uint32))
    assert np.array_equal(p["radii"].view(np.uint32), eng.cache("radii")[S].view(np.uint32))
    sv = p["aabb"][:, 2] > p["aabb"][:, 0]
    for k, ch in [("xy", 2), ("depth", 1), ("conic", 3), ("opac", 1), ("rgb", 3)]:
        got = eng.cache(k).reshape(n, ch)[S][sv]
        assert np.array_equal(got.view(np.uint32), p[k].reshape(S.size, ch)[sv].view(np.uint32)), k
    counts = oracle.tile_count(S.size, p["aabb"], p["xy"], p["conic"], p["opac"], w, h)
    assert np.array_equal(np.bincount(flat, minlength=n)[S], counts)

    # ---- forward image: invariants and sampled float64 brute force over the tile's sorted list ----
    rgb, depth, T = eng.render()
    last = eng.cache("last_ids").reshape(h, w)
    assert np.isfinite(rgb).all() and np.isfinite(depth).all()
    assert np.all((T >= 0) & (T <= 1)) and np.all(rgb >= 0)
    empty = T == 1.0
    assert not np.any(rgb[empty]) and not np.any(last[empty])
    scr = {k: eng.cache(k) for k in ["xy", "depth", "conic", "opac", "rgb"]}
    ends = np.concatenate([offs[1:], [K]])
    checked = 0
    for _ in range(40):
        py, px = int(rng.integers(h)), int(rng.integers(w))
        t = (py // 16) * sc.tile_w + px // 16
        g = flat[offs[t]:ends[t]]
        if g.size == 0 or g.size > 3000:
            continue
        fr = dict(xy=scr["xy"].reshape(n, 2)[g].astype(np.float64), conic=scr["conic"].reshape(n, 3)[g].astype(np.float64),
                  opac=scr["opac"][g].astype(np.float64), rgb=scr["rgb"].reshape(n, 3)[g].astype(np.float64),
                  depth=scr["depth"][g].astype(np.float64))
        c, d, Tr, lk = ref64.composite(px + 0.5, py + 0.5, fr)
        # a float64 restatement may put a splat on the other side of the 1/255 or 1e-4 thresholds: allow one splat's worth
        assert np.abs(c - rgb[py, px]).max() < 6e-3 and abs(Tr - T[py, px]) < 6e-3
        checked += np.abs(c - rgb[py, px]).max() < 3e-5
        if Tr < 1.0 and abs(Tr - T[py, px]) < 1e-6:
            assert offs[t] + lk == last[py, px]
    assert checked >= 10

    # ---- gradients: zero outside the view, finite; reference order agrees; linear; idempotent ----
    g1 = eng.grads()
    for k, v in g1.items():
        assert np.isfinite(v).all(), k
        assert not np.any(v[~vis]), k
    eng.forward()
    eng.backward()
    g1b = eng.grads()
    rgb2, _, T2 = eng.render()
    assert np.array_equal(rgb, rgb2) and np.array_equal(T, T2)
    ref = host.Engine(sc, fuse_tile_count=False, visible_list=False, packed_rows=False, overwrite_world_grads=False,
                      packed_vscreen=False, tile_sort=False)
    ref.forward()
    ref.backward()
    assert np.array_equal(ref.cache("sorted_ids").view(np.uint64), keys)
    assert np.array_equal(ref.cache("sorted_flat"), flat)
    rgb3, depth3, T3 = ref.render()
    assert np.array_equal(rgb, rgb3) and np.array_equal(T, T3) and np.array_equal(depth, depth3)
    g3 = ref.grads()

    def close(a, b, what):
        # Two GPU runs against each other, without the oracle's magnitude sums to derive a floor from: an opacity
        # gradient that cancels to a thousandth of its terms differs between two summation orders by more than 1e-3
        # of itself, so a few elements per million may (the element-wise bar against the oracle, with floors, is
        # test_gpu_parity.py::test_bench_configs_full_against_the_oracle).
        world_grad_check(a, b, n, f"config{cfg}/{what[0]}/{what[1]}", bad_frac=1e-5)

    for k in g1:
        close(g1b[k], g1[k], ("idempotent", k))
        close(g3[k], g1[k], ("reference order", k))
    # packed projection outputs: same image, same gradients, ids = the visible splats in order (config 4 as the
    # benchmark runs it: the projection backward reads the parameter rows that the packed projection keeps)
    pk = host.Engine(sc, packed_projection=True, packed_world_rows=(cfg == 4))
    pk.forward()
    pk.backward()
    assert np.array_equal(pk.cache("gaussian_ids"), np.nonzero(vis)[0])
    rgb4, depth4, T4 = pk.render()
    assert np.array_equal(rgb, rgb4) and np.array_equal(T, T4) and np.array_equal(depth, depth4)
    g4 = pk.grads()
    for k in g1:
        close(g4[k], g1[k], ("packed projection", k))
        assert not np.any(g4[k][~vis]), k
    del pk, ref
    # twice the cotangent gives twice the gradient
    eng2 = host.Engine(sc)
    eng2.d_vrgb = lib.DeviceArray.from_host((2.0 * sc.v_rgb).astype(np.float32))
    eng2.d_vdepth = lib.DeviceArray.from_host((2.0 * sc.v_depth).astype(np.float32))
    eng2.d_vT = lib.DeviceArray.from_host((2.0 * sc.v_T).astype(np.float32))
    eng2.forward()
    eng2.backward()
    g2 = eng2.grads()
    for k in g1:
        close(0.5 * g2[k], g1[k], ("linear", k))


def test_full_size_default_training_step(pkg, oracle, H):
    """The reference trainer's default step at the headline size (config 2, 1 M splats): packed projection, fused
    optimizer at quantization level 1 with 16-bit non-SH moments, scale-agnostic mean step. Checked through what
    holds at any size: every block's bounds are the exact extremes of what it stores (each block contains the codes
    0 and full scale of every quantity), a first Adam step moves every visible coefficient by the learning rate,
    and the run agrees with the fp32-state step on the same scene up to the codecs' resolution."""
    host, lib = H
    S = pkg.scenes
    sc = S.make_scene(2)
    S.apply_sh_codec(sc, 2, bounds_stride=256 * 45)
    n, R = sc.n, 45
    nb = (n + 255) // 256
    h = dict(lr_means=1.6e-4, lr_quats=1e-3, lr_scales=5e-3, lr_opacs=5e-2, lr_features_dc=2.5e-3, lr_features_sh=1.25e-3,
             max_gauss_ratio=10.0, scale_regularization_weight=0.1, mcmc_opacity_reg_weight=0.01, mcmc_scale_reg_weight=0.01,
             erank_reg_weight=0.1, erank_reg_weight_s3=0.02, quat_norm_reg_weight=0.01, sh_reg_weight=0.05)
    eng = host.Engine(sc, packed_projection=True)
    eng.forward()
    q0 = eng.sh_quant_state()
    v0 = oracle.decode_sh_values(q0, n)
    eng.backward_fused_optimizer(h, 1, scale_agnostic_mean=True, quantization_level=1, non_sh_optim_bits=16)
    q1 = eng.sh_quant_state()
    ns = eng.non_sh_quant_state()
    ids = eng.cache("gaussian_ids")
    vis = np.zeros(n, bool)
    vis[ids] = True
    print(f"[full default step] N={n} visible={int(vis.sum())}", flush=True)
    assert 0.5 * n < vis.sum() < n
    # ---- every block holds both endpoints of each stored quantity ----
    full = n // 256
    codes = q1["value_packed"][: full * 256 * R].reshape(full, 256 * R)
    assert (codes.min(axis=1) == 0).all() and (codes.max(axis=1) == 65535).all()
    st = q1["state_packed"][: full * 256 * R].reshape(full, 256 * R)
    assert ((st & 255).min(axis=1) == 0).all() and ((st & 255).max(axis=1) == 255).all()
    assert ((st >> 8).min(axis=1) == 0).all() and ((st >> 8).max(axis=1) == 255).all()
    for t, prims in enumerate(oracle.NON_SH_PRIMS):
        c = ns["packed"][t][: full * 256 * prims].reshape(full, 256 * prims)
        assert ((c & 65535).min(axis=1) == 0).all() and ((c & 65535).max(axis=1) == 65535).all(), t
        assert ((c >> 16).min(axis=1) == 0).all() and ((c >> 16).max(axis=1) == 65535).all(), t
    vb = q1["value_bounds"]
    assert np.isfinite(vb).all() and (vb[:, 1] >= vb[:, 0]).all() and np.isfinite(q1["state_bounds"]).all()
    # ---- first Adam step from zero moments: +-lr for every coefficient with a gradient ----
    v1 = oracle.decode_sh_values(q1, n)
    step = (vb[:, 1] - vb[:, 0]) / 65535
    tol = np.repeat(step, 256)[:n, None, None] * 0.51 + 2e-6
    moved = np.abs(v1.astype(np.float64) - v0)
    assert (moved <= h["lr_features_sh"] * 1.001 + tol).all()
    assert (np.abs(moved[vis] - h["lr_features_sh"]) <= tol[vis]).mean() > 0.98     # visible splats: a full step (the regularizer alone moves the rest)
    # ---- against the fp32-state step on the same scene ----
    ref = S.make_scene(2)
    ref.features_sh = v0.copy()
    pq = eng.params()                      # before the next engine takes the (single) engine state over
    e32 = host.Engine(ref, packed_projection=True)
    e32.forward()
    e32.backward_fused_optimizer(h, 1, scale_agnostic_mean=True)
    p32 = e32.params()
    for k, lr in [("means", None), ("quats", "lr_quats"), ("log_scales", "lr_scales"), ("opacity_logits", "lr_opacs"), ("features_dc", "lr_features_dc")]:
        d = np.abs(p32[k].astype(np.float64) - pq[k])
        if lr is None:      # the scale-agnostic step of the means is not bounded by the rate; compare relatively
            s = np.abs(p32[k].astype(np.float64) - ref.means)
            assert (d > 0.02 * s + 1e-6).mean() < 1e-3, k
        else:
            assert (d > 0.02 * h[lr]).mean() < 1e-3, (k, float((d > 0.02 * h[lr]).mean()))
    d = np.abs(p32["features_sh"].astype(np.float64) - v1)
    assert (d > tol + 0.02 * h["lr_features_sh"]).mean() < 1e-3
