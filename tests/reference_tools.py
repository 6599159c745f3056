"""Inputs of the reference's backend parity tools (src/backend/tests/*_parity.cpp, accum_weight_map.cpp),
regenerated bit for bit: they draw everything from std::mt19937 through
`lo + (hi - lo) * (float)(rng() & 0xffffff) / 16777215.0f`, which is portable. The tools compare a CUDA
dump (not in the repository) with another backend, so they hold no expected outputs; what they do fix is
the scene family, the camera / lens fixture (tests/golden/distortion_rows.json) and the variants swept,
and accum_weight_map.cpp carries its own expectations. One camera per call here (the tools batch two)."""
from __future__ import annotations

import dataclasses
import json
import math
import os

import numpy as np

_GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "distortion_rows.json")
N_TOOL, W_TOOL, H_TOOL, C_TOOL = 3000, 200, 150, 2
SEED_RENDER, SEED_RASTER_BWD, SEED_PROJ, SEED_PROJ_BWD, SEED_FPBO = 654321, 112233, 123456, 445566, 990011


def fixture():
    return json.load(open(_GOLDEN))


class Mt19937:
    """std::mt19937: 32-bit Mersenne twister, init_genrand seeding, tempered outputs."""

    def __init__(self, seed: int):
        mt = np.empty(624, np.uint64)
        mt[0] = seed & 0xFFFFFFFF
        for i in range(1, 624):
            mt[i] = (1812433253 * (int(mt[i - 1]) ^ (int(mt[i - 1]) >> 30)) + i) & 0xFFFFFFFF
        self.mt = mt.astype(np.uint32)
        self.buf = np.empty(0, np.uint32)

    def _twist(self):
        mt = self.mt
        up, lo, mag = np.uint32(0x80000000), np.uint32(0x7FFFFFFF), np.uint32(0x9908B0DF)

        def mix(a, b, far):
            y = (a & up) | (b & lo)
            return far ^ (y >> np.uint32(1)) ^ np.where(y & np.uint32(1), mag, np.uint32(0))
        new = np.empty_like(mt)
        new[0:227] = mix(mt[0:227], mt[1:228], mt[397:624])
        new[227:454] = mix(mt[227:454], mt[228:455], new[0:227])
        new[454:623] = mix(mt[454:623], mt[455:624], new[227:396])
        new[623] = mix(mt[623:624], new[0:1], new[396:397])[0]
        self.mt = new
        y = new.copy()
        y ^= y >> np.uint32(11)
        y ^= (y << np.uint32(7)) & np.uint32(0x9D2C5680)
        y ^= (y << np.uint32(15)) & np.uint32(0xEFC60000)
        y ^= y >> np.uint32(18)
        return y

    def raw(self, n: int) -> np.ndarray:
        while self.buf.size < n:
            self.buf = np.concatenate([self.buf, self._twist()])
        out, self.buf = self.buf[:n], self.buf[n:]
        return out

    def uf(self, n: int, lo: float, hi: float) -> np.ndarray:
        """The tools' uniform: float32 arithmetic in the order written there."""
        lo32, hi32 = np.float32(lo), np.float32(hi)
        x = (self.raw(n) & np.uint32(0xFFFFFF)).astype(np.float32)
        return (lo32 + ((hi32 - lo32) * x) / np.float32(16777215.0)).astype(np.float32)


def tool_world(seed: int, n: int = N_TOOL):
    """The splats every tool starts from (e.g. render_parity.cpp:91-111): per splat 4 draws for the mean
    (z is drawn again over a wider range), 4 quaternion, 3 log-scale, 1 opacity logit, 3 DC; then all SH."""
    rng = Mt19937(seed)
    per = rng.raw(15 * n).reshape(n, 15)
    f = lambda cols, lo, hi: np.ascontiguousarray(np.float32(lo) + ((np.float32(hi) - np.float32(lo))
                                                                    * (per[:, cols] & np.uint32(0xFFFFFF)).astype(np.float32))
                                                  / np.float32(16777215.0), np.float32)
    means = f([0, 1, 3], -4.0, 4.0)
    means[:, 2] = f([3], -2.0, 8.0)[:, 0]
    quats = f([4, 5, 6, 7], -1.0, 1.0)
    small = (quats.astype(np.float32) ** 2).sum(axis=1) < 1e-6
    quats[small, 0] = 1.0
    w = dict(means=np.ascontiguousarray(means), quats=np.ascontiguousarray(quats), log_scales=f([8, 9, 10], -5.0, -1.5), opacity_logits=f([11], -3.0, 5.0)[:, 0],
             features_dc=f([12, 13, 14], -0.5, 1.5), features_sh=rng.uf(n * 45, -0.3, 0.3).reshape(n, 15, 3))
    return w, rng


def tool_camera(cam: int):
    fx = fixture()
    c, s = np.float32(math.cos(np.float32(0.2))), np.float32(math.sin(np.float32(0.2)))
    vm = [np.array([[1, 0, 0, 0], [0, 1, 0, 0], [0, 0, 1, 4], [0, 0, 0, 1]], np.float32),
          np.array([[c, 0, s, 0.3], [0, 1, 0, -0.2], [-s, 0, c, 5.0], [0, 0, 0, 1]], np.float32)][cam]
    return vm, np.array(fx["intrins"][cam], np.float32)


def tool_lens(tier: int, cam: int) -> np.ndarray:
    row = np.array(fixture()["rows"][tier], np.float32)
    return (np.float32(1.0 - 0.3 * (cam % 3)) * row).astype(np.float32)


def tool_scene(pkg, seed: int, cam: int, model: int = 0, tier: int = 0, n: int = N_TOOL, cotangents=None, mip: bool = False):
    """One camera of a tool's two-camera batch as a scene of this package. cotangents: dict with the [C,H,W,..]
    arrays the tool draws (raster_bwd_cotangents), of which camera `cam`'s slice is used."""
    w, rng = tool_world(seed, n)
    vm, intr = tool_camera(cam)
    z3 = np.zeros((H_TOOL, W_TOOL, 3), np.float32)
    z1 = np.zeros((H_TOOL, W_TOOL), np.float32)
    ct = cotangents or {}
    sc = pkg.scenes.Scene(name=f"tool-{seed}-cam{cam}", n=n, width=W_TOOL, height=H_TOOL, camera_model=model, viewmat=vm,
                          intrins=intr, v_rgb=ct["v_rgb"][cam] if ct else z3, v_depth=ct["v_depth"][cam] if ct else z1,
                          v_T=ct["v_T"][cam] if ct else z1, distortion=tier, dist_coeffs=tool_lens(tier, cam), antialiased=mip, **w)
    return sc, rng


def raster_bwd_cotangents(rng: Mt19937):
    """raster_bwd_parity.cpp:133-139, drawn right after the splats: seven [C,H,W,..] arrays in this order."""
    npx = C_TOOL * H_TOOL * W_TOOL
    shape1, shape3 = (C_TOOL, H_TOOL, W_TOOL), (C_TOOL, H_TOOL, W_TOOL, 3)
    return dict(v_rgb=rng.uf(npx * 3, -1.0, 1.0).reshape(shape3), v_depth=rng.uf(npx, -0.2, 0.2).reshape(shape1),
                v_T=rng.uf(npx, -0.5, 0.5).reshape(shape1), v_median=rng.uf(npx, -0.1, 0.1).reshape(shape1),
                v_dist_rgb=rng.uf(npx * 3, -0.05, 0.05).reshape(shape3), v_dist_depth=rng.uf(npx, -0.05, 0.05).reshape(shape1),
                accum_map=rng.uf(npx, 0.0, 1.0).reshape(shape1))


def accum_finalize(aw: np.ndarray, n: int, mode: int) -> np.ndarray:
    """Avg arrives as [numerator, denominator] planar; densify_accum_finalize_kernel
    (src/kernels/densify/DensifyScoring.cu:281-291) leaves num / den (0 where den <= 0) in the first lane."""
    if mode != 3:
        return aw[:n].copy()
    num, den = aw[:n], aw[n:2 * n]
    return np.where(den > 0, num / np.where(den > 0, den, 1), 0).astype(np.float32)


def accum_weight_map_checks(run, xy_own, xy_other, mode: int, label: str):
    """The expectations of src/backend/tests/accum_weight_map.cpp:203-290 for one camera. run(map[H,W]) -> the
    finalized per-splat score [N]; xy_own / xy_other: [N,2] screen centres per WORLD splat under this camera and
    under the batch's other one (-1e9 where culled)."""
    RX0, RX1, RY0, RY1 = 10, 45, 100, 140      # asymmetric probe rectangle (:31-33)
    W, H = W_TOOL, H_TOOL
    # 1) a rectangle scores the splats that sit under it, under this camera's projection and no other
    m = np.zeros((H, W), np.float32)
    m[RY0:RY1, RX0:RX1] = 1.0
    aw = run(m)
    scored = aw > 0
    def inside(xy, swap):
        sx, sy = (xy[:, 1], xy[:, 0]) if swap else (xy[:, 0], xy[:, 1])
        return (sx >= RX0 - 8) & (sx <= RX1 + 8) & (sy >= RY0 - 8) & (sy <= RY1 + 8)
    n_scored = int(scored.sum())
    own, other, transposed = [int((scored & inside(xy, sw)).sum()) for xy, sw in [(xy_own, False), (xy_other, False), (xy_own, True)]]
    print(f"[{label}] rectangle: {n_scored} scored; own/other camera explain {own}/{other}, transposed {transposed}", flush=True)
    assert n_scored > 20, "rectangle scored too few splats"
    assert own > 0.8 * n_scored, "map did not reach the splats under it"
    assert other < 0.5 * n_scored, "map reached the wrong image"
    assert transposed == 0, "pixel index looks transposed"
    # 2) the value carried is the map value where the splat sits
    peak = run(np.ones((H, W), np.float32))
    f = lambda x, y: np.float32(0.5) + np.float32(0.45) * np.sin(np.float32(6.2831853) * x / np.float32(W)) * np.sin(np.float32(6.2831853) * y / np.float32(H))
    yy, xx = np.meshgrid(np.arange(H, dtype=np.float32), np.arange(W, dtype=np.float32), indexing="ij")
    sm = run(f(xx, yy).astype(np.float32))
    sx, sy = xy_own[:, 0], xy_own[:, 1]
    sel = (peak > 1e-3) & ~((sx < 4) | (sy < 4) | (sx > W - 5) | (sy > H - 5))
    d = sm[sel].astype(np.float64) / peak[sel] - f(np.round(sx[sel]), np.round(sy[sel]))
    rms = float(np.sqrt((d * d).mean())) if sel.any() else 1.0
    print(f"[{label}] score/peak vs map at splat centre: n={int(sel.sum())} rms={rms:.4f}", flush=True)
    assert sel.sum() > 500, "too few splats to judge the carried value"
    assert rms < 0.15, "score does not track the map value at the splat"
    # 3) every mode is linear in the map; avg of an all-ones map is 1 for any covered splat
    k = np.float32(0.7)
    flat = run(np.full((H, W), k, np.float32))
    c = peak > 1e-3
    worst_lin = float((np.abs(flat[c] - k * peak[c]).astype(np.float64) / (k * peak[c])).max())
    print(f"[{label}] constant map: n={int(c.sum())} worst |score - c*ones|/(c*ones) = {worst_lin:.2e}", flush=True)
    assert c.sum() > 500, "too few splats to judge linearity"
    assert worst_lin < 1e-4, "score is not linear in the map"
    if mode == 3:
        worst_one = float(np.abs(peak[c] - 1.0).max())
        print(f"[{label}] avg normalization: worst |ones_score - 1| = {worst_one:.2e}", flush=True)
        assert worst_one < 1e-5, "avg is not normalized by the covered weight"


FPBO_HYPER = dict(lr_means=1.6e-4, lr_quats=1e-3, lr_scales=5e-3, lr_opacs=5e-2, lr_features_dc=2.5e-3, lr_features_sh=1.25e-4,
                  max_gauss_ratio=10.0, scale_regularization_weight=0.1, mcmc_opacity_reg_weight=0.01, mcmc_scale_reg_weight=0.01,
                  erank_reg_weight=0.1, erank_reg_weight_s3=0.02, quat_norm_reg_weight=0.01, sh_reg_weight=0.05)   # fpbo_parity.cpp:383-389
N_FPBO = 3072


def fpbo_row_inputs(rng: Mt19937, n: int = N_FPBO):
    """What fpbo_parity.cpp draws for one unpacked fp32-state 3dgs row with every world gradient present
    (:281-320): screen gradients for the C * N rows of both cameras, world gradients of the five non-SH tensors, then
    first and second moments tensor by tensor."""
    rows = C_TOOL * n
    vs = dict(v_xy=rng.uf(rows * 2, -0.5, 0.5).reshape(C_TOOL, n, 2), v_depth=rng.uf(rows, -0.2, 0.2).reshape(C_TOOL, n),
              v_conic=rng.uf(rows * 3, -0.02, 0.02).reshape(C_TOOL, n, 3), v_opac=rng.uf(rows, -0.5, 0.5).reshape(C_TOOL, n),
              v_rgb=rng.uf(rows * 3, -1.0, 1.0).reshape(C_TOOL, n, 3))
    keys = ["means", "quats", "log_scales", "opacity_logits", "features_dc", "features_sh"]
    shapes = [(n, 3), (n, 4), (n, 3), (n,), (n, 3), (n, 15, 3)]
    v_world = {k: rng.uf(int(np.prod(s)), -0.05, 0.05).reshape(s) for k, s in list(zip(keys, shapes))[:5]}
    g1, g2 = {}, {}
    for k, s in zip(keys, shapes):
        g1[k] = rng.uf(int(np.prod(s)), -0.02, 0.02).reshape(s)
        g2[k] = rng.uf(int(np.prod(s)), 0.0, 4e-4).reshape(s)
    return vs, v_world, g1, g2


COMPILED_TIERS = {0: [0, 1, 2, 3], 1: [0, 1, 2], 2: [0, 1, 2], 3: [0]}   # DistortionFixture.h:19-25


def projection_quant_inputs(rng: Mt19937, n: int = N_TOOL):
    """projection_parity.cpp:165-180: random 8- and 16-bit SH codes, then (min, max) bounds per 256 cells and per
    256 splats (the layout the fused optimizer keeps), drawn right after the splats."""
    cells = n * 45
    q8 = (rng.raw(cells) & np.uint32(0xFF)).astype(np.uint8)
    q16 = (rng.raw(cells) & np.uint32(0xFFFF)).astype(np.uint16)

    def gen_bounds(stride):
        nb = (cells + stride - 1) // stride
        d = rng.raw(2 * nb).reshape(nb, 2)
        u = lambda col, lo, hi: (np.float32(lo) + ((np.float32(hi) - np.float32(lo)) * (d[:, col] & np.uint32(0xFFFFFF)).astype(np.float32))
                                 / np.float32(16777215.0)).astype(np.float32)
        lo = u(0, -0.5, 0.1)
        return np.ascontiguousarray(np.stack([lo, (lo + u(1, 0.05, 0.8)).astype(np.float32)], axis=1), np.float32)
    return dict(q8=q8, q16=q16, bounds_cell=gen_bounds(256), bounds_block=gen_bounds(256 * 45))


def screen_gradients(rng: Mt19937, rows: int):
    """The 2D-layout screen gradients proj_bwd_parity.cpp:247-254 and fpbo_parity.cpp:281-287 draw for `rows` rows."""
    return dict(v_xy=rng.uf(rows * 2, -0.5, 0.5).reshape(rows, 2), v_depth=rng.uf(rows, -0.2, 0.2),
                v_conic=rng.uf(rows * 3, -0.02, 0.02).reshape(rows, 3), v_opac=rng.uf(rows, -0.5, 0.5),
                v_rgb=rng.uf(rows * 3, -1.0, 1.0).reshape(rows, 3))
