"""ctypes binding of the CPU oracle (oracle/libssr_oracle.so). Test infrastructure only."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_SO = os.path.join(_ROOT, "oracle", "libssr_oracle.so")


class OrCamera(C.Structure):
    _fields_ = [("model", C.c_int32), ("width", C.c_uint32), ("height", C.c_uint32),
                ("viewmat", C.c_float * 16), ("fx", C.c_float), ("fy", C.c_float),
                ("cx", C.c_float), ("cy", C.c_float), ("distortion", C.c_int32), ("dist_coeffs", C.c_float * 8),
                ("antialiased", C.c_int32)]


class OrShSource(C.Structure):
    _fields_ = [("codec", C.c_int32), ("sh_f32", C.c_void_p), ("packed", C.c_void_p),
                ("bounds", C.c_void_p), ("bounds_stride", C.c_int64),
                ("num_sh_buffer", C.c_uint32), ("scale_f16", C.c_void_p)]


def build():
    subprocess.check_call(["make", "-s", "-C", os.path.join(_ROOT, "oracle")])


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
        _lib.or_projection_fwd.restype = C.c_int64
        _lib.or_tile_write.restype = C.c_int64
        _lib.or_num_threads.restype = C.c_int
        _lib.or_erank_reg.restype = C.c_float
    return _lib


def _p(a):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"], "the oracle reads raw row-major buffers"
    return a.ctypes.data_as(C.c_void_p)


def camera_of(scene) -> OrCamera:
    cam = OrCamera()
    cam.model = scene.camera_model
    cam.width, cam.height = scene.width, scene.height
    vm = np.ascontiguousarray(scene.viewmat, np.float32).reshape(-1)
    for i in range(16):
        cam.viewmat[i] = float(vm[i])
    cam.fx, cam.fy, cam.cx, cam.cy = [float(v) for v in scene.intrins]
    cam.distortion = int(getattr(scene, "distortion", 0))
    dc = np.zeros(8, np.float32) if getattr(scene, "dist_coeffs", None) is None else np.asarray(scene.dist_coeffs, np.float32)
    for i in range(8):
        cam.dist_coeffs[i] = float(dc[i])
    cam.antialiased = 1 if getattr(scene, "antialiased", False) else 0
    return cam


def sh_source_of(scene, keep):
    """keep: list that receives arrays which must outlive the struct."""
    s = OrShSource()
    s.codec = scene.sh_codec
    s.num_sh_buffer = 15
    s.bounds_stride = scene.sh_bounds_stride
    if scene.sh_codec == 0:
        a = np.ascontiguousarray(scene.features_sh, np.float32)
        keep.append(a)
        s.sh_f32 = a.ctypes.data
    else:
        a = np.ascontiguousarray(scene.sh_packed)
        keep.append(a)
        s.packed = a.ctypes.data
        if scene.sh_bounds is not None:
            b = np.ascontiguousarray(scene.sh_bounds, np.float32)
            keep.append(b)
            s.bounds = b.ctypes.data
        if scene.sh_scale_f16 is not None:
            h = np.ascontiguousarray(scene.sh_scale_f16.view(np.uint16))
            keep.append(h)
            s.scale_f16 = h.ctypes.data
    return s


def math(op, a, b=None):
    a = np.ascontiguousarray(a, np.float32)
    b = np.ascontiguousarray(a if b is None else b, np.float32)
    out = np.empty_like(a)
    lib().or_math(C.c_int(op), C.c_int64(a.size), _p(a), _p(b), _p(out))
    return out


def projection_fwd(scene, sh_degree=3):
    n = scene.n
    keep = []
    cam, sh = camera_of(scene), sh_source_of(scene, keep)
    o = dict(aabb=np.zeros((n, 4), np.float32), sort_depth=np.zeros(n, np.float32),
             radii=np.zeros(n, np.float32), xy=np.zeros((n, 2), np.float32),
             depth=np.zeros(n, np.float32), conic=np.zeros((n, 3), np.float32),
             opac=np.zeros(n, np.float32), rgb=np.zeros((n, 3), np.float32))
    o["visible"] = lib().or_projection_fwd(
        C.c_int64(n), C.c_int(sh_degree), _p(scene.means), _p(scene.quats), _p(scene.log_scales),
        _p(scene.opacity_logits), _p(scene.features_dc), C.byref(sh), C.byref(cam),
        _p(o["aabb"]), _p(o["sort_depth"]), _p(o["radii"]), _p(o["xy"]), _p(o["depth"]),
        _p(o["conic"]), _p(o["opac"]), _p(o["rgb"]))
    return o


def tile_count(n, aabb, xy, conic, opac, w, h, tile_active=None):
    out = np.zeros(n, np.int64)
    lib().or_tile_count_masked(C.c_int64(n), _p(aabb), _p(xy), _p(conic), _p(opac), C.c_uint32(w),
                               C.c_uint32(h), _p(tile_active), _p(out))
    return out


def compute_tile_active(mask, w, h):
    mask = np.ascontiguousarray(mask, np.uint8)
    out = np.zeros(((h + 15) // 16) * ((w + 15) // 16), np.int32)
    lib().or_compute_tile_active(_p(mask), C.c_int32(mask.shape[0]), C.c_int32(mask.shape[1]), C.c_uint32(w),
                                 C.c_uint32(h), _p(out))
    return out


def inclusive_sum(a):
    a = np.ascontiguousarray(a, np.int64)
    out = np.empty_like(a)
    lib().or_inclusive_sum_i64(C.c_int64(a.size), _p(a), _p(out))
    return out


def tile_write(n, aabb, sort_depth, xy, conic, opac, cum, w, h, tile_active=None):
    k = int(cum[-1]) if n else 0
    ids = np.zeros(k, np.int64)
    flat = np.zeros(k, np.int32)
    lib().or_tile_write_masked.restype = C.c_int64
    pads = lib().or_tile_write_masked(C.c_int64(n), _p(aabb), _p(sort_depth), _p(xy), _p(conic), _p(opac),
                                      _p(cum), C.c_uint32(w), C.c_uint32(h), _p(tile_active), _p(ids), _p(flat))
    return ids, flat, pads


def sort_pairs(keys, vals, begin_bit, end_bit):
    keys = np.ascontiguousarray(keys, np.int64)
    vals = np.ascontiguousarray(vals, np.int32)
    ko, vo = np.empty_like(keys), np.empty_like(vals)
    lib().or_sort_pairs(C.c_int64(keys.size), _p(keys), _p(vals), C.c_int(begin_bit),
                        C.c_int(end_bit), _p(ko), _p(vo))
    return ko, vo


def tile_offsets(sorted_ids, n_tiles):
    out = np.full(n_tiles, -1, np.int32)
    lib().or_tile_offsets(C.c_int64(sorted_ids.size), _p(sorted_ids), C.c_uint32(n_tiles), _p(out))
    return out


def tile_n_bits(n_tiles):
    b = 0
    while (1 << b) <= n_tiles:   # src/kernels/tile/IntersectTile.cu:489-490
        b += 1
    return b


def raster_fwd(n, scr, w, h, offsets, flat, dist_type=0, median=False):
    """dist_type 0 none / 1 depth / 2 rgb+depth distortion; median: also the median depth image."""
    o = dict(rgb=np.zeros((h, w, 3), np.float32), depth=np.zeros((h, w), np.float32),
             T=np.zeros((h, w), np.float32), last_ids=np.zeros((h, w), np.int32))
    if dist_type:
        o["dist_depth"] = np.zeros((h, w), np.float32)
        if dist_type == 2:
            o["dist_rgb"] = np.zeros((h, w, 3), np.float32)
    if median:
        o["median"] = np.zeros((h, w), np.float32)
    stats = np.zeros(5, np.int64)
    lib().or_raster_fwd_ex(C.c_int64(n), _p(scr["xy"]), _p(scr["depth"]), _p(scr["conic"]),
                           _p(scr["opac"]), _p(scr["rgb"]), C.c_uint32(w), C.c_uint32(h), _p(offsets),
                           _p(flat), C.c_int64(flat.size), _p(o["rgb"]), _p(o["depth"]), _p(o["T"]),
                           _p(o["last_ids"]), _p(stats), C.c_int(dist_type), _p(o.get("dist_rgb")),
                           _p(o.get("dist_depth")), _p(o.get("median")))
    o["K_f"], o["K_b"] = int(stats[0]), int(stats[1])
    o["visits_fwd"], o["visits_bwd"], o["visits_bwd_productive"] = int(stats[2]), int(stats[3]), int(stats[4])
    return o


def raster_lane_stats(scr, w, h, offsets, flat, last_ids):
    """Lane statistics of the compositing backward: visits per block size and compositing pairs."""
    out = np.zeros(7, np.int64)
    last_ids = np.ascontiguousarray(last_ids, np.int32)
    lib().or_raster_lane_stats(_p(scr["xy"]), _p(scr["depth"]), _p(scr["conic"]), _p(scr["opac"]), _p(scr["rgb"]),
                               C.c_uint32(w), C.c_uint32(h), _p(offsets), _p(flat), C.c_int64(flat.size),
                               _p(last_ids), _p(out))
    v8, v4, v2, pairs, p8, p4, p2 = (int(x) for x in out)
    return dict(visits={8: v8, 4: v4, 2: v2}, productive={8: p8, 4: p4, 2: p2}, pairs=pairs,
                utilisation={8: pairs / max(1, 64 * v8), 4: pairs / max(1, 16 * v4), 2: pairs / max(1, 4 * v2)})


def raster_bwd(n, scr, w, h, offsets, flat, fwd, v_rgb, v_depth, v_T, with_abs=True, dist_type=0,
               v_dist_rgb=None, v_dist_depth=None, v_median=None, accum_mode=0, accum_map=None,
               gaussian_ids=None, n_world=None):
    g = dict(v_xy=np.zeros((n, 2), np.float32), v_depth=np.zeros(n, np.float32),
             v_conic=np.zeros((n, 3), np.float32), v_opac=np.zeros(n, np.float32),
             v_rgb=np.zeros((n, 3), np.float32))
    abs_terms = np.zeros((n, 10), np.float64) if with_abs else None
    n_world = n if n_world is None else n_world
    if accum_mode:
        g["accum_weight"] = np.zeros(n_world * (2 if accum_mode == 3 else 1), np.float32)
    f32 = lambda a: None if a is None else np.ascontiguousarray(a, np.float32)
    keep = [f32(v_rgb), f32(v_depth), f32(v_T), f32(v_dist_rgb), f32(v_dist_depth), f32(v_median), f32(accum_map),
            None if gaussian_ids is None else np.ascontiguousarray(gaussian_ids, np.int32)]
    lib().or_raster_bwd_ex(C.c_int64(n), _p(scr["xy"]), _p(scr["depth"]), _p(scr["conic"]),
                           _p(scr["opac"]), _p(scr["rgb"]), C.c_uint32(w), C.c_uint32(h), _p(offsets),
                           _p(flat), C.c_int64(flat.size), _p(fwd["T"]), _p(fwd["last_ids"]),
                           _p(fwd["depth"]), _p(keep[0]), _p(keep[1]), _p(keep[2]),
                           _p(g["v_xy"]), _p(g["v_depth"]), _p(g["v_conic"]), _p(g["v_opac"]),
                           _p(g["v_rgb"]), _p(abs_terms), C.c_int(dist_type), _p(fwd["rgb"]), _p(fwd.get("dist_rgb")),
                           _p(fwd.get("dist_depth")), _p(keep[3]), _p(keep[4]), _p(keep[5]), C.c_int(accum_mode),
                           _p(keep[6]), _p(keep[7]), C.c_int64(n_world), _p(g.get("accum_weight")))
    g["abs_terms"] = abs_terms
    return g


def projection_bwd(scene, aabb, vs, sh_degree=3, pose=False):
    """pose=True: also the camera-pose gradient, g["v_viewmat"] [4,4] laid out like the [R|t] view matrix."""
    n = scene.n
    keep = []
    cam, sh = camera_of(scene), sh_source_of(scene, keep)
    g = dict(v_means=np.zeros((n, 3), np.float32), v_quats=np.zeros((n, 4), np.float32),
             v_scales=np.zeros((n, 3), np.float32), v_opacities=np.zeros(n, np.float32),
             v_dc=np.zeros((n, 3), np.float32), v_sh=np.zeros((n, 15, 3), np.float32))
    if pose:
        g["v_viewmat"] = np.zeros((4, 4), np.float32)
    lib().or_projection_bwd_pose(
        C.c_int64(n), C.c_int(sh_degree), _p(scene.means), _p(scene.quats), _p(scene.log_scales),
        _p(scene.opacity_logits), _p(scene.features_dc), C.byref(sh), C.byref(cam), _p(aabb),
        _p(vs["v_xy"]), _p(vs["v_depth"]), _p(vs["v_conic"]), _p(vs["v_opac"]), _p(vs["v_rgb"]),
        _p(g["v_means"]), _p(g["v_quats"]), _p(g["v_scales"]), _p(g["v_opacities"]), _p(g["v_dc"]),
        _p(g["v_sh"]), _p(g.get("v_viewmat")))
    return g


_SCREEN_CHANNELS = [("v_xy", 0), ("v_xy", 1), ("v_depth", None), ("v_conic", 0), ("v_conic", 1), ("v_conic", 2),
                    ("v_opac", None), ("v_rgb", 0), ("v_rgb", 1), ("v_rgb", 2)]   # the order of abs_terms' columns


def world_grad_floors(scene, r, sh_degree=3, afrac=2e-6, arith=4e-6, sens_draws=3, sens_rel=6e-7, sens_factor=4.0, row_ulps=32):
    """Per-element floor of the parameter gradients of pipeline result `r`: how far two correct float32 evaluations
    of the same chain may lie apart in that element. Two parts.

    (a) What the summation-order freedom of the screen gradients becomes after the projection VJP. Screen channel j
    of a splat is a float sum of terms whose magnitudes add up to abs_terms[:, j]; any order of that sum is right to
    afrac * abs_terms, and the VJP's last sum to `arith` of |J_ej v_j| per term. The VJP is linear and the splats are
    independent, so running it on the cotangent (afrac * abs_terms_j + arith * |v_j|) e_j, one screen channel at a
    time, and adding the magnitudes of the results gives sum_j |J_ej| (afrac abs_terms_j + arith |v_j|) for every
    element e at once.

    (b) The conditioning of the VJP itself: an element that is a small difference of large intermediate products
    (a scale gradient is a quadratic form of an indefinite matrix, say) is not defined to 1e-3 by float32 arithmetic
    in any order. A backward-stable evaluation returns the exact result for inputs moved by a few ulp, so the
    spread between correct evaluations is bounded by the element's sensitivity to such moves: the VJP is re-run
    `sens_draws` times with every parameter and screen gradient multiplied by 1 +- sens_rel (about five ulp, random
    signs) and sens_factor times the largest change seen is added to the floor. A well-conditioned element moves by
    1e-6 of itself, far below the 1e-3 bar; one that cancels a thousandfold gets the thousandfold floor."""
    import copy
    vs, aabb, n = r["vscreen"], r["proj"]["aabb"], scene.n
    ab = vs["abs_terms"]
    floors = None
    for j, (name, col) in enumerate(_SCREEN_CHANNELS):
        one = dict(v_xy=np.zeros((n, 2), np.float32), v_depth=np.zeros(n, np.float32), v_conic=np.zeros((n, 3), np.float32),
                   v_opac=np.zeros(n, np.float32), v_rgb=np.zeros((n, 3), np.float32))
        v = vs[name] if col is None else vs[name][:, col]
        c = (afrac * ab[:, j] + arith * np.abs(v.astype(np.float64))).astype(np.float32)
        if col is None:
            one[name][:] = c
        else:
            one[name][:, col] = c
        g = projection_bwd(scene, aabb, one, sh_degree)
        if floors is None:
            floors = {k: np.abs(a.astype(np.float64)) for k, a in g.items()}
        else:
            for k, a in g.items():
                floors[k] += np.abs(a.astype(np.float64))
    base = {k: a.astype(np.float64) for k, a in projection_bwd(scene, aabb, vs, sh_degree).items()}
    rng = np.random.default_rng(20261125)
    jiggle = lambda a: (a.astype(np.float64) * (1.0 + sens_rel * rng.choice([-1.0, 1.0], a.shape))).astype(np.float32)
    spread = {k: np.zeros_like(a) for k, a in base.items()}
    for _ in range(sens_draws):
        sc2 = copy.copy(scene)
        for k in ["means", "quats", "log_scales", "opacity_logits", "features_dc"]:
            setattr(sc2, k, jiggle(getattr(scene, k)))
        if getattr(scene, "sh_codec", 0) == 0 and getattr(scene, "features_sh", None) is not None:
            sc2.features_sh = jiggle(scene.features_sh)
        vs2 = {k: jiggle(vs[k]) for k in ["v_xy", "v_depth", "v_conic", "v_opac", "v_rgb"]}
        g = projection_bwd(sc2, aabb, vs2, sh_degree)
        for k, a in g.items():
            spread[k] = np.maximum(spread[k], np.abs(a.astype(np.float64) - base[k]))
    for k in floors:
        floors[k] += sens_factor * spread[k]
        # (c) the components of one row come out of shared matrix products (a quaternion gradient is tangent to the
        # unit sphere, a scale gradient a diagonal of R^T M R): each inherits roundings of the size of an ulp of the
        # row's largest entry, whatever its own size. row_ulps ulp of that entry are added (2e-6 of it, against the
        # 1e-3 of the row maximum that a norm-wise bar would allow).
        # (An SH gradient is basis value times colour gradient, entry by entry: what its entries share is the
        # direction polynomial, so its "row" is the fifteen coefficients of one colour channel.)
        if base[k].ndim == 3:
            floors[k] += row_ulps * 6e-8 * np.abs(base[k]).max(axis=1, keepdims=True)
        else:
            rows = np.abs(base[k]).reshape(n, -1).max(axis=1)
            floors[k] += (row_ulps * 6e-8 * rows).reshape((n,) + (1,) * (base[k].ndim - 1))
    return floors


HYPER = ["lr_means", "lr_quats", "lr_scales", "lr_opacs", "lr_features_dc", "lr_features_sh", "max_gauss_ratio",
         "scale_regularization_weight", "mcmc_opacity_reg_weight", "mcmc_scale_reg_weight", "quat_norm_reg_weight",
         "sh_reg_weight", "erank_reg_weight", "erank_reg_weight_s3", "color_trust_linear", "eps_tr", "v_in_sh"]
WORLD_KEYS = ["means", "quats", "log_scales", "opacity_logits", "features_dc", "features_sh"]


def fused_projection_bwd_optimizer(scene, aabb, vs, params, g1, g2, hyper, step=1, steps=None, v_in=None,
                                   sh_degree=3, densify=True, radii=None):
    """Updates params / g1 / g2 (dicts of float32 arrays keyed by WORLD_KEYS, fp32 SH [N,15,3]) in place
    and returns the densification score."""
    n = scene.n
    cam = camera_of(scene)
    PF = C.POINTER(C.c_float)

    def ptrs(d):
        arr = (C.c_void_p * 6)()
        for i, k in enumerate(WORLD_KEYS):
            a = None if d is None else d.get(k)
            arr[i] = None if a is None else a.ctypes.data
        return arr
    hv = np.array([hyper.get(k, 0.0) for k in HYPER], np.float32)
    score = np.zeros(n, np.float32) if densify else None
    for d in (params, g1, g2):
        for k in WORLD_KEYS:
            assert d[k].dtype == np.float32 and d[k].flags.c_contiguous
    lib().or_fused_projection_bwd_optimizer(
        C.c_int64(n), C.c_int(sh_degree), *[_p(params[k]) for k in WORLD_KEYS], C.byref(cam), _p(aabb),
        _p(vs["v_xy"]), _p(vs["v_depth"]), _p(vs["v_conic"]), _p(vs["v_opac"]), _p(vs["v_rgb"]),
        ptrs(v_in) if v_in is not None else None, ptrs(g1), ptrs(g2), _p(score), _p(hv), C.c_int32(step),
        _p(None if steps is None else np.ascontiguousarray(steps, np.int32)),
        _p(None if radii is None else np.ascontiguousarray(radii, np.float32)))
    return score


class OrShQuantState(C.Structure):
    _fields_ = [("state_packed", C.c_void_p), ("state_bounds", C.c_void_p), ("value_packed", C.c_void_p),
                ("value_bounds", C.c_void_p), ("num_sh_buffer", C.c_uint32)]


def quant_codec(op, a=None, b=None, mm=None, codes=None):
    """The codecs of the quantized optimizer state on arrays: op 0 Adam-state encode (g1, g2 -> codes),
    1 decode (codes -> g1, g2), 2 16-bit value encode, 3 value decode, 4 / 5 the 16-bit Adam-state encode / decode."""
    mm = np.ascontiguousarray(mm, np.float32)
    if op in (0, 2, 4):
        a = np.ascontiguousarray(a, np.float32)
        b = np.ascontiguousarray(a if b is None else b, np.float32)
        codes = np.zeros(a.size, np.uint32)
        lib().or_quant_codec(C.c_int(op), C.c_int64(a.size), _p(a), _p(b), _p(mm), _p(codes))
        return codes
    codes = np.ascontiguousarray(codes, np.uint32)
    a = np.zeros(codes.size, np.float32)
    b = np.zeros(codes.size, np.float32)
    lib().or_quant_codec(C.c_int(op), C.c_int64(codes.size), _p(a), _p(b), _p(mm), _p(codes))
    return (a, b) if op in (1, 5) else a


def quantize_sh_state(features_sh, num_sh_buffer=15):
    """fp32 SH [N, num_sh_buffer, 3] -> the level-1 state: 16-bit values against per-256-splat (min, max),
    all-zero moments (packed zeros with zero bounds decode to g1 = g2 = 0)."""
    n = features_sh.shape[0]
    R = 3 * num_sh_buffer
    flat = np.ascontiguousarray(features_sh, np.float32).reshape(n, R)
    nb = (n + 255) // 256
    vb = np.zeros((nb, 2), np.float32)
    vp = np.zeros(n * R, np.uint16)
    for blk in range(nb):
        rows = flat[blk * 256:(blk + 1) * 256]
        vb[blk] = [rows.min(), rows.max()]
        vp[blk * 256 * R: blk * 256 * R + rows.size] = quant_codec(2, rows.reshape(-1), mm=vb[blk]).astype(np.uint16)
    return dict(state_packed=np.zeros(n * R, np.uint16), state_bounds=np.zeros((nb, 4), np.float32), value_packed=vp,
                value_bounds=vb, num_sh_buffer=num_sh_buffer)


def decode_sh_values(q, n):
    R = 3 * q["num_sh_buffer"]
    out = np.zeros((n, R), np.float32)
    for blk in range((n + 255) // 256):
        c = q["value_packed"][blk * 256 * R: min((blk + 1) * 256, n) * R]
        out[blk * 256: blk * 256 + c.size // R] = quant_codec(3, codes=c.astype(np.uint32), mm=q["value_bounds"][blk]).reshape(-1, R)
    return out.reshape(n, q["num_sh_buffer"], 3)


def decode_sh_moments(q, n):
    R = 3 * q["num_sh_buffer"]
    g1, g2 = np.zeros((n, R), np.float32), np.zeros((n, R), np.float32)
    for blk in range((n + 255) // 256):
        c = q["state_packed"][blk * 256 * R: min((blk + 1) * 256, n) * R]
        a, b = quant_codec(1, codes=c.astype(np.uint32), mm=q["state_bounds"][blk])
        g1[blk * 256: blk * 256 + c.size // R] = a.reshape(-1, R)
        g2[blk * 256: blk * 256 + c.size // R] = b.reshape(-1, R)
    return g1, g2


class OrNonShQuantState(C.Structure):
    _fields_ = [("packed", C.c_void_p * 5), ("bounds", C.c_void_p * 5)]


NON_SH_KEYS = ["means", "quats", "log_scales", "opacity_logits", "features_dc"]
NON_SH_PRIMS = [3, 4, 3, 1, 3]


def zero_non_sh_state(n):
    """The all-zero quantized non-SH state (decodes to zero moments): per tensor [N * prims] uint32 cells and
    [ceil(N / 256), 4] float32 bounds."""
    nb = (n + 255) // 256
    return dict(packed=[np.zeros(n * p, np.uint32) for p in NON_SH_PRIMS], bounds=[np.zeros((nb, 4), np.float32) for _ in range(5)])


def encode_non_sh_state(g1, g2, n):
    """fp32 moments (dicts keyed by NON_SH_KEYS) -> the quantized non-SH state, by the codec's definition."""
    st = zero_non_sh_state(n)
    for t, (k, prims) in enumerate(zip(NON_SH_KEYS, NON_SH_PRIMS)):
        a, b = g1[k].reshape(-1).astype(np.float32), g2[k].reshape(-1).astype(np.float32)
        for blk in range((n + 255) // 256):
            sl = slice(blk * 256 * prims, min((blk + 1) * 256, n) * prims)
            sq = np.sqrt(np.maximum(b[sl], 0)).astype(np.float32)
            u = (a[sl] / (sq + np.float32(1e-15))).astype(np.float32)
            # log_s through the codec's own log1p: encode a lone cell against (0, 1) bounds is not available, so
            # take the bounds from decode(encode) fixed points: min / max of log1p(sq / eps) computed in float64
            ls = np.log1p(sq.astype(np.float64) / 1e-15).astype(np.float32)
            mm = np.array([u.min(), u.max(), ls.min(), ls.max()], np.float32)
            st["bounds"][t][blk] = mm
            st["packed"][t][sl] = quant_codec(4, a[sl], b[sl], mm=mm)
    return st


def decode_non_sh_state(st, n):
    g1, g2 = {}, {}
    for t, (k, prims) in enumerate(zip(NON_SH_KEYS, NON_SH_PRIMS)):
        a, b = np.zeros(n * prims, np.float32), np.zeros(n * prims, np.float32)
        for blk in range((n + 255) // 256):
            sl = slice(blk * 256 * prims, min((blk + 1) * 256, n) * prims)
            a[sl], b[sl] = quant_codec(5, codes=st["packed"][t][sl], mm=st["bounds"][t][blk])
        shape = (n,) if prims == 1 else (n, prims)
        g1[k], g2[k] = a.reshape(shape), b.reshape(shape)
    return g1, g2


def fused_projection_bwd_optimizer_q(scene, aabb, vs, params, q, g1, g2, hyper, step=1, steps=None, v_in=None,
                                     sh_degree=3, densify=True, radii=None, non_sh=None):
    """The fused optimizer with the SH coefficients and their moments in the quantized state q (updated in
    place); params / g1 / g2 hold the five non-SH arrays (a features_sh entry is ignored). non_sh: the quantized
    state of the non-SH moments (zero_non_sh_state layout, updated in place); g1 / g2 may then be None."""
    n = scene.n
    cam = camera_of(scene)

    def ptrs(d):
        arr = (C.c_void_p * 6)()
        for i, k in enumerate(WORLD_KEYS):
            a = None if d is None or k == "features_sh" else d.get(k)
            arr[i] = None if a is None else a.ctypes.data
        return arr
    hv = np.array([hyper.get(k, 0.0) for k in HYPER], np.float32)
    score = np.zeros(n, np.float32) if densify else None
    st = OrShQuantState()
    for k in ["state_packed", "state_bounds", "value_packed", "value_bounds"]:
        assert q[k].flags.c_contiguous
        setattr(st, k, q[k].ctypes.data)
    st.num_sh_buffer = q["num_sh_buffer"]
    ns = None
    if non_sh is not None:
        ns = OrNonShQuantState()
        for t in range(5):
            assert non_sh["packed"][t].dtype == np.uint32 and non_sh["packed"][t].flags.c_contiguous
            assert non_sh["bounds"][t].dtype == np.float32 and non_sh["bounds"][t].flags.c_contiguous
            ns.packed[t] = non_sh["packed"][t].ctypes.data
            ns.bounds[t] = non_sh["bounds"][t].ctypes.data
    lib().or_fused_projection_bwd_optimizer_q(
        C.c_int64(n), C.c_int(sh_degree), *[_p(params[k]) for k in WORLD_KEYS[:5]], C.byref(st),
        C.byref(ns) if ns is not None else None, C.byref(cam), _p(aabb),
        _p(vs["v_xy"]), _p(vs["v_depth"]), _p(vs["v_conic"]), _p(vs["v_opac"]), _p(vs["v_rgb"]),
        ptrs(v_in) if v_in is not None else None, ptrs(g1), ptrs(g2), _p(score), _p(hv), C.c_int32(step),
        _p(None if steps is None else np.ascontiguousarray(steps, np.int32)),
        _p(None if radii is None else np.ascontiguousarray(radii, np.float32)))
    return score


def colour_map(op, x):
    """op 0: slope of the sRGB curve, 1: splat_dc_encode, 2: splat_dc_decode."""
    x = np.ascontiguousarray(x, np.float32)
    y = np.zeros_like(x)
    lib().or_colour_map(C.c_int(op), C.c_int64(x.size), _p(x), _p(y))
    return y


def erank_reg(log_scales, w, w3):
    """Loss and gradient of the effective-rank regularizer for one splat."""
    ls = np.ascontiguousarray(log_scales, np.float32)
    g = np.zeros(3, np.float32)
    loss = lib().or_erank_reg(_p(ls), C.c_float(w), C.c_float(w3), _p(g))
    return float(loss), g


def pipeline(scene, sh_degree=3, backward=True, tile_active=None, variant=None):
    """The whole iteration in the reference's order (src/engine/EngineForward.cpp:166-293,
    src/engine/EngineLoss.cpp:138-240,359-368). tile_active: optional tile-skip map for the tile stage."""
    n, w, h = scene.n, scene.width, scene.height
    p = projection_fwd(scene, sh_degree)
    counts = tile_count(n, p["aabb"], p["xy"], p["conic"], p["opac"], w, h, tile_active)
    cum = inclusive_sum(counts)
    ids, flat, pads = tile_write(n, p["aabb"], p["sort_depth"], p["xy"], p["conic"], p["opac"], cum, w, h, tile_active)
    n_tiles = scene.tile_w * scene.tile_h
    sk, sv = sort_pairs(ids, flat, 0, 32 + tile_n_bits(n_tiles))
    offs = tile_offsets(sk, n_tiles)
    # variant: dict(dist_type=, median=bool, v_dist_rgb=, v_dist_depth=, v_median=, accum_mode=, accum_map=)
    va = variant or {}
    f = raster_fwd(n, p, w, h, offs, sv, va.get("dist_type", 0), va.get("median", False))
    out = dict(proj=p, counts=counts, cum=cum, isect_ids=ids, flatten_ids=flat, pads=pads,
               sorted_ids=sk, sorted_flat=sv, offsets=offs, fwd=f)
    if backward:
        out["vscreen"] = raster_bwd(n, p, w, h, offs, sv, f, scene.v_rgb, scene.v_depth, scene.v_T,
                                    dist_type=va.get("dist_type", 0), v_dist_rgb=va.get("v_dist_rgb"),
                                    v_dist_depth=va.get("v_dist_depth"), v_median=va.get("v_median") if va.get("median") else None,
                                    accum_mode=va.get("accum_mode", 0), accum_map=va.get("accum_map"))
        out["grads"] = projection_bwd(scene, p["aabb"], out["vscreen"], sh_degree)
    return out


def pack_projection(p):
    """projection_3dgs_packed_forward restated on the unpacked oracle outputs: the visibility mask
    is the clamped-extent test (src/kernels/projection/ProjectionPackedFwd_kernel.cuh:89-93), which
    is exactly the rule under which the unpacked kernel keeps a non-zero aabb
    (src/kernels/projection/ProjectionFwd_kernel.cuh:97-110); the packed arrays are the visible rows
    in ascending splat order (inclusive scan of the mask, ProjectionPackedFwd.cu:112-119)."""
    a = p["aabb"]
    mask = (a[:, 2] - a[:, 0] > np.float32(1e-3)) & (a[:, 3] - a[:, 1] > np.float32(1e-3))
    gids = np.nonzero(mask)[0].astype(np.int32)
    q = {k: np.ascontiguousarray(p[k][gids]) for k in ["aabb", "sort_depth", "xy", "depth", "conic", "opac", "rgb"]}
    q["gaussian_ids"] = gids
    q["camera_ids"] = np.zeros(gids.size, np.int32)
    q["radii"] = p["radii"]
    q["visible"] = int(gids.size)
    return q


def pipeline_packed(scene, sh_degree=3, backward=True, tile_active=None, variant=None):
    """The iteration with packed projection outputs (engine path with packed=true,
    src/engine/EngineForward.cpp:119-162,215-217): every later stage sees nnz rows, flatten ids are
    packed row numbers, v_screen has nnz rows, and the projection backward maps row i to splat
    gaussian_ids[i] (src/kernels/projection/ProjectionBwd_kernel.cuh:51-56)."""
    n, w, h = scene.n, scene.width, scene.height
    full = projection_fwd(scene, sh_degree)
    p = pack_projection(full)
    m = p["visible"]
    counts = tile_count(m, p["aabb"], p["xy"], p["conic"], p["opac"], w, h, tile_active)
    cum = inclusive_sum(counts)
    ids, flat, pads = tile_write(m, p["aabb"], p["sort_depth"], p["xy"], p["conic"], p["opac"], cum, w, h, tile_active)
    n_tiles = scene.tile_w * scene.tile_h
    sk, sv = sort_pairs(ids, flat, 0, 32 + tile_n_bits(n_tiles))
    offs = tile_offsets(sk, n_tiles)
    va = variant or {}
    f = raster_fwd(m, p, w, h, offs, sv, va.get("dist_type", 0), va.get("median", False))
    out = dict(proj=p, full_proj=full, counts=counts, cum=cum, isect_ids=ids, flatten_ids=flat, pads=pads,
               sorted_ids=sk, sorted_flat=sv, offsets=offs, fwd=f)
    if backward:
        vs = raster_bwd(m, p, w, h, offs, sv, f, scene.v_rgb, scene.v_depth, scene.v_T,
                        dist_type=va.get("dist_type", 0), v_dist_rgb=va.get("v_dist_rgb"), v_dist_depth=va.get("v_dist_depth"),
                        v_median=va.get("v_median") if va.get("median") else None, accum_mode=va.get("accum_mode", 0),
                        accum_map=va.get("accum_map"), gaussian_ids=p["gaussian_ids"], n_world=n)
        out["vscreen"] = vs
        shapes = dict(v_xy=(n, 2), v_depth=(n,), v_conic=(n, 3), v_opac=(n,), v_rgb=(n, 3))
        spread = {}
        for k, shp in shapes.items():
            spread[k] = np.zeros(shp, np.float32)
            spread[k][p["gaussian_ids"]] = vs[k]
        out["grads"] = projection_bwd(scene, full["aabb"], spread, sh_degree)
    return out
