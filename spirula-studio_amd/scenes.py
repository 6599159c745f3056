"""Seeded synthetic scenes for the five benchmark configurations.

Random numbers come from counter-based splitmix64 streams, so any slice of any array can be
regenerated independently and the arrays do not depend on generation order. Normals are
Box-Muller on consecutive pairs in float64; the cast to float32 is the last step.

Array layouts are the reference's world buffers (src/primitives/PrimitiveBase3DGS.cuh:87-139):
means [N,3], quats [N,4] (w,x,y,z), log_scales [N,3], opacity_logits [N], features_dc [N,3],
features_sh [N,15,3]; cameras as viewmats [4,4] row-major world->camera and (fx, fy, cx, cy)
(src/engine/EngineSetup.cpp:50-87).
"""
from __future__ import annotations

import ctypes
import dataclasses
import math
import os

import numpy as np

CAM_PINHOLE = 0         # src/core/Common.cuh CameraModelType
CAM_FISHEYE = 1
CAM_EQUISOLID = 2
CAM_EQUIRECT = 3
LENS_NONE, LENS_OPENCV, LENS_THIN_PRISM, LENS_RATIONAL = 0, 1, 2, 3   # CameraDistortionType, src/core/CameraModel.h:37-42
# mild coefficient sets per tier (each in its own order), strong enough to move pixels by several percent
LENS_PRESETS = {
    0: [0, 0, 0, 0, 0, 0, 0, 0],
    1: [0.05, -0.01, 0.002, -0.001, 0, 0, 0, 0],                        # k1 k2 p1 p2
    2: [0.04, -0.008, 0.001, -0.0002, 0.001, -0.0015, 0.0008, -0.0005],  # k1 k2 k3 k4 p1 p2 sx1 sy1
    3: [0.06, 0.01, 0.001, 0.02, 0.005, 0.0005, 0.001, -0.001],          # k1 k2 k3 k4 k5 k6 p1 p2
}

SH_F32 = 0              # fp32 coefficients
SH_REF_Q8 = 1           # uint8 codes + per-block fp32 (min,max), src/core/Tensor.h:1313-1392
SH_REF_Q16 = 2
SH_I8_F16SCALE = 3      # int8 codes * one fp16 scale per Gaussian (benchmark storage format)

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def _splitmix64(z: np.ndarray) -> np.ndarray:
    with np.errstate(over="ignore"):
        z = z + _GOLDEN
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        return z ^ (z >> np.uint64(31))


def _u01(seed: int, stream: int, idx: np.ndarray) -> np.ndarray:
    with np.errstate(over="ignore"):
        base = _splitmix64(np.array([np.uint64(seed) ^ (np.uint64(stream) * _GOLDEN)], dtype=np.uint64))
        h = _splitmix64(base + idx.astype(np.uint64))
    return (h >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)


def _native():
    """The same generators in native code (libssr_host.so), used when that library is built."""
    global _NATIVE
    if _NATIVE is None:
        _NATIVE = False
        so = os.path.join(os.path.dirname(os.path.abspath(__file__)), "host", "libssr_host.so")
        hip = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "libssr_hip.so")
        if os.path.exists(so) and os.path.exists(hip):
            try:
                ctypes.CDLL(hip, mode=ctypes.RTLD_GLOBAL)
                h = ctypes.CDLL(so)
                h.ssrh_rng_uniform.argtypes = [ctypes.c_uint64, ctypes.c_uint64, ctypes.c_int64, ctypes.c_int64,
                                               ctypes.c_double, ctypes.c_double, ctypes.c_void_p]
                h.ssrh_rng_normal.argtypes = [ctypes.c_uint64, ctypes.c_uint64, ctypes.c_int64, ctypes.c_double,
                                              ctypes.c_double, ctypes.c_void_p]
                _NATIVE = h
            except OSError:
                _NATIVE = False
    return _NATIVE


_NATIVE = None


def uniform(seed: int, stream: int, n: int, lo: float, hi: float, start: int = 0) -> np.ndarray:
    h = _native()
    if h:
        out = np.empty(n, np.float32)
        h.ssrh_rng_uniform(seed, stream, start, n, lo, hi, out.ctypes.data)
        return out
    idx = np.arange(start, start + n, dtype=np.uint64)
    return (lo + (hi - lo) * _u01(seed, stream, idx)).astype(np.float32)


def normal(seed: int, stream: int, n: int, mean: float, sigma: float) -> np.ndarray:
    h = _native()
    if h:
        out = np.empty(n, np.float32)
        h.ssrh_rng_normal(seed, stream, n, mean, sigma, out.ctypes.data)
        return out
    idx = np.arange(n, dtype=np.uint64)
    pair = idx >> np.uint64(1)
    u1 = 1.0 - _u01(seed, stream, pair * np.uint64(2))
    u2 = _u01(seed, stream, pair * np.uint64(2) + np.uint64(1))
    r = np.sqrt(-2.0 * np.log(u1))
    a = 2.0 * math.pi * u2
    v = np.where((idx & np.uint64(1)) == 1, r * np.sin(a), r * np.cos(a))
    return (mean + sigma * v).astype(np.float32)


@dataclasses.dataclass
class Scene:
    name: str
    n: int
    width: int
    height: int
    camera_model: int
    viewmat: np.ndarray          # [4,4] float32
    intrins: np.ndarray          # [4] float32 fx fy cx cy
    means: np.ndarray
    quats: np.ndarray
    log_scales: np.ndarray
    opacity_logits: np.ndarray
    features_dc: np.ndarray
    features_sh: np.ndarray      # [N,15,3] float32 (the dequantized values when sh_codec != SH_F32)
    v_rgb: np.ndarray            # [H,W,3]
    v_depth: np.ndarray          # [H,W]
    v_T: np.ndarray              # [H,W]
    sh_codec: int = SH_F32
    sh_packed: np.ndarray | None = None      # uint8 / uint16 / int8 codes
    sh_bounds: np.ndarray | None = None      # [n_bounds,2] float32 (reference codecs)
    sh_bounds_stride: int = 0
    sh_scale_f16: np.ndarray | None = None   # [N] float16 (int8 codec)
    distortion: int = 0                      # lens distortion tier (LENS_*)
    dist_coeffs: np.ndarray | None = None    # [8] float32 in the tier's own order
    antialiased: bool = False                # the "mip" variant of the primitive (blur 0.1, opacity compensation)

    @property
    def tile_w(self) -> int:
        return (self.width + 15) // 16

    @property
    def tile_h(self) -> int:
        return (self.height + 15) // 16


def quantize_ref(values: np.ndarray, bits: int, stride: int):
    """QuantizedTensor<bits,256>::encode_v over blocks of `stride` cells (src/core/Tensor.h:1364-1392).

    Returns (codes, bounds[n_blocks,2], decoded float32 values)."""
    flat = values.reshape(-1).astype(np.float32)
    n = flat.size
    nb = (n + stride - 1) // stride
    pad = nb * stride - n
    padded = np.concatenate([flat, np.full(pad, flat[-1] if n else 0, np.float32)]).reshape(nb, stride)
    lo = padded.min(axis=1).astype(np.float32)
    hi = padded.max(axis=1).astype(np.float32)
    qmax = np.float32(65535.0 if bits == 16 else 255.0)
    rng = np.maximum(hi - lo, np.float32(1e-30)).astype(np.float32)
    t = (qmax * (padded - lo[:, None])).astype(np.float32) / rng[:, None]
    # roundf: half away from zero (operands are non-negative here)
    q = np.clip(np.floor(t.astype(np.float32) + np.float32(0.5)), 0, qmax).astype(np.float32)
    inv = np.float32(1.0) / qmax
    dec = (lo[:, None] + (hi - lo)[:, None] * (q * inv).astype(np.float32)).astype(np.float32)
    codes = q.reshape(-1)[:n].astype(np.uint16 if bits == 16 else np.uint8)
    bounds = np.stack([lo, hi], axis=1).astype(np.float32)
    return codes, bounds, dec.reshape(-1)[:n].reshape(values.shape)


def quantize_i8_f16(values: np.ndarray):
    """int8 codes with one fp16 scale per Gaussian: v = code * scale."""
    v = values.reshape(values.shape[0], -1).astype(np.float32)
    nat = _native()
    if nat is not None and hasattr(nat, "ssrh_quantize_i8_f16") and v.shape[0] >= 100000:
        v = np.ascontiguousarray(v)
        q = np.empty(v.shape, np.int8)
        scale = np.empty(v.shape[0], np.uint16)
        dec = np.empty(v.shape, np.float32)
        nat.ssrh_quantize_i8_f16(ctypes.c_int64(v.shape[0]), ctypes.c_int(v.shape[1]), v.ctypes.data_as(ctypes.c_void_p),
                                 q.ctypes.data_as(ctypes.c_void_p), scale.ctypes.data_as(ctypes.c_void_p),
                                 dec.ctypes.data_as(ctypes.c_void_p))
        return q.reshape(-1), scale.view(np.float16), dec.reshape(values.shape)
    amax = np.abs(v).max(axis=1)
    scale = (amax / np.float32(127.0)).astype(np.float16)
    scale = np.where((scale == 0) & (amax > 0), np.float16(6e-8), scale).astype(np.float16)
    s32 = scale.astype(np.float32)
    safe = np.where(s32 > 0, s32, np.float32(1.0))
    q = np.clip(np.rint(v / safe[:, None]), -127, 127).astype(np.int8)
    q = np.where(s32[:, None] > 0, q, np.int8(0)).astype(np.int8)
    dec = (q.astype(np.float32) * s32[:, None]).astype(np.float32)
    return q.reshape(-1), scale, dec.reshape(values.shape)


def _viewmat(t) -> np.ndarray:
    m = np.eye(4, dtype=np.float32)
    m[:3, 3] = np.asarray(t, np.float32)
    return m


def _common(seed: int, n: int, scale_mu=-4.5, scale_sigma=0.5):
    log_scales = normal(seed, 1, 3 * n, scale_mu, scale_sigma).reshape(n, 3)
    q = normal(seed, 2, 4 * n, 0.0, 1.0).reshape(n, 4).astype(np.float64)
    nrm = np.sqrt((q * q).sum(axis=1, keepdims=True))
    nrm[nrm == 0] = 1.0
    quats = (q / nrm).astype(np.float32)
    opac = normal(seed, 3, n, 0.0, 1.0)
    dc = normal(seed, 4, 3 * n, 0.0, 0.5).reshape(n, 3)
    sh = normal(seed, 5, 45 * n, 0.0, 0.05).reshape(n, 15, 3)
    return log_scales, quats, opac, dc, sh


def _seeds(seed: int, w: int, h: int, parity_variant: bool):
    v_rgb = uniform(seed, 6, 3 * w * h, -1.0, 1.0).reshape(h, w, 3)
    if parity_variant:
        v_depth = uniform(seed, 8, w * h, -0.2, 0.2).reshape(h, w)
        v_T = uniform(seed, 9, w * h, -0.5, 0.5).reshape(h, w)
    else:
        v_depth = np.zeros((h, w), np.float32)
        v_T = np.zeros((h, w), np.float32)
    return v_rgb, v_depth, v_T


# (name, N, W, H, focal, camera model, translation, SH codec, seed)
CONFIGS = {
    1: dict(name="cfg1_100k_800x800", n=100_000, w=800, h=800, f=800.0, model=CAM_PINHOLE,
            t=(0, 0, 4), codec=SH_F32, seed=0xC0FFEE01),
    2: dict(name="cfg2_1M_1080p", n=1_000_000, w=1920, h=1080, f=1500.0, model=CAM_PINHOLE,
            t=(0, 0, 8), codec=SH_F32, seed=0xC0FFEE02),
    3: dict(name="cfg3_3M_q8_1080p", n=3_000_000, w=1920, h=1080, f=1500.0, model=CAM_PINHOLE,
            t=(0, 0, 25), codec=SH_I8_F16SCALE, seed=0xC0FFEE03),
    4: dict(name="cfg4_10M_q8_4k", n=10_000_000, w=3840, h=2160, f=3000.0, model=CAM_PINHOLE,
            t=(0, 0, 0), codec=SH_I8_F16SCALE, seed=0xC0FFEE04),
    5: dict(name="cfg5_6M_equirect", n=6_000_000, w=4096, h=2048, f=4096 / (2 * math.pi),
            model=CAM_EQUIRECT, t=(0, 0, 0), codec=SH_F32, seed=0xC0FFEE05),
}


def make_scene(config: int, n: int | None = None, width: int | None = None,
               height: int | None = None, sh_codec: int | None = None,
               parity_variant: bool = False, seed: int | None = None) -> Scene:
    """Build one of the five configurations; `n`, `width`, `height` shrink it for parity tests
    (focal length and principal point scale with the image width so the framing is kept)."""
    c = CONFIGS[config]
    n = c["n"] if n is None else n
    w = c["w"] if width is None else width
    h = c["h"] if height is None else height
    seed = c["seed"] if seed is None else seed
    f = c["f"] * (w / c["w"])
    codec = c["codec"] if sh_codec is None else sh_codec

    if config == 1:
        means = uniform(seed, 0, 3 * n, -1.0, 1.0).reshape(n, 3)
        rest = _common(seed, n)
    elif config == 2:
        means = uniform(seed, 0, 3 * n, -3.0, 3.0).reshape(n, 3)
        rest = _common(seed, n)
    elif config == 3:
        centres = uniform(seed, 7, 9, -10.0, 10.0).reshape(3, 3)
        which = np.minimum((uniform(seed, 7, n, 0.0, 3.0, start=16)).astype(np.int64), 2)
        means = (centres[which] + normal(seed, 0, 3 * n, 0.0, 1.5).reshape(n, 3)).astype(np.float32)
        rest = _common(seed, n)
    elif config == 4:
        u = uniform(seed, 0, 3 * n, 0.0, 1.0).reshape(n, 3)
        means = np.stack([u[:, 0] * 40 - 20, u[:, 1] * 10 - 5, u[:, 2] * 40 - 20], axis=1).astype(np.float32)
        rest = _common(seed, n, -5.5, 0.7)
    elif config == 5:
        d = normal(seed, 0, 3 * n, 0.0, 1.0).reshape(n, 3).astype(np.float64)
        d /= np.maximum(np.sqrt((d * d).sum(axis=1, keepdims=True)), 1e-12)
        r = uniform(seed, 7, n, 5.0, 30.0).astype(np.float64)
        means = (d * r[:, None]).astype(np.float32)
        rest = _common(seed, n)
    else:
        raise ValueError(f"unknown config {config}")
    log_scales, quats, opac, dc, sh = rest
    v_rgb, v_depth, v_T = _seeds(seed, w, h, parity_variant)
    sc = Scene(name=c["name"], n=n, width=w, height=h, camera_model=c["model"],
               viewmat=_viewmat(c["t"]),
               intrins=np.array([f, f, w / 2.0, h / 2.0], np.float32),
               means=means, quats=quats, log_scales=log_scales, opacity_logits=opac,
               features_dc=dc, features_sh=sh, v_rgb=v_rgb, v_depth=v_depth, v_T=v_T)
    apply_sh_codec(sc, codec)
    return sc


def apply_sh_codec(sc: Scene, codec: int, bounds_stride: int = 256) -> None:
    """Quantize features_sh in place of the fp32 storage; features_sh becomes the decoded values."""
    sc.sh_codec = codec
    if codec == SH_F32:
        return
    if codec in (SH_REF_Q8, SH_REF_Q16):
        bits = 8 if codec == SH_REF_Q8 else 16
        stride = bounds_stride if bounds_stride > 0 else 256 * 45
        codes, bounds, dec = quantize_ref(sc.features_sh, bits, stride)
        sc.sh_packed, sc.sh_bounds, sc.sh_bounds_stride = codes, bounds, bounds_stride
        sc.features_sh = dec
    elif codec == SH_I8_F16SCALE:
        codes, scale, dec = quantize_i8_f16(sc.features_sh)
        sc.sh_packed, sc.sh_scale_f16 = codes, scale
        sc.features_sh = dec
    else:
        raise ValueError(f"unknown SH codec {codec}")


def subset(sc: Scene, idx: np.ndarray) -> Scene:
    """The scene restricted to the splats `idx` (same camera and cotangents). Per-splat codecs keep
    their codes; the block-wise reference codecs become fp32 storage of the decoded values, which
    projects to the same bits."""
    idx = np.asarray(idx, np.int64)
    out = dataclasses.replace(
        sc, n=int(idx.size), means=np.ascontiguousarray(sc.means[idx]), quats=np.ascontiguousarray(sc.quats[idx]),
        log_scales=np.ascontiguousarray(sc.log_scales[idx]), opacity_logits=np.ascontiguousarray(sc.opacity_logits[idx]),
        features_dc=np.ascontiguousarray(sc.features_dc[idx]), features_sh=np.ascontiguousarray(sc.features_sh[idx]))
    if sc.sh_codec == SH_I8_F16SCALE:
        out.sh_packed = np.ascontiguousarray(sc.sh_packed.reshape(sc.n, -1)[idx])
        out.sh_scale_f16 = np.ascontiguousarray(sc.sh_scale_f16[idx])
    elif sc.sh_codec != SH_F32:
        out.sh_codec, out.sh_packed, out.sh_bounds, out.sh_bounds_stride = SH_F32, None, None, 0
    return out


def with_lens(sc: Scene, tier: int) -> Scene:
    """The scene seen through a lens of the given distortion tier."""
    return dataclasses.replace(sc, distortion=int(tier), dist_coeffs=np.array(LENS_PRESETS[int(tier)], np.float32))


def tiny_scene(n: int = 300, width: int = 64, height: int = 48, seed: int = 7,
               camera_model: int = CAM_PINHOLE, big: bool = True) -> Scene:
    """A small scene with large, overlapping splats (many tiles per splat, early termination)."""
    if camera_model == CAM_PINHOLE:
        means = uniform(seed, 0, 3 * n, -1.0, 1.0).reshape(n, 3)
        t, f = (0, 0, 4), float(width)
    elif camera_model in (CAM_FISHEYE, CAM_EQUISOLID):
        # splats all around a camera whose image width spans 180 degrees: those behind it fall outside
        d = normal(seed, 0, 3 * n, 0.0, 1.0).reshape(n, 3).astype(np.float64)
        d /= np.maximum(np.sqrt((d * d).sum(axis=1, keepdims=True)), 1e-12)
        means = (d * uniform(seed, 7, n, 2.0, 6.0).astype(np.float64)[:, None]).astype(np.float32)
        t, f = (0, 0, 0), width / math.pi
    else:
        d = normal(seed, 0, 3 * n, 0.0, 1.0).reshape(n, 3).astype(np.float64)
        d /= np.maximum(np.sqrt((d * d).sum(axis=1, keepdims=True)), 1e-12)
        means = (d * uniform(seed, 7, n, 2.0, 6.0).astype(np.float64)[:, None]).astype(np.float32)
        t, f = (0, 0, 0), width / (2 * math.pi)
    log_scales, quats, opac, dc, sh = _common(seed, n, -2.0 if big else -3.5, 0.6)
    opac = (opac + np.float32(1.0)).astype(np.float32)
    v_rgb, v_depth, v_T = _seeds(seed, width, height, True)
    return Scene(name="tiny", n=n, width=width, height=height, camera_model=camera_model,
                 viewmat=_viewmat(t), intrins=np.array([f, f, width / 2.0, height / 2.0], np.float32),
                 means=means, quats=quats, log_scales=log_scales, opacity_logits=opac,
                 features_dc=dc, features_sh=sh, v_rgb=v_rgb, v_depth=v_depth, v_T=v_T)
