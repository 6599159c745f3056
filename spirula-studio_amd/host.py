"""ctypes binding of libssr_host.so: the C++ host layer that mirrors the reference's backend
interface and engine call order (spirula-studio_amd/host/ssr_engine.hpp). Fails loudly when the
library is not built."""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

from . import lib as _lib

_HERE = os.path.dirname(os.path.abspath(__file__))
SO_PATH = os.path.join(_HERE, "host", "libssr_host.so")

vp = C.c_void_p
SYMBOLS = {
    "ssrh_last_error": (C.c_char_p, []),
    "ssrh_init": (C.c_int, [C.c_int]),
    "ssrh_reset": (C.c_int, []),
    "ssrh_set_options": (C.c_int, [C.c_int] * 8),
    "ssrh_set_data_3dgs": (C.c_int, [C.c_int64, vp, vp, vp, vp, vp, vp, C.c_int]),
    "ssrh_set_sh_value_quant": (C.c_int, [C.c_int, vp, C.c_int64, C.c_int, vp, C.c_int64, C.c_int, C.c_int64]),
    "ssrh_set_camera_params": (C.c_int, [C.c_int, C.c_int, C.c_char_p, C.c_char_p, vp, vp, vp, C.c_int]),
    "ssrh_backward_with_variants": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, C.c_int]),
    "ssrh_backward_fused_optimizer": (C.c_int, [vp, vp, vp, vp, C.c_int, C.c_int, C.c_int, C.c_int]),
    "ssrh_copy_non_sh_quant_state": (C.c_int, [vp, vp]),
    "ssrh_backward_with_pose_grad": (C.c_int, [vp, vp, vp, vp]),
    "ssrh_copy_sh_quant_state": (C.c_int, [vp, vp, vp, vp]),
    "ssrh_copy_params_to_host": (C.c_int, [vp, vp, vp, vp, vp, vp]),
    "ssrh_set_tile_mask": (C.c_int, [vp, C.c_int, C.c_int]),
    "ssrh_set_loss_map": (C.c_int, [vp, C.c_int]),
    "ssrh_set_deferred_counts": (C.c_int, [C.c_int, C.c_int64]),
    "ssrh_deferred_capacity": (C.c_int64, []),
    "ssrh_set_packed_world_rows": (C.c_int, [C.c_int]),
    "ssrh_set_backward_schedule": (C.c_int, [C.c_int]),
    "ssrh_forward_3dgs": (C.c_int, [C.c_char_p, C.c_int, C.c_int, C.c_int, C.c_int]),
    "ssrh_backward_from_render_grad": (C.c_int, [vp, vp, vp]),
    "ssrh_copy_render_to_host": (C.c_int, [vp, vp, vp]),
    "ssrh_copy_grads_to_host": (C.c_int, [vp] * 6),
    "ssrh_cache_pointer": (C.c_int, [C.c_int, C.POINTER(vp), C.POINTER(C.c_int64)]),
    "ssrh_last_n_isects": (C.c_int64, []),
    "ssrh_last_n_visible": (C.c_int64, []),
    "ssrh_short_frames": (C.c_int64, []),
    "ssrh_last_stage_times": (C.c_int, [vp]),
    "ssrh_time_iterations": (C.c_int, [C.c_int, C.c_int, vp, vp, vp, C.c_int, vp]),
    "ssrh_pool_bytes": (C.c_size_t, []),
    "ssrh_sort_pairs_i64_i32": (C.c_int, [vp, vp, vp, vp, C.c_int64, C.c_int, C.c_int, C.POINTER(C.c_int)]),
    "ssrh_inclusive_sum_i64": (C.c_int, [vp, vp, C.c_int64]),
}

_h = None


def load():
    global _h
    if _h is None:
        _lib.load()   # libssr_hip.so first: the host library links against it
        if not os.path.exists(SO_PATH):
            raise _lib.SsrError(f"{SO_PATH} is not built; run `make -C {os.path.dirname(SO_PATH)}`")
        h = C.CDLL(SO_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(h, name)
            fn.restype, fn.argtypes = res, args
        _h = h
    return _h


def check(rc):
    if rc != 0:
        raise _lib.SsrError(load().ssrh_last_error().decode() or f"host error {rc}")


_MODEL = {0: b"PINHOLE", 1: b"FISHEYE", 2: b"EQUISOLID", 3: b"EQUIRECTANGULAR"}
_LENS = {0: b"NONE", 1: b"OPENCV", 2: b"THIN_PRISM", 3: b"RATIONAL"}

CACHE = dict(aabb=(0, np.float32), sort_depth=(1, np.float32), xy=(2, np.float32), depth=(3, np.float32),
             conic=(4, np.float32), opac=(5, np.float32), rgb=(6, np.float32), sorted_ids=(7, np.int64),
             sorted_flat=(8, np.int32), offsets=(9, np.int32), last_ids=(10, np.int32), radii=(11, np.float32),
             v_xy=(12, np.float32), v_depth=(13, np.float32), v_conic=(14, np.float32), v_opac=(15, np.float32),
             v_rgb=(16, np.float32), gaussian_ids=(17, np.int32), camera_ids=(18, np.int32),
             dist_rgb=(19, np.float32), dist_depth=(20, np.float32), median=(21, np.float32),
             accum_weight=(22, np.float32))


class Engine:
    """Drives the engine harness for one scene: upload once, then forward / backward."""

    def __init__(self, scene, device=0, fuse_tile_count=True, visible_list=True, packed_rows=True, overwrite_world_grads=True,
                 stage_profiling=False, sh_degree=3, packed_projection=False, packed_vscreen=True,
                 tile_sort=True, deferred_counts=False, packed_world_rows=False, backward_schedule=-1):
        """packed_projection: forward_3dgs(packed=true), the compacted projection outputs of
        projection_3dgs_packed_forward (the visible-splat work list then has no role).
        packed_world_rows (with packed_projection): that projection also keeps each visible splat's parameters as
        64 bytes in four planes, which the projection backward reads instead of gathering from five arrays.
        backward_schedule: -1 lets the adapter choose the cut of the compositing backward, 0 / 1 force rows / lanes.
        deferred_counts (with tile_sort): after the first iteration the forward no longer waits for the
        intersection count; see set_deferred_counts."""
        self.h = load()
        self.packed_projection = bool(packed_projection)
        self.dist_type, self.output_median = 0, False   # variants of the next forward (set_variants)
        self.sc = scene
        self.sh_degree = sh_degree
        check(self.h.ssrh_init(device))
        check(self.h.ssrh_reset())
        self.opts = [int(fuse_tile_count), int(visible_list), int(packed_rows), int(overwrite_world_grads),
                     int(scene.sh_codec == 3)]
        self.packed_vscreen = int(packed_vscreen)
        self.tile_sort = int(tile_sort)
        check(self.h.ssrh_set_options(*self.opts, int(stage_profiling), self.packed_vscreen, self.tile_sort))
        self.set_deferred_counts(deferred_counts, 0)
        check(self.h.ssrh_set_packed_world_rows(int(bool(packed_world_rows))))
        check(self.h.ssrh_set_backward_schedule(int(backward_schedule)))
        f32 = lambda a: np.ascontiguousarray(a, np.float32)
        self._keep = [f32(scene.means), f32(scene.quats), f32(scene.log_scales), f32(scene.opacity_logits),
                      f32(scene.features_dc), f32(scene.features_sh)]
        p = [a.ctypes.data for a in self._keep]
        check(self.h.ssrh_set_data_3dgs(scene.n, *p, 15))
        if scene.sh_codec != 0:
            packed = np.ascontiguousarray(scene.sh_packed)
            if scene.sh_codec == 3:
                bounds = np.ascontiguousarray(scene.sh_scale_f16.view(np.uint16))
                bits = 8
            else:
                bounds = np.ascontiguousarray(scene.sh_bounds, np.float32).reshape(-1, 2)
                bits = 8 if scene.sh_codec == 1 else 16
            be = bounds.itemsize if scene.sh_codec == 3 else 8
            check(self.h.ssrh_set_sh_value_quant(bits, packed.ctypes.data, packed.size, packed.itemsize,
                                                 bounds.ctypes.data, bounds.shape[0], be, scene.sh_bounds_stride))
        # a [C,4,4] viewmat (with [C,4] intrins, [C,8] coefficients and [C,H,W,...] cotangents) renders C
        # cameras in one pass; a [4,4] one is the single camera
        vm, it = f32(scene.viewmat), f32(scene.intrins)
        self.num_cameras = vm.shape[0] if vm.ndim == 3 else 1
        tier = int(getattr(scene, "distortion", 0))
        dc = f32(np.zeros(8 * self.num_cameras) if getattr(scene, "dist_coeffs", None) is None else scene.dist_coeffs)
        assert vm.size == 16 * self.num_cameras and it.size == 4 * self.num_cameras and dc.size == 8 * self.num_cameras
        check(self.h.ssrh_set_camera_params(scene.width, scene.height, _MODEL[scene.camera_model], _LENS[tier],
                                            vm.ctypes.data, it.ctypes.data, dc.ctypes.data, self.num_cameras))
        assert np.size(scene.v_T) == self.num_cameras * scene.height * scene.width
        # cotangents resident on the device
        self.d_vrgb = _lib.DeviceArray.from_host(f32(scene.v_rgb))
        self.d_vdepth = _lib.DeviceArray.from_host(f32(scene.v_depth))
        self.d_vT = _lib.DeviceArray.from_host(f32(scene.v_T))

    def set_stage_profiling(self, on):
        check(self.h.ssrh_set_options(*self.opts, int(on), self.packed_vscreen, self.tile_sort))

    def set_tile_mask(self, mask):
        """Tile-skip map for the next forward only, from a [h_mask, w_mask] byte mask (one camera) or a
        [C, h_mask, w_mask] stack with one mask per camera of the set."""
        mask = np.ascontiguousarray(mask, np.uint8)
        check(self.h.ssrh_set_tile_mask(mask.ctypes.data, mask.shape[-2], mask.shape[-1]))

    def forward(self):
        """The scene's `antialiased` flag selects the reference's "mip" primitive."""
        primitive = b"mip" if getattr(self.sc, "antialiased", False) else b"3dgs"
        check(self.h.ssrh_forward_3dgs(primitive, self.sh_degree, int(self.packed_projection), int(self.output_median),
                                       int(self.dist_type)))

    def set_variants(self, dist_type=0, median=False):
        """dist_type 0 none / 1 depth / 2 rgb+depth distortion; median: also render the median depth."""
        self.dist_type, self.output_median = int(dist_type), bool(median)

    def backward_with_variants(self, v_dist_rgb=None, v_dist_depth=None, v_median=None, accum_map=None, accum_mode=0):
        f32 = lambda a: None if a is None else np.ascontiguousarray(a, np.float32)
        keep = [f32(v_dist_rgb), f32(v_dist_depth), f32(v_median), f32(accum_map)]
        ptr = lambda a: None if a is None else a.ctypes.data
        check(self.h.ssrh_backward_with_variants(self.d_vrgb.ptr, self.d_vdepth.ptr, self.d_vT.ptr, ptr(keep[0]), ptr(keep[1]),
                                                 ptr(keep[2]), ptr(keep[3]), int(accum_mode)))

    def backward(self):
        check(self.h.ssrh_backward_from_render_grad(self.d_vrgb.ptr, self.d_vdepth.ptr, self.d_vT.ptr))

    def backward_with_pose_grad(self):
        """The backward plus the camera-pose gradient: returns dL/d[R|t] as [4,4] (last row zero)."""
        out = np.zeros((self.num_cameras, 4, 4), np.float32)
        check(self.h.ssrh_backward_with_pose_grad(self.d_vrgb.ptr, self.d_vdepth.ptr, self.d_vT.ptr, out.ctypes.data))
        return out if self.num_cameras > 1 else out[0]

    HYPER = ["lr_means", "lr_quats", "lr_scales", "lr_opacs", "lr_features_dc", "lr_features_sh", "max_gauss_ratio",
             "scale_regularization_weight", "mcmc_opacity_reg_weight", "mcmc_scale_reg_weight", "quat_norm_reg_weight",
             "sh_reg_weight", "erank_reg_weight", "erank_reg_weight_s3", "color_trust_linear", "eps_tr"]

    def set_deferred_counts(self, on, capacity=None):
        """on: the forward sizes its key arrays from the previous iteration's intersection count (plus 1/16 and
        65536 entries) and leaves the count on the device instead of waiting for it; the backward (or n_isects)
        raises if the count turned out larger, and the iteration must then be repeated (the next forward reads its
        count). capacity: entries for the next forward's arrays; 0 makes it read its count; None keeps the current."""
        check(self.h.ssrh_set_deferred_counts(int(bool(on)), -1 if capacity is None else int(capacity)))

    @property
    def deferred_capacity(self):
        return int(self.h.ssrh_deferred_capacity())

    def set_loss_map(self, device_ptr, accum_mode):
        """The [C,H,W] loss map (a device pointer that stays valid) the fused training step accumulates per splat:
        accum_mode 1 max, 2 sum, 3 avg; None or 0 switches it off."""
        check(self.h.ssrh_set_loss_map(device_ptr, int(accum_mode)))

    def backward_fused_optimizer(self, hyper, step, scale_agnostic_mean=False, quantization_level=0, non_sh_optim_bits=32):
        """Compositing backward, then the projection backward fused with the Adam step: the engine's
        parameters and its Adam moments are updated in place. quantization_level 1: quantized SH values and
        moments; non_sh_optim_bits 16 (with level 1): the other moments as 16-bit cells too."""
        hv = np.array([hyper.get(k, 0.0) for k in self.HYPER], np.float32)
        check(self.h.ssrh_backward_fused_optimizer(self.d_vrgb.ptr, self.d_vdepth.ptr, self.d_vT.ptr, hv.ctypes.data, int(step),
                                                   int(scale_agnostic_mean), int(quantization_level), int(non_sh_optim_bits)))

    def non_sh_quant_state(self):
        """non_sh_optim_bits 16: the engine's quantized non-SH moments, per tensor (means, quats, log_scales,
        opacity_logits, features_dc) the 32-bit cells and the [blocks, 4] bounds."""
        n = self.sc.n
        nb = (n + 255) // 256
        pk, bd = np.zeros(n * 14, np.uint32), np.zeros((5, nb, 4), np.float32)
        check(self.h.ssrh_copy_non_sh_quant_state(pk.ctypes.data, bd.ctypes.data))
        off = [0, 3, 7, 10, 11, 14]
        return dict(packed=[pk[n * off[t]: n * off[t + 1]].copy() for t in range(5)], bounds=[bd[t].copy() for t in range(5)])

    def sh_quant_state(self):
        """Quantization level 1: the engine's SH moments and values as host arrays."""
        n, R = self.sc.n, 45
        nb = (n + 255) // 256
        q = dict(state_packed=np.zeros(n * R, np.uint16), state_bounds=np.zeros((nb, 4), np.float32),
                 value_packed=np.zeros(n * R, np.uint16), value_bounds=np.zeros((nb, 2), np.float32), num_sh_buffer=15)
        check(self.h.ssrh_copy_sh_quant_state(*[q[k].ctypes.data for k in ["state_packed", "state_bounds", "value_packed", "value_bounds"]]))
        return q

    def params(self):
        n = self.sc.n
        g = dict(means=np.zeros((n, 3), np.float32), quats=np.zeros((n, 4), np.float32),
                 log_scales=np.zeros((n, 3), np.float32), opacity_logits=np.zeros(n, np.float32),
                 features_dc=np.zeros((n, 3), np.float32), features_sh=np.zeros((n, 15, 3), np.float32))
        check(self.h.ssrh_copy_params_to_host(*[g[k].ctypes.data for k in
                                                ["means", "quats", "log_scales", "opacity_logits", "features_dc", "features_sh"]]))
        return g

    def time_iterations(self, iters):
        ms = np.zeros(iters, np.float32)
        check(self.h.ssrh_time_iterations(self.sh_degree, int(self.packed_projection), self.d_vrgb.ptr, self.d_vdepth.ptr, self.d_vT.ptr,
                                          iters, ms.ctypes.data))
        return ms

    def stage_times(self):
        t = np.zeros(9, np.float32)
        check(self.h.ssrh_last_stage_times(t.ctypes.data))
        return dict(zip(["K1", "K2", "K3", "K4", "K5", "K6", "K7", "K8", "K9"], [float(v) for v in t]))

    @property
    def n_isects(self):
        v = int(self.h.ssrh_last_n_isects())
        if v == -2:
            check(1)
        return v

    @property
    def short_frames(self):
        """Intersections so far that did not fit the arrays they were left to (deferred counts)."""
        return int(self.h.ssrh_short_frames())

    def render(self):
        h, w = self.sc.height, self.sc.width
        lead = (self.num_cameras,) if self.num_cameras > 1 else ()
        rgb, depth, T = np.zeros(lead + (h, w, 3), np.float32), np.zeros(lead + (h, w), np.float32), np.zeros(lead + (h, w), np.float32)
        check(self.h.ssrh_copy_render_to_host(rgb.ctypes.data, depth.ctypes.data, T.ctypes.data))
        return rgb, depth, T

    def grads(self):
        n = self.sc.n
        g = dict(v_means=np.zeros((n, 3), np.float32), v_quats=np.zeros((n, 4), np.float32),
                 v_scales=np.zeros((n, 3), np.float32), v_opacities=np.zeros(n, np.float32),
                 v_dc=np.zeros((n, 3), np.float32), v_sh=np.zeros((n, 15, 3), np.float32))
        check(self.h.ssrh_copy_grads_to_host(*[g[k].ctypes.data for k in
                                               ["v_means", "v_quats", "v_scales", "v_opacities", "v_dc", "v_sh"]]))
        return g

    def cache(self, name):
        which, dt = CACHE[name]
        ptr, cnt = vp(), C.c_int64()
        check(self.h.ssrh_cache_pointer(which, C.byref(ptr), C.byref(cnt)))
        out = np.zeros(cnt.value, dt)
        if cnt.value:
            _lib.check(_lib.load().ssr_memcpy(out.ctypes.data, ptr, out.nbytes, _lib.D2H, None, 0))
        return out
