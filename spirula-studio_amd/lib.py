"""ctypes binding of libssr_hip.so, the C ABI declared in include/ssr_backend.h.

Loading fails loudly when the library has not been built (`make -C spirula-studio_amd/csrc` or
`__graft_entry__.build()`); there is no fallback path.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
SO_PATH = os.path.join(_HERE, "csrc", "libssr_hip.so")

CAM_PINHOLE, CAM_FISHEYE, CAM_EQUISOLID, CAM_EQUIRECT = 0, 1, 2, 3
LENS_NONE, LENS_OPENCV, LENS_THIN_PRISM, LENS_RATIONAL = 0, 1, 2, 3
SH_F32, SH_REF_Q8, SH_REF_Q16, SH_I8_F16SCALE = 0, 1, 2, 3
H2D, D2H, D2D, H2H, AUTO = 0, 1, 2, 3, 4

vp = C.c_void_p


class World(C.Structure):
    _fields_ = [("means", vp), ("quats", vp), ("log_scales", vp), ("opacity_logits", vp),
                ("features_dc", vp), ("features_sh", vp), ("sh_stride", C.c_int32)]


class Screen(C.Structure):
    _fields_ = [("xy", vp), ("depth", vp), ("conic", vp), ("opac", vp), ("rgb", vp)]


class ShQuant(C.Structure):
    _fields_ = [("codec", C.c_int32), ("packed", vp), ("bounds", vp), ("bounds_stride", C.c_int64),
                ("num_sh_buffer", C.c_uint32), ("scale_f16", vp)]


class Camera(C.Structure):
    _fields_ = [("camera_model", C.c_int32), ("num_cameras", C.c_uint32), ("width", C.c_uint32),
                ("height", C.c_uint32), ("viewmats", vp), ("intrins", vp), ("dist_coeffs", vp),
                ("distortion", C.c_int32)]


class ProjectionFwdParams(C.Structure):
    _fields_ = [("num_splats", C.c_int64), ("sh_degree", C.c_int32), ("world", World),
                ("sh", ShQuant), ("camera", Camera), ("aabb", vp), ("sort_depth", vp),
                ("radii", vp), ("screen", Screen), ("tiles_per_splat", vp), ("visible_ids", vp),
                ("visible_count", vp), ("packed_rows", vp),
                ("antialiased", C.c_int32), ("radii_store", C.c_int32), ("clear_count", vp)]


class RasterFwdParams(C.Structure):
    _fields_ = [("num_splats", C.c_int64), ("screen", Screen), ("width", C.c_uint32),
                ("height", C.c_uint32), ("tile_offsets", vp), ("flatten_ids", vp),
                ("n_isects", C.c_int64), ("render_rgb", vp), ("render_depth", vp),
                ("render_T", vp), ("last_ids", vp), ("packed_rows", vp), ("dist_type", C.c_int32),
                ("distortion_rgb", vp), ("distortion_depth", vp), ("render_median", vp),
                ("num_images", C.c_int32), ("tile_order", vp), ("tile_offsets_closed", C.c_int32), ("block_masks", vp)]


class RasterBwdParams(C.Structure):
    _fields_ = [("num_splats", C.c_int64), ("screen", Screen), ("width", C.c_uint32),
                ("height", C.c_uint32), ("tile_offsets", vp), ("flatten_ids", vp),
                ("n_isects", C.c_int64), ("render_T", vp), ("last_ids", vp), ("render_depth", vp),
                ("v_render_rgb", vp), ("v_render_depth", vp), ("v_render_T", vp),
                ("v_screen", Screen), ("packed_rows", vp), ("v_rows", vp), ("dist_type", C.c_int32), ("render_rgb", vp),
                ("distortion_rgb", vp), ("distortion_depth", vp), ("v_distortion_rgb", vp),
                ("v_distortion_depth", vp), ("v_render_median", vp), ("accum_mode", C.c_int32),
                ("accum_weight_map", vp), ("gaussian_ids", vp), ("num_world", C.c_int64), ("accum_weight", vp),
                ("num_images", C.c_int32), ("tile_order", vp), ("tile_offsets_closed", C.c_int32), ("schedule", C.c_int32), ("block_masks", vp)]


class TileWriteCappedParams(C.Structure):
    _fields_ = [("n", C.c_int64), ("rows_per_image", C.c_int64), ("image_ids", vp), ("num_images", C.c_int32),
                ("aabb", vp), ("sort_depth", vp), ("xy", vp), ("conic", vp), ("opac", vp), ("cum_tiles", vp),
                ("width", C.c_uint32), ("height", C.c_uint32), ("isect_ids", vp), ("flatten_ids", vp),
                ("capacity", C.c_int64), ("visible_ids", vp), ("n_visible", vp),
                ("tile_active", vp)]


class ProjectionBwdParams(C.Structure):
    _fields_ = [("num_splats", C.c_int64), ("sh_degree", C.c_int32), ("world", World),
                ("sh", ShQuant), ("camera", Camera), ("aabb", vp), ("v_screen", Screen),
                ("v_world", World), ("accumulate", C.c_int32), ("visible_ids", vp),
                ("n_visible", C.c_int64), ("packed_gaussian_ids", vp), ("num_packed", C.c_int64), ("v_rows", vp),
                ("v_viewmat", vp),
                ("antialiased", C.c_int32), ("packed_ids_unique", C.c_int32), ("packed_world_rows", vp), ("packed_world_stride", C.c_int64)]


class ProjectionPackedParams(C.Structure):
    _fields_ = [("num_splats", C.c_int64), ("sh_degree", C.c_int32), ("world", World),
                ("sh", ShQuant), ("camera", Camera), ("radii", vp), ("scratch", vp),
                ("scratch_bytes", C.c_size_t), ("nnz", vp), ("max_rows", C.c_int64),
                ("camera_ids", vp), ("gaussian_ids", vp), ("aabb", vp), ("sort_depth", vp),
                ("screen", Screen), ("tiles_per_splat", vp), ("packed_rows", vp),
                ("antialiased", C.c_int32), ("camera_index", C.c_int32), ("world_rows", vp), ("world_rows_stride", C.c_int64), ("stage_world_rows", C.c_int32)]


class FpboParams(C.Structure):
    _fields_ = [("num_splats", C.c_int64), ("sh_degree", C.c_int32), ("world", World), ("camera", Camera),
                ("aabb", vp), ("v_screen", Screen), ("v_rows", vp), ("v_world_in", World), ("g1", World), ("g2", World),
                ("densify_score", vp),
                ("lr_means", C.c_float), ("lr_quats", C.c_float), ("lr_scales", C.c_float), ("lr_opacs", C.c_float),
                ("lr_features_dc", C.c_float), ("lr_features_sh", C.c_float),
                ("max_gauss_ratio", C.c_float), ("scale_regularization_weight", C.c_float),
                ("mcmc_opacity_reg_weight", C.c_float), ("mcmc_scale_reg_weight", C.c_float),
                ("quat_norm_reg_weight", C.c_float), ("sh_reg_weight", C.c_float),
                ("step", C.c_int32), ("steps", vp), ("erank_reg_weight", C.c_float), ("erank_reg_weight_s3", C.c_float),
                ("scale_agnostic_radii", vp), ("packed_row_of", vp), ("sh_state_packed", vp), ("sh_state_bounds", vp),
                ("sh_value_packed", vp), ("sh_value_bounds", vp), ("num_sh_buffer", C.c_uint32),
                ("non_sh_packed", vp * 5), ("non_sh_bounds", vp * 5), ("color_trust_linear", C.c_int32), ("eps_tr", C.c_float),
                ("antialiased", C.c_int32), ("v_sh_in", vp), ("v_sh_in_stride", C.c_int32)]


# every symbol include/ssr_backend.h declares: (name, restype, argtypes)
_i64, _u32, _i32, _sz = C.c_int64, C.c_uint32, C.c_int, C.c_size_t
SYMBOLS = {
    "ssr_projection_fwd": (_i32, [C.POINTER(ProjectionFwdParams), vp]),
    "ssr_projection_packed_scratch_bytes": (_sz, [_i64]),
    "ssr_projection_packed_scratch_bytes_world_rows": (_sz, [_i64]),
    "ssr_projection_packed_mask": (_i32, [C.POINTER(ProjectionPackedParams), vp]),
    "ssr_projection_packed_emit": (_i32, [C.POINTER(ProjectionPackedParams), vp]),
    "ssr_tile_count": (_i32, [_i64, vp, vp, vp, vp, _u32, _u32, vp, vp, vp]),
    "ssr_compute_tile_active": (_i32, [vp, _i32, _i32, _u32, _u32, vp, vp]),
    "ssr_scan_scratch_bytes": (_sz, [_i64]),
    "ssr_inclusive_sum_i64": (_i32, [vp, vp, _i64, vp, vp, _sz, vp]),
    "ssr_inclusive_sum_i64_static": (_i32, [vp, vp, _i64, vp, vp]),
    "ssr_read_i64": (_i32, [vp, C.POINTER(C.c_int64), _i32, vp]),
    "ssr_tile_write": (_i32, [_i64, vp, vp, vp, vp, vp, vp, _u32, _u32, vp, vp, vp, _i64, vp, vp]),
    "ssr_tile_count_images": (_i32, [_i64, _i64, vp, _i32, vp, vp, vp, vp, _u32, _u32, vp, vp, vp]),
    "ssr_tile_write_images": (_i32, [_i64, _i64, vp, _i32, vp, vp, vp, vp, vp, vp, _u32, _u32, vp, vp, vp, vp]),
    "ssr_tile_write_capped": (_i32, [C.POINTER(TileWriteCappedParams), vp]),
    "ssr_sort_scratch_bytes": (_sz, [_i64]),
    "ssr_sort_pairs_u64_i32": (_i32, [vp, vp, vp, vp, _i64, _i32, _i32, C.POINTER(C.c_int), vp, _sz, vp]),
    "ssr_tile_offsets": (_i32, [_i64, vp, _u32, vp, vp]),
    "ssr_tile_order_scratch_bytes": (C.c_size_t, [C.c_uint32]),
    "ssr_tile_order": (_i32, [vp, C.c_uint32, _i64, vp, vp, C.c_size_t, vp]),
    "ssr_sort_end_bit": (_i32, [_u32]),
    "ssr_sort_tile_scratch_bytes": (_sz, [_i64, _u32]),
    "ssr_sort_tile_pairs": (_i32, [vp, vp, vp, vp, _i64, _u32, vp, C.POINTER(C.c_int), vp, _sz, vp]),
    "ssr_sort_tile_pairs_capped": (_i32, [vp, vp, vp, vp, _i64, vp, _u32, vp, C.POINTER(C.c_int), vp, _sz, vp]),
    "ssr_tile_offsets_capped": (_i32, [_i64, vp, vp, _u32, vp, vp]),
    "ssr_raster_fwd": (_i32, [C.POINTER(RasterFwdParams), vp]),
    "ssr_raster_bwd": (_i32, [C.POINTER(RasterBwdParams), vp]),
    "ssr_projection_bwd": (_i32, [C.POINTER(ProjectionBwdParams), vp]),
    "ssr_fused_projection_bwd_optimizer": (_i32, [C.POINTER(FpboParams), vp]),
    "ssr_packed_row_map": (_i32, [vp, _i64, _i64, vp, vp]),
    "ssr_zero_world_rows": (_i32, [C.POINTER(World), vp, _i64, vp, vp, _i64, vp]),
    "ssr_fill_u32": (_i32, [vp, _u32, _i64, vp]),
    "ssr_init": (_i32, [_i32]),
    "ssr_device_count": (_i32, []),
    "ssr_device_name": (C.c_char_p, []),
    "ssr_device_malloc": (vp, [_sz]),
    "ssr_device_free": (_i32, [vp]),
    "ssr_host_malloc_pinned": (vp, [_sz]),
    "ssr_host_free_pinned": (_i32, [vp]),
    "ssr_memcpy": (_i32, [vp, vp, _sz, _i32, vp, _i32]),
    "ssr_memset": (_i32, [vp, _i32, _sz, vp, _i32]),
    "ssr_is_device_pointer": (_i32, [vp]),
    "ssr_device_synchronize": (_i32, []),
    "ssr_stream_synchronize": (_i32, [vp]),
    "ssr_stream_create": (vp, []),
    "ssr_stream_destroy": (_i32, [vp]),
    "ssr_event_create": (vp, []),
    "ssr_event_record": (_i32, [vp, vp]),
    "ssr_event_synchronize": (_i32, [vp]),
    "ssr_event_elapsed_ms": (_i32, [vp, vp, C.POINTER(C.c_float)]),
    "ssr_event_destroy": (_i32, [vp]),
    "ssr_last_error": (C.c_char_p, []),
    "ssr_debug_math": (_i32, [_i32, _i64, vp, vp, vp, vp]),
}


class SsrError(RuntimeError):
    pass


_lib = None


def load():
    """Load libssr_hip.so and set every prototype. Raises if the library is missing."""
    global _lib
    if _lib is None:
        if not os.path.exists(SO_PATH):
            raise SsrError(f"{SO_PATH} is not built; run `make -C {os.path.dirname(SO_PATH)}` "
                           "(there is no CPU fallback)")
        lib = C.CDLL(SO_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def check(rc):
    if rc != 0:
        raise SsrError(load().ssr_last_error().decode() or f"error code {rc}")


class DeviceArray:
    """A device allocation with a numpy-like shape/dtype, owned by this object."""

    def __init__(self, shape, dtype):
        self.shape = tuple(int(s) for s in (shape if isinstance(shape, (tuple, list)) else (shape,)))
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        self.ptr = load().ssr_device_malloc(self.nbytes) if self.nbytes else None
        if self.nbytes and not self.ptr:
            raise SsrError(load().ssr_last_error().decode() or "device allocation failed")

    @classmethod
    def from_host(cls, a):
        a = np.ascontiguousarray(a)
        d = cls(a.shape, a.dtype)
        if d.nbytes:
            check(load().ssr_memcpy(d.ptr, a.ctypes.data, d.nbytes, H2D, None, 0))
        return d

    def to_host(self):
        out = np.empty(self.shape, self.dtype)
        if self.nbytes:
            check(load().ssr_memcpy(out.ctypes.data, self.ptr, self.nbytes, D2H, None, 0))
        return out

    def fill_zero(self, stream=None):
        if self.nbytes:
            check(load().ssr_memset(self.ptr, 0, self.nbytes, stream, 1))

    def free(self):
        if getattr(self, "ptr", None):
            load().ssr_device_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass
