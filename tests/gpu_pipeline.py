"""Drives the hot path stage by stage through the C ABI (libssr_hip.so) from Python, for the GPU
parity tests. Mirrors the call order of the reference's engine
(src/engine/EngineForward.cpp:166-293, src/engine/EngineLoss.cpp:138-240,359-368)."""
from __future__ import annotations

import ctypes as C

import numpy as np


WORLD_GRAD_RTOL = 1e-3   # the bar for parameter gradients, relative, per element
MARGINS = {}             # label -> largest err / rowmax seen, for the report at the end of a run


def world_grad_check(got, ref, n, name, rtol=WORLD_GRAD_RTOL, bad_frac=0.0, scale=None, row_floor=None, elem_floor=None):
    """Parameter-gradient bar. With elem_floor (oracle_lib.world_grad_floors: what the summation order of the screen
    gradients can move each element by): per element, |got - ref| <= rtol * |ref| + elem_floor. Without it (runs that
    have no oracle chain to derive the floor from): |got - ref| <= rtol * max|ref row| + a floor of 2e-5 of the
    tensor's mean magnitude. Either way the largest error relative to the row maximum is printed, with and without
    the floor, so that the margin is on record."""
    got = np.asarray(got, np.float64).reshape(n, -1)
    ref = np.asarray(ref, np.float64).reshape(n, -1)
    if scale is None:   # a caller that sums several cameras passes the sum of their row maxima
        scale = np.abs(ref).max(axis=1, keepdims=True)
    scale = scale + 1e-30
    floor = 2e-5 * (np.abs(ref).mean() + 1e-12)
    if row_floor is not None:   # what the summation-order floor of a screen gradient becomes in this row
        floor = floor + np.asarray(row_floor, np.float64).reshape(n, 1)
    err = np.abs(got - ref)
    raw = float((err / scale).max()) if err.size else 0.0
    over = float((np.maximum(err - floor, 0.0) / scale).max()) if err.size else 0.0
    MARGINS[name] = max(MARGINS.get(name, 0.0), over)
    if elem_floor is None:
        print(f"  grad {name}: max err/rowmax {raw:.3e}, beyond the floor {over:.3e} (bar {rtol:.0e})", flush=True)
        bad = err > rtol * scale + floor
        assert bad.mean() <= bad_frac, (name, over, float(bad.mean()))
        return
    ef = np.asarray(elem_floor, np.float64).reshape(n, -1) + 1e-30
    excess = np.maximum(err - ef, 0.0) / (np.abs(ref) + 1e-300)   # relative error left once the floor is taken off
    worst = float(excess.max()) if err.size else 0.0
    print(f"  grad {name}: max err/rowmax {raw:.3e}; per element beyond its floor {worst:.3e} of |ref| (bar {rtol:.0e})", flush=True)
    bad = err > rtol * np.abs(ref) + ef
    if bad.mean() > bad_frac:
        i = np.argwhere(bad)[:4]
        raise AssertionError((name, int(bad.sum()), [(tuple(ix), got[tuple(ix)], ref[tuple(ix)], ef[tuple(ix)]) for ix in i]))


class GpuRun:
    def __init__(self, pkg, scene, sh_degree=3, use_list=False, use_packed=False, packed_projection=False,
                 read_nnz=True, use_vrows=False, tile_sort=False, capacity=None, world_rows=False, bwd_lanes=False, block_masks=False):
        """use_packed: 48-byte fragment rows for the compositing kernels. packed_projection: the
        compacted (nnz-row) projection outputs of projection_3dgs_packed_forward; read_nnz=False
        sizes the outputs for all N splats instead of reading nnz back between the two calls."""
        self.use_list = use_list
        self.use_packed = use_packed
        self.bwd_lanes = bwd_lanes   # SSR_BWD_SCHEDULE_LANES for the compositing backward (plain variant only)
        self.block_masks = block_masks   # the forward records every entry's block mask and the backward reads them
        self.packed_projection = packed_projection
        self.read_nnz = read_nnz
        # world_rows (with packed_projection): the projection also writes each visible splat's parameters (four
        # planes of 16-byte entries), and the projection backward reads those
        self.world_rows = world_rows
        assert packed_projection or not world_rows
        self.tile_sort = tile_sort   # ssr_sort_tile_pairs instead of the whole-key sort + ssr_tile_offsets
        # capacity (with tile_sort): the key arrays hold that many entries and nothing is read back between the scan
        # and the compositing (ssr_tile_write_capped, ssr_sort_tile_pairs_capped, closed offsets)
        self.capacity = capacity
        assert capacity is None or tile_sort
        self.use_vrows = use_vrows   # one 12-float gradient row per splat between K8 and K9
        assert not (packed_projection and use_list)
        self.L = pkg.lib
        self.lib = self.L.load()
        self.check = self.L.check
        self.sc = scene
        self.sh_degree = sh_degree
        D = self.L.DeviceArray
        sc = scene
        n = sc.n
        self.n = n
        self.d = {}
        for k in ["means", "quats", "log_scales", "opacity_logits", "features_dc"]:
            self.d[k] = D.from_host(getattr(sc, k).astype(np.float32))
        if sc.sh_codec == 0:
            self.d["features_sh"] = D.from_host(sc.features_sh.astype(np.float32))
        else:
            self.d["sh_packed"] = D.from_host(sc.sh_packed)
            if sc.sh_bounds is not None:
                self.d["sh_bounds"] = D.from_host(sc.sh_bounds.astype(np.float32))
            if sc.sh_scale_f16 is not None:
                self.d["sh_scale"] = D.from_host(sc.sh_scale_f16.view(np.uint16))
        self.d["viewmat"] = D.from_host(sc.viewmat.astype(np.float32))
        self.d["intrins"] = D.from_host(sc.intrins.astype(np.float32))
        for k, shape in [("aabb", (n, 4)), ("sort_depth", (n,)), ("radii", (n,)), ("xy", (n, 2)),
                         ("depth", (n,)), ("conic", (n, 3)), ("opac", (n,)), ("rgb", (n, 3))]:
            self.d[k] = D(shape, np.float32)
        self.d["counts"] = D((n,), np.int64)
        self.d["cum"] = D((n,), np.int64)
        self.d["vis_ids"] = D((n,), np.int32)
        self.d["counters"] = D((2,), np.int64)     # [n_isects, n_visible]
        self.d["packed"] = D((n, 12), np.float32)
        self.V = None
        self.rows = n          # rows of the projection outputs: N, or nnz in packed mode
        self.tile_active = None   # device tile-skip map (set_tile_mask)
        # variants of the compositing kernels: dict(dist_type=, median=bool, v_dist_rgb=, v_dist_depth=,
        # v_median=, accum_mode=, accum_map=)
        self.variant = {}

    def ptr(self, k):
        a = self.d.get(k)
        return a.ptr if a is not None else None

    def world(self, prefix=""):
        w = self.L.World()
        w.means, w.quats, w.log_scales = self.ptr(prefix + "means"), self.ptr(prefix + "quats"), self.ptr(prefix + "log_scales")
        w.opacity_logits, w.features_dc = self.ptr(prefix + "opacity_logits"), self.ptr(prefix + "features_dc")
        w.features_sh = self.ptr(prefix + "features_sh")
        w.sh_stride = 45
        return w

    def shq(self):
        q = self.L.ShQuant()
        q.codec = self.sc.sh_codec
        q.packed, q.bounds, q.scale_f16 = self.ptr("sh_packed"), self.ptr("sh_bounds"), self.ptr("sh_scale")
        q.bounds_stride = self.sc.sh_bounds_stride
        q.num_sh_buffer = 15
        return q

    def camera(self):
        c = self.L.Camera()
        c.camera_model, c.num_cameras = self.sc.camera_model, 1
        c.width, c.height = self.sc.width, self.sc.height
        c.viewmats, c.intrins = self.ptr("viewmat"), self.ptr("intrins")
        c.distortion = int(getattr(self.sc, "distortion", 0))
        if "dist_coeffs" not in self.d:
            dc = getattr(self.sc, "dist_coeffs", None)
            self.d["dist_coeffs"] = self.L.DeviceArray.from_host(np.zeros(8, np.float32) if dc is None else np.asarray(dc, np.float32))
        c.dist_coeffs = self.ptr("dist_coeffs")
        return c

    def screen(self, prefix=""):
        s = self.L.Screen()
        s.xy, s.depth, s.conic = self.ptr(prefix + "xy"), self.ptr(prefix + "depth"), self.ptr(prefix + "conic")
        s.opac, s.rgb = self.ptr(prefix + "opac"), self.ptr(prefix + "rgb")
        return s

    def set_tile_mask(self, mask):
        """compute_tile_active on the device from a [h_mask, w_mask] byte mask."""
        D = self.L.DeviceArray
        mask = np.ascontiguousarray(mask, np.uint8)
        self.d["mask"] = D.from_host(mask)
        self.d["tile_active"] = D((self.sc.tile_w * self.sc.tile_h,), np.int32)
        self.check(self.lib.ssr_compute_tile_active(self.ptr("mask"), mask.shape[0], mask.shape[1], self.sc.width,
                                                    self.sc.height, self.ptr("tile_active"), None))
        self.tile_active = self.ptr("tile_active")

    # ---- stages ----
    def projection_packed_fwd(self, fused_count=False):
        D = self.L.DeviceArray
        n = self.n
        self.d["radii"].fill_zero()
        sb = (self.lib.ssr_projection_packed_scratch_bytes_world_rows(n) if self.world_rows
              else self.lib.ssr_projection_packed_scratch_bytes(n))
        self.d["pk_scratch"] = D((sb,), np.uint8)
        self.d["nnz"] = D((1,), np.int64)
        p = self.L.ProjectionPackedParams()
        p.num_splats, p.sh_degree = n, self.sh_degree
        p.antialiased = 1 if getattr(self.sc, "antialiased", False) else 0
        p.world, p.sh, p.camera = self.world(), self.shq(), self.camera()
        p.radii, p.scratch, p.scratch_bytes, p.nnz = self.ptr("radii"), self.ptr("pk_scratch"), sb, self.ptr("nnz")
        p.stage_world_rows = 1 if self.world_rows else 0
        self.check(self.lib.ssr_projection_packed_mask(C.byref(p), None))
        if self.read_nnz:
            k = (C.c_int64 * 1)(0)
            self.check(self.lib.ssr_read_i64(self.ptr("nnz"), k, 1, None))
            cap = int(k[0])
        else:
            cap = n
        for nm, shape, dt in [("camera_ids", (cap,), np.int32), ("gaussian_ids", (cap,), np.int32),
                              ("aabb", (cap, 4), np.float32), ("sort_depth", (cap,), np.float32),
                              ("xy", (cap, 2), np.float32), ("depth", (cap,), np.float32),
                              ("conic", (cap, 3), np.float32), ("opac", (cap,), np.float32),
                              ("rgb", (cap, 3), np.float32), ("counts", (cap,), np.int64),
                              ("cum", (cap,), np.int64), ("packed", (cap, 12), np.float32),
                              ("world_rows", (4, cap, 4), np.float32)]:
            self.d[nm] = D(shape, dt)
            if cap:   # poison, so that rows past nnz are seen to stay untouched
                self.check(self.lib.ssr_fill_u32(self.d[nm].ptr, 0x7fc12345, self.d[nm].nbytes // 4, None))
        p.max_rows = cap
        p.camera_ids, p.gaussian_ids = self.ptr("camera_ids"), self.ptr("gaussian_ids")
        p.aabb, p.sort_depth, p.screen = self.ptr("aabb"), self.ptr("sort_depth"), self.screen()
        p.tiles_per_splat = self.ptr("counts") if fused_count else None
        p.packed_rows = self.ptr("packed") if self.use_packed else None
        p.world_rows = self.ptr("world_rows") if self.world_rows else None
        p.world_rows_stride = cap
        self.check(self.lib.ssr_projection_packed_emit(C.byref(p), None))
        if not self.read_nnz:
            k = (C.c_int64 * 1)(0)
            self.check(self.lib.ssr_read_i64(self.ptr("nnz"), k, 1, None))
        self.nnz = self.rows = int(k[0])
        self.cap = cap

    def projection_fwd(self, fused_count=False):
        if self.packed_projection:
            return self.projection_packed_fwd(fused_count)
        # with the work list the launch stores every radius itself (radii_store): the buffer then starts out holding
        # a large value in every row instead of the zero-fill, and a spare counter must come back cleared
        store = bool(self.use_list)
        if store:
            self.check(self.lib.ssr_fill_u32(self.ptr("radii"), 0x7F000000, self.n, None))
            self.d["spare_count"] = self.L.DeviceArray.from_host(np.array([12345], np.int64))
        else:
            self.d["radii"].fill_zero()
        p = self.L.ProjectionFwdParams()
        p.radii_store = 1 if store else 0
        p.clear_count = self.ptr("spare_count") if store else None
        p.num_splats, p.sh_degree = self.n, self.sh_degree
        p.antialiased = 1 if getattr(self.sc, "antialiased", False) else 0
        p.world, p.sh, p.camera = self.world(), self.shq(), self.camera()
        p.aabb, p.sort_depth, p.radii = self.ptr("aabb"), self.ptr("sort_depth"), self.ptr("radii")
        p.screen = self.screen()
        p.tiles_per_splat = self.ptr("counts") if fused_count else None
        if self.use_packed:
            p.packed_rows = self.ptr("packed")
        if self.use_list:
            self.d["counters"].fill_zero()
            p.visible_ids = self.ptr("vis_ids")
            p.visible_count = self.d["counters"].ptr + 8
        self.check(self.lib.ssr_projection_fwd(C.byref(p), None))
        if store:
            assert int(self.host("spare_count")[0]) == 0, "clear_count was not cleared"

    def tiles(self, fused_count=False):
        sc, D = self.sc, self.L.DeviceArray
        n = self.rows
        if not fused_count or self.tile_active:   # fused counts know nothing of the tile-skip map
            self.check(self.lib.ssr_tile_count(n, self.ptr("aabb"), self.ptr("xy"), self.ptr("conic"),
                                               self.ptr("opac"), sc.width, sc.height, self.tile_active,
                                               self.ptr("counts"), None))
        sb = self.lib.ssr_scan_scratch_bytes(n)
        self.d["scan_scratch"] = D((max(sb, 8),), np.uint8)
        self.check(self.lib.ssr_inclusive_sum_i64(self.ptr("counts"), self.ptr("cum"), n, self.ptr("counters"),
                                                  self.ptr("scan_scratch"), sb, None))
        if self.capacity is not None:
            return self.tiles_capped()
        k = (C.c_int64 * 2)(0, 0)
        if n:
            self.check(self.lib.ssr_read_i64(self.ptr("counters"), k, 2, None))
        self.K = K = int(k[0])
        self.V = int(k[1]) if self.use_list else None
        n_tiles = sc.tile_w * sc.tile_h
        self.d["offsets"] = D((n_tiles,), np.int32)
        for nm in ["keys_a", "keys_b"]:
            self.d[nm] = D((K,), np.int64)
        for nm in ["vals_a", "vals_b"]:
            self.d[nm] = D((K,), np.int32)
        self.sel = 0
        if K:
            self.check(self.lib.ssr_tile_write(n, self.ptr("aabb"), self.ptr("sort_depth"), self.ptr("xy"),
                                               self.ptr("conic"), self.ptr("opac"), self.ptr("cum"), sc.width,
                                               sc.height, self.ptr("keys_a"), self.ptr("vals_a"),
                                               self.ptr("vis_ids") if self.use_list else None,
                                               self.V if self.use_list else 0, self.tile_active, None))
            self.unsorted_keys = self.d["keys_a"].to_host()
            self.unsorted_vals = self.d["vals_a"].to_host()
            sb = (self.lib.ssr_sort_tile_scratch_bytes(K, n_tiles) if self.tile_sort else self.lib.ssr_sort_scratch_bytes(K))
            self.d["sort_scratch"] = D((sb,), np.uint8)
            sel = C.c_int(0)
            if self.tile_sort:
                self.check(self.lib.ssr_sort_tile_pairs(self.ptr("keys_a"), self.ptr("keys_b"), self.ptr("vals_a"),
                                                        self.ptr("vals_b"), K, n_tiles, self.ptr("offsets"),
                                                        C.byref(sel), self.ptr("sort_scratch"), sb, None))
            else:
                self.check(self.lib.ssr_sort_pairs_u64_i32(self.ptr("keys_a"), self.ptr("keys_b"), self.ptr("vals_a"),
                                                           self.ptr("vals_b"), K, 0, self.lib.ssr_sort_end_bit(n_tiles),
                                                           C.byref(sel), self.ptr("sort_scratch"), sb, None))
            self.sel = sel.value
        else:
            self.unsorted_keys = np.zeros(0, np.int64)
            self.unsorted_vals = np.zeros(0, np.int32)
        self.keys = "keys_b" if self.sel else "keys_a"
        self.vals = "vals_b" if self.sel else "vals_a"
        if not (self.tile_sort and K):
            self.check(self.lib.ssr_tile_offsets(K, self.ptr(self.keys), n_tiles, self.ptr("offsets"), None))

    def tiles_capped(self):
        """K4-K6 without knowing the counts on the host; self.K becomes the capacity, self.K_real the count read
        back after everything was launched."""
        sc, D = self.sc, self.L.DeviceArray
        n, cap = self.rows, int(self.capacity)
        n_tiles = sc.tile_w * sc.tile_h
        self.d["offsets"] = D((n_tiles + 1,), np.int32)
        for nm in ["keys_a", "keys_b"]:
            self.d[nm] = D((cap,), np.int64)
        for nm in ["vals_a", "vals_b"]:
            self.d[nm] = D((cap,), np.int32)
        p = self.L.TileWriteCappedParams()
        p.n, p.num_images = n, 1
        p.aabb, p.sort_depth, p.xy, p.conic, p.opac = (self.ptr("aabb"), self.ptr("sort_depth"), self.ptr("xy"),
                                                       self.ptr("conic"), self.ptr("opac"))
        p.cum_tiles, p.width, p.height = self.ptr("cum"), sc.width, sc.height
        p.isect_ids, p.flatten_ids, p.capacity = self.ptr("keys_a"), self.ptr("vals_a"), cap
        if self.use_list:
            p.visible_ids, p.n_visible = self.ptr("vis_ids"), self.ptr("counters") + 8
        p.tile_active = self.tile_active
        self.check(self.lib.ssr_tile_write_capped(C.byref(p), None))
        sb = self.lib.ssr_sort_tile_scratch_bytes(cap, n_tiles)
        self.d["sort_scratch"] = D((sb,), np.uint8)
        sel = C.c_int(0)
        self.check(self.lib.ssr_sort_tile_pairs_capped(self.ptr("keys_a"), self.ptr("keys_b"), self.ptr("vals_a"),
                                                       self.ptr("vals_b"), cap, self.ptr("counters"), n_tiles,
                                                       self.ptr("offsets"),
                                                       C.byref(sel), self.ptr("sort_scratch"), sb, None))
        self.sel = sel.value
        self.keys = "keys_b" if self.sel else "keys_a"
        self.vals = "vals_b" if self.sel else "vals_a"
        self.K = cap
        k = (C.c_int64 * 2)(0, 0)
        self.check(self.lib.ssr_read_i64(self.ptr("counters"), k, 2, None))
        self.K_real = int(k[0])
        self.V = int(k[1]) if self.use_list else None

    def order_tiles(self):
        """ssr_tile_order on the current offsets, checked here: a permutation of the tiles whose fragment counts fall
        class by class (32 fragments a class, everything from 8160 up in the first)."""
        D = self.L.DeviceArray
        n_tiles = self.sc.tile_w * self.sc.tile_h
        sb = self.lib.ssr_tile_order_scratch_bytes(n_tiles)
        self.d["tile_order"], self.d["tile_order_scratch"] = D((n_tiles,), np.int32), D((sb,), np.uint8)
        closed = self.capacity is not None
        self.check(self.lib.ssr_tile_order(self.ptr("offsets"), n_tiles, -1 if closed else self.K, self.ptr("tile_order"),
                                           self.ptr("tile_order_scratch"), sb, None))
        order = self.host("tile_order")
        assert np.array_equal(np.sort(order), np.arange(n_tiles))
        offs = self.host("offsets").ravel().astype(np.int64)
        cls = np.minimum(np.diff(offs if closed else np.concatenate([offs, [self.K]])) >> 5, 255)[order]
        assert np.all(cls[1:] <= cls[:-1])

    def raster_fwd(self):
        sc, D = self.sc, self.L.DeviceArray
        h, w = sc.height, sc.width
        if self.tile_sort and self.K:   # the native stage order also launches the longest tiles first
            self.order_tiles()
        for k, shape, dt in [("r_rgb", (h, w, 3), np.float32), ("r_depth", (h, w), np.float32),
                             ("r_T", (h, w), np.float32), ("r_last", (h, w), np.int32)]:
            self.d[k] = D(shape, dt)
        p = self.L.RasterFwdParams()
        p.num_splats, p.screen, p.width, p.height = self.rows, self.screen(), w, h
        p.tile_offsets, p.flatten_ids, p.n_isects = self.ptr("offsets"), self.ptr(self.vals), self.K
        p.render_rgb, p.render_depth, p.render_T, p.last_ids = (self.ptr("r_rgb"), self.ptr("r_depth"),
                                                                self.ptr("r_T"), self.ptr("r_last"))
        if self.use_packed:
            p.packed_rows = self.ptr("packed")
            p.screen = self.L.Screen()   # not read
        va = self.variant
        p.dist_type = va.get("dist_type", 0)
        if p.dist_type:
            self.d["r_dist_depth"] = D((h, w), np.float32)
            p.distortion_depth = self.ptr("r_dist_depth")
            if p.dist_type == 2:
                self.d["r_dist_rgb"] = D((h, w, 3), np.float32)
                p.distortion_rgb = self.ptr("r_dist_rgb")
        if va.get("median"):
            self.d["r_median"] = D((h, w), np.float32)
            p.render_median = self.ptr("r_median")
        p.tile_order = self.ptr("tile_order")
        p.tile_offsets_closed = 1 if self.capacity is not None else 0
        if self.block_masks and self.K > 0:
            self.d["block_masks"] = D((self.K,), np.uint16)
            p.block_masks = self.ptr("block_masks")
        self.check(self.lib.ssr_raster_fwd(C.byref(p), None))

    def raster_bwd(self, v_rgb=None, v_depth=None, v_T=None):
        sc, D = self.sc, self.L.DeviceArray
        n = self.rows
        self.d["g_rgb"] = D.from_host(np.asarray(sc.v_rgb if v_rgb is None else v_rgb, np.float32))
        self.d["g_depth"] = D.from_host(np.asarray(sc.v_depth if v_depth is None else v_depth, np.float32))
        self.d["g_T"] = D.from_host(np.asarray(sc.v_T if v_T is None else v_T, np.float32))
        for k, shape in [("v_xy", (n, 2)), ("v_depth", (n,)), ("v_conic", (n, 3)), ("v_opac", (n,)), ("v_rgb", (n, 3))]:
            if k not in self.d:
                self.d[k] = D(shape, np.float32)
            self.d[k].fill_zero()
        p = self.L.RasterBwdParams()
        p.num_splats, p.screen, p.width, p.height = n, self.screen(), sc.width, sc.height
        p.tile_offsets, p.flatten_ids, p.n_isects = self.ptr("offsets"), self.ptr(self.vals), self.K
        p.render_T, p.last_ids, p.render_depth = self.ptr("r_T"), self.ptr("r_last"), self.ptr("r_depth")
        p.v_render_rgb, p.v_render_depth, p.v_render_T = self.ptr("g_rgb"), self.ptr("g_depth"), self.ptr("g_T")
        p.v_screen = self.screen("v_")
        if self.use_packed:
            p.packed_rows = self.ptr("packed")
            p.screen = self.L.Screen()
        if self.use_vrows:
            self.d["v_rows"] = D((n, 12), np.float32)
            self.d["v_rows"].fill_zero()
            p.v_rows = self.ptr("v_rows")
            if n:   # the five arrays must stay untouched
                for k in ["v_xy", "v_depth", "v_conic", "v_opac", "v_rgb"]:
                    self.check(self.lib.ssr_fill_u32(self.d[k].ptr, 0x7fc12345, self.d[k].nbytes // 4, None))
        va = self.variant
        f32 = lambda a: D.from_host(np.ascontiguousarray(a, np.float32))
        p.dist_type = va.get("dist_type", 0)
        if p.dist_type:
            self.d["g_dist_depth"] = f32(va["v_dist_depth"])
            p.distortion_depth, p.v_distortion_depth = self.ptr("r_dist_depth"), self.ptr("g_dist_depth")
            if p.dist_type == 2:
                self.d["g_dist_rgb"] = f32(va["v_dist_rgb"])
                p.render_rgb, p.distortion_rgb, p.v_distortion_rgb = self.ptr("r_rgb"), self.ptr("r_dist_rgb"), self.ptr("g_dist_rgb")
        if va.get("median"):
            self.d["g_median"] = f32(va["v_median"])
            p.v_render_median = self.ptr("g_median")
        p.accum_mode = va.get("accum_mode", 0)
        if p.accum_mode:
            self.d["accum_map"] = f32(va["accum_map"])
            self.d["accum_weight"] = D((self.n * (2 if p.accum_mode == 3 else 1),), np.float32)
            self.d["accum_weight"].fill_zero()
            p.accum_weight_map, p.accum_weight, p.num_world = self.ptr("accum_map"), self.ptr("accum_weight"), self.n
            if self.packed_projection:
                p.gaussian_ids = self.ptr("gaussian_ids")
        p.tile_order = self.ptr("tile_order")
        p.tile_offsets_closed = 1 if self.capacity is not None else 0
        p.schedule = 1 if self.bwd_lanes else 0
        if self.block_masks and "block_masks" in self.d:
            p.block_masks = self.ptr("block_masks")
        self.check(self.lib.ssr_raster_bwd(C.byref(p), None))
        if self.use_vrows and n:   # unpack for the comparisons, after checking the arrays were left alone
            for k in ["v_xy", "v_depth", "v_conic", "v_opac", "v_rgb"]:
                assert np.all(self.host(k).view(np.uint32) == 0x7fc12345), k
            rows = self.host("v_rows")
            if p.accum_mode in (2, 3):   # the weight sums travel in the two spare floats of a row
                aw = self.host("accum_weight")
                if not self.packed_projection:   # row = world row: the sums, as they were moved on
                    assert np.allclose(rows[:, 10], aw[:self.n], rtol=1e-6, atol=0)
                    if p.accum_mode == 3:
                        assert np.allclose(rows[:, 11], aw[self.n:], rtol=1e-6, atol=0)
            else:
                assert not np.any(rows[:, 10:])
            for k, sl in [("v_xy", slice(0, 2)), ("v_depth", 2), ("v_conic", slice(3, 6)), ("v_opac", 6), ("v_rgb", slice(7, 10))]:
                self.d[k] = D.from_host(np.ascontiguousarray(rows[:, sl]))

    def projection_bwd(self, accumulate=True, poison=False, pose=False, misalign_sh_rows=False, use_world_rows=True):
        """use_world_rows=False: gather the parameters although the projection left their rows. pose=True: also the camera-pose gradient, read back with host("v_viewmat") as [4,4].
        misalign_sh_rows: the SH gradient rows start 4 bytes into their buffer, which takes the launcher off the
        kernel that stages them through LDS (it needs 16-byte alignment); read back with sh_rows_misaligned()."""
        D = self.L.DeviceArray
        n = self.n
        for k, shape in [("w_means", (n, 3)), ("w_quats", (n, 4)), ("w_log_scales", (n, 3)),
                         ("w_opacity_logits", (n,)), ("w_features_dc", (n, 3)), ("w_features_sh", (n, 15, 3))]:
            if k not in self.d:
                self.d[k] = D(shape, np.float32)
            if poison:
                self.check(self.lib.ssr_fill_u32(self.d[k].ptr, 0x7fc00000, self.d[k].nbytes // 4, None))
            else:
                self.d[k].fill_zero()
        p = self.L.ProjectionBwdParams()
        p.num_splats, p.sh_degree = n, self.sh_degree
        p.antialiased = 1 if getattr(self.sc, "antialiased", False) else 0
        p.world, p.sh, p.camera = self.world(), self.shq(), self.camera()
        p.aabb, p.v_screen, p.v_world = self.ptr("aabb"), self.screen("v_"), self.world("w_")
        p.accumulate = 1 if accumulate else 0
        if self.use_list:
            p.visible_ids, p.n_visible = self.ptr("vis_ids"), self.V
        if self.use_vrows:
            p.v_rows = self.ptr("v_rows")
            p.v_screen = self.L.Screen()   # not read
        if pose:
            self.d["v_viewmat"] = D((4, 4), np.float32)
            self.d["v_viewmat"].fill_zero()
            p.v_viewmat = self.ptr("v_viewmat")
        if self.packed_projection:
            if self.rows == 0:   # nothing visible: the launcher has nothing to run (ProjectionBwd.cu:86-97)
                return
            p.aabb = None
            p.packed_gaussian_ids, p.num_packed = self.ptr("gaussian_ids"), self.rows
            if self.world_rows and use_world_rows:
                p.packed_world_rows = self.ptr("world_rows")
                p.packed_world_stride = self.cap
        if misalign_sh_rows:
            raw = D((n * 45 + 4,), np.float32)
            if poison:
                self.check(self.lib.ssr_fill_u32(raw.ptr, 0x7fc00000, n * 45 + 4, None))
            else:
                raw.fill_zero()
            self.d["w_features_sh_raw"] = raw
            p.v_world.features_sh = raw.ptr + 4
        self.check(self.lib.ssr_projection_bwd(C.byref(p), None))

    def sh_rows_misaligned(self):
        return self.d["w_features_sh_raw"].to_host()[1:1 + self.n * 45].reshape(self.n, 15, 3)

    def fused_optimizer(self, g1, g2, hyper, step=1, steps=None, v_in=None, scale_agnostic=False, quant_state=None, non_sh=None):
        """ssr_fused_projection_bwd_optimizer on the device copies of the parameters (fp32 SH);
        g1 / g2 are host dicts keyed like the world arrays. Returns (params, g1, g2, score) from the device."""
        D = self.L.DeviceArray
        keys = ["means", "quats", "log_scales", "opacity_logits", "features_dc", "features_sh"]
        for pre, src in (("m1_", g1), ("m2_", g2)):
            for k in keys:
                if (quant_state is not None and k == "features_sh") or (non_sh is not None and k != "features_sh"):
                    self.d[pre + k] = None
                    continue
                self.d[pre + k] = D.from_host(np.ascontiguousarray(src[k], np.float32))
        for k in keys:
            a = None if v_in is None else v_in.get(k)
            self.d["vi_" + k] = None if a is None else D.from_host(np.ascontiguousarray(a, np.float32))
        self.d["score"] = D((self.n,), np.float32)
        p = self.L.FpboParams()
        p.num_splats, p.sh_degree = self.n, self.sh_degree
        p.antialiased = 1 if getattr(self.sc, "antialiased", False) else 0
        p.world, p.camera, p.aabb = self.world(), self.camera(), self.ptr("aabb")
        p.v_screen, p.v_world_in, p.g1, p.g2 = self.screen("v_"), self.world("vi_"), self.world("m1_"), self.world("m2_")
        p.densify_score = self.ptr("score")
        for k, v in hyper.items():
            setattr(p, k, v)
        p.step = step
        if steps is not None:
            self.d["steps"] = D.from_host(np.ascontiguousarray(steps, np.int32))
            p.steps = self.ptr("steps")
        if self.packed_projection:   # aabb and v_screen hold the nnz packed rows
            self.d["row_of"] = D((self.n,), np.int32)
            self.check(self.lib.ssr_packed_row_map(self.ptr("gaussian_ids") if self.rows else None, self.rows, self.n,
                                                   self.ptr("row_of"), None))
            p.packed_row_of = self.ptr("row_of")
        if self.use_vrows:
            p.v_rows = self.ptr("v_rows")
        if scale_agnostic:
            p.scale_agnostic_radii = self.ptr("radii")
        if quant_state is not None:
            # the reference's quantization level 1: SH values are the scene's 16-bit codes (one (min, max) per 256
            # splats, which the forward already read), their moments the 8-bit (u, log_s) cells given here
            assert self.sc.sh_codec == 2 and self.sc.sh_bounds_stride == 256 * 45
            self.d["sh_state_packed"] = D.from_host(np.ascontiguousarray(quant_state["state_packed"], np.uint16))
            self.d["sh_state_bounds"] = D.from_host(np.ascontiguousarray(quant_state["state_bounds"], np.float32))
            p.sh_state_packed, p.sh_state_bounds = self.ptr("sh_state_packed"), self.ptr("sh_state_bounds")
            p.sh_value_packed, p.sh_value_bounds = self.ptr("sh_packed"), self.ptr("sh_bounds")
            p.num_sh_buffer = 15
            w = p.world
            w.features_sh = None
            p.world = w
        if non_sh is not None:   # quantized non-SH moments: five arrays of 32-bit cells, five of float4 bounds
            for t in range(5):
                self.d[f"ns_packed{t}"] = D.from_host(np.ascontiguousarray(non_sh["packed"][t], np.uint32))
                self.d[f"ns_bounds{t}"] = D.from_host(np.ascontiguousarray(non_sh["bounds"][t], np.float32))
                p.non_sh_packed[t], p.non_sh_bounds[t] = self.ptr(f"ns_packed{t}"), self.ptr(f"ns_bounds{t}")
        self.check(self.lib.ssr_fused_projection_bwd_optimizer(C.byref(p), None))
        self.check(self.lib.ssr_device_synchronize())
        if quant_state is not None:
            keys = keys[:5]
        out = lambda pre: {k: (self.host(pre + k) if self.d.get(pre + k) is not None else None) for k in keys}
        res = out(""), out("m1_"), out("m2_"), self.host("score")
        if non_sh is not None:
            self.non_sh_out = dict(packed=[self.host(f"ns_packed{t}") for t in range(5)], bounds=[self.host(f"ns_bounds{t}") for t in range(5)])
        if quant_state is not None:
            q = dict(state_packed=self.host("sh_state_packed"), state_bounds=self.host("sh_state_bounds"),
                     value_packed=self.host("sh_packed").view(np.uint16), value_bounds=self.host("sh_bounds"), num_sh_buffer=15)
            return res + (q,)
        return res

    def run_all(self, backward=True, fused_count=False):
        self.projection_fwd(fused_count)
        self.tiles(fused_count)
        self.raster_fwd()
        if backward:
            self.raster_bwd()
            self.projection_bwd()
        self.check(self.lib.ssr_device_synchronize())
        return self

    def host(self, k):
        return self.d[k].to_host()

    def proj_host(self):
        return {k: self.host(k) for k in ["aabb", "sort_depth", "radii", "xy", "depth", "conic", "opac", "rgb"]}
