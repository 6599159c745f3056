"""CPU-only: the C-ABI library loads and exports every symbol include/ssr_backend.h declares, the
argument checks that need no device work, the scene generators and the SH codecs."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def L(pkg):
    from spirula_studio_amd import lib
    lib.load()
    return lib


def test_every_declared_symbol_is_exported(L):
    hdr = open(os.path.join(ROOT, "include", "ssr_backend.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    declared = set(re.findall(r"\b(ssr_[a-z0-9_]+)\s*\(", hdr))
    assert len(declared) >= 35
    assert declared == set(L.SYMBOLS), (declared ^ set(L.SYMBOLS))
    raw = C.CDLL(L.SO_PATH)
    for name in declared:
        assert hasattr(raw, name), name


def test_host_library_exports(pkg):
    from spirula_studio_amd import host
    h = host.load()
    for name in host.SYMBOLS:
        assert hasattr(h, name), name
    # the reference-named C++ launch functions are defined in it as well
    out = os.popen(f"nm -DC {host.SO_PATH}").read()
    for sym in ["projection_3dgs_forward(", "do_intersect_tile_generic(", "rasterize_to_pixels_3dgs_fwd(",
                "rasterize_to_pixels_3dgs_bwd(", "projection_3dgs_backward(", "backend::device_malloc(",
                "backend::memcpy_sync(", "backend::last_error()", "forward_3dgs(", "set_data_3dgs(",
                "engine_backward_from_render_grad("]:
        assert sym in out, sym


def test_argument_checks_without_device(L):
    lib = L.load()
    assert lib.ssr_sort_end_bit(2500) == 44 and lib.ssr_sort_end_bit(8160) == 45
    assert lib.ssr_sort_end_bit(32400) == 47 and lib.ssr_sort_end_bit(32768) == 48
    assert lib.ssr_scan_scratch_bytes(0) == 0 and lib.ssr_scan_scratch_bytes(2049) == 16
    assert lib.ssr_sort_scratch_bytes(0) == 0 and lib.ssr_sort_scratch_bytes(4097) == (3 * 256 + 256) * 4   # three 2048-key blocks
    # the staging area of the packed projection: the parameter rows add 48 bytes per splat behind the rest
    for n in (1, 1000, 1025, 10_000_000):
        assert lib.ssr_projection_packed_scratch_bytes_world_rows(n) == lib.ssr_projection_packed_scratch_bytes(n) + 48 * n
    assert lib.ssr_projection_packed_scratch_bytes_world_rows(0) == lib.ssr_projection_packed_scratch_bytes(0)
    assert lib.ssr_projection_fwd(None, None) != 0 and b"null params" in lib.ssr_last_error()
    assert lib.ssr_last_error() == b""                     # cleared by the read
    p = L.ProjectionFwdParams()
    p.num_splats, p.sh_degree = 10, 7
    assert lib.ssr_projection_fwd(C.byref(p), None) != 0 and b"SH degree" in lib.ssr_last_error()
    p.sh_degree = 3
    p.camera.camera_model, p.camera.num_cameras, p.camera.width, p.camera.height = 7, 1, 8, 8
    assert lib.ssr_projection_fwd(C.byref(p), None) != 0 and b"camera model" in lib.ssr_last_error()
    # pairs the reference does not instantiate (src/kernels/projection/CameraVariants.cuh:11-22)
    for model, tier in [(1, 3), (2, 3), (3, 1), (0, 4)]:
        p.camera.camera_model, p.camera.distortion = model, tier
        assert lib.ssr_projection_fwd(C.byref(p), None) != 0 and b"camera model" in lib.ssr_last_error()
    p.camera.camera_model, p.camera.distortion = 1, 2
    p.camera.viewmats = p.camera.intrins = 16     # non-null, never read: the coefficient check comes first
    assert lib.ssr_projection_fwd(C.byref(p), None) != 0 and b"lens coefficients" in lib.ssr_last_error()
    p.camera.viewmats = p.camera.intrins = None
    p.camera.distortion = 0
    p.camera.camera_model, p.camera.num_cameras = 0, 2
    p.camera.viewmats = p.camera.intrins = 16
    assert lib.ssr_projection_fwd(C.byref(p), None) != 0 and b"one camera" in lib.ssr_last_error()
    r = L.RasterFwdParams()
    assert lib.ssr_raster_fwd(C.byref(r), None) != 0 and b"empty image" in lib.ssr_last_error()
    assert lib.ssr_device_malloc(0) is None
    assert lib.ssr_memcpy(None, None, 0, 0, None, 0) == 0
    assert lib.ssr_fill_u32(None, 0, 0, None) == 0
    assert lib.ssr_tile_offsets(-1, None, 4, None, None) != 0 and lib.ssr_last_error() != b""
    # gradient rows are addressed as 12 * row in 32 bits: more rows than that are refused, not wrapped
    b = L.RasterBwdParams()
    b.width = b.height = 16
    b.n_isects = 1
    for f in ("tile_offsets", "flatten_ids", "render_T", "last_ids", "render_depth", "v_render_rgb", "v_render_depth",
              "v_render_T", "packed_rows", "v_rows"):
        setattr(b, f, 16)          # non-null, aligned, never read: the check comes before any launch
    b.num_splats = 0xFFFFFFFF // 12 + 1
    assert lib.ssr_raster_bwd(C.byref(b), None) != 0 and b"357913941" in lib.ssr_last_error()
    b.num_splats = 1 << 30
    assert lib.ssr_raster_bwd(C.byref(b), None) != 0 and b"2^30" in lib.ssr_last_error()
    # the allocation-free scan refuses what its fixed scratch cannot hold
    assert lib.ssr_inclusive_sum_i64_static(16, 16, (1 << 27) + 1, None, None) != 0 and b"static" in lib.ssr_last_error()
    assert lib.ssr_zero_world_rows(None, None, 0, None, None, 0, None) != 0 and b"null world" in lib.ssr_last_error()
    assert lib.ssr_tile_order_scratch_bytes(8160) == 8 * 256 * 4
    assert lib.ssr_tile_order(16, 100, 5, 16, None, 0, None) != 0 and b"scratch" in lib.ssr_last_error()
    assert lib.ssr_tile_order(None, 0, 0, None, None, 0, None) == 0
    # the entry points that leave the counts on the device
    from spirula_studio_amd import lib as L
    w = L.TileWriteCappedParams()
    assert lib.ssr_tile_write_capped(None, None) != 0 and b"null params" in lib.ssr_last_error()
    w.n, w.capacity, w.num_images = 10, 1 << 31, 1
    assert lib.ssr_tile_write_capped(C.byref(w), None) != 0 and b"capacity" in lib.ssr_last_error()
    w.capacity = 0
    assert lib.ssr_tile_write_capped(C.byref(w), None) == 0      # nothing can be written: no launch
    w.capacity, w.num_images = 100, 0
    assert lib.ssr_tile_write_capped(C.byref(w), None) != 0 and b"num_images" in lib.ssr_last_error()
    w.num_images, w.aabb, w.sort_depth, w.xy, w.conic, w.opac, w.cum_tiles = 1, 16, 16, 16, 16, 16, 16
    w.isect_ids, w.flatten_ids, w.width, w.height, w.visible_ids = 16, 16, 64, 64, 16
    assert lib.ssr_tile_write_capped(C.byref(w), None) != 0 and b"device count" in lib.ssr_last_error()
    sel = C.c_int(0)
    assert lib.ssr_sort_tile_pairs_capped(16, 16, 16, 16, 0, 16, 10, 16, C.byref(sel), 16, 1 << 20, None) != 0
    assert b"capacity" in lib.ssr_last_error()
    assert lib.ssr_sort_tile_pairs_capped(16, 16, 16, 16, 100, None, 10, 16, C.byref(sel), 16, 1 << 20, None) != 0
    assert b"null count" in lib.ssr_last_error()
    assert lib.ssr_tile_offsets_capped(100, None, 16, 10, 16, None) != 0 and b"null pointer" in lib.ssr_last_error()
    assert lib.ssr_tile_offsets_capped(0, 16, 16, 10, 16, None) != 0 and b"capacity" in lib.ssr_last_error()


def test_missing_library_fails_loudly(pkg, monkeypatch):
    from spirula_studio_amd import lib
    monkeypatch.setattr(lib, "_lib", None)
    monkeypatch.setattr(lib, "SO_PATH", "/nonexistent/libssr_hip.so")
    with pytest.raises(lib.SsrError, match="no CPU fallback"):
        lib.load()


def test_scene_streams_are_counter_based(pkg):
    S = pkg.scenes
    a = S.uniform(11, 3, 1000, -1.0, 1.0)
    b = S.uniform(11, 3, 400, -1.0, 1.0, start=600)
    assert np.array_equal(a[600:], b)
    native = S._NATIVE
    try:
        S._NATIVE = False                       # numpy definition
        assert np.array_equal(a, S.uniform(11, 3, 1000, -1.0, 1.0))
        n1 = S.normal(5, 2, 5001, 0.5, 2.0)
    finally:
        S._NATIVE = native
    n2 = S.normal(5, 2, 5001, 0.5, 2.0)
    assert np.abs(n1 - n2).max() <= 1e-6
    assert abs(float(n2.mean()) - 0.5) < 0.1 and abs(float(n2.std()) - 2.0) < 0.1
    sc1, sc2 = S.make_scene(1, n=2000, width=64, height=64), S.make_scene(1, n=2000, width=64, height=64)
    assert np.array_equal(sc1.means, sc2.means) and np.array_equal(sc1.v_rgb, sc2.v_rgb)
    assert np.allclose(np.linalg.norm(sc1.quats, axis=1), 1.0, atol=1e-6)
    sc5 = S.make_scene(5, n=3000, width=128, height=64)
    r = np.linalg.norm(sc5.means, axis=1)
    assert r.min() >= 4.99 and r.max() <= 30.01 and sc5.camera_model == S.CAM_EQUIRECT
    assert abs(float(sc5.intrins[0]) - 128 / (2 * np.pi)) < 1e-4


def test_codecs_match_the_oracle_encoders(pkg, oracle):
    S = pkg.scenes
    rng = np.random.default_rng(0)
    v = rng.normal(0, 0.05, (513, 15, 3)).astype(np.float32)
    for bits, stride in [(8, 256), (16, 256), (8, 256 * 45)]:
        codes, bounds, dec = S.quantize_ref(v, bits, stride)
        n = v.size
        packed = np.zeros(n * (2 if bits == 16 else 1), np.uint8)
        ob = np.zeros(((n + stride - 1) // stride, 2), np.float32)
        oracle.lib().or_quantize_ref(C.c_int(bits), C.c_int64(n), C.c_int64(stride), v.ctypes.data_as(C.c_void_p),
                                     packed.ctypes.data_as(C.c_void_p), ob.ctypes.data_as(C.c_void_p))
        ocodes = packed.view(np.uint16) if bits == 16 else packed
        assert np.array_equal(bounds, ob)
        assert (codes.astype(np.int64) != ocodes.astype(np.int64)).mean() < 1e-3   # ties of the rounding only
        qmax = 65535 if bits == 16 else 255
        assert np.abs(dec - v).max() <= (bounds[:, 1] - bounds[:, 0]).max() / qmax * 0.51 + 1e-7
    codes, scale, dec = S.quantize_i8_f16(v)
    oc = np.zeros(v.size, np.int8)
    osc = np.zeros(v.shape[0], np.uint16)
    oracle.lib().or_quantize_i8_f16(C.c_int64(v.shape[0]), C.c_int(45), v.ctypes.data_as(C.c_void_p),
                                    oc.ctypes.data_as(C.c_void_p), osc.ctypes.data_as(C.c_void_p))
    assert np.array_equal(scale.view(np.uint16), osc)
    assert np.array_equal(codes, oc)
    assert np.abs(dec - v).max() <= float(scale.astype(np.float32).max()) * 0.51


def test_ctypes_structures_match_the_header(pkg, tmp_path):
    """Every parameter structure of include/ssr_backend.h has the same size and the same offset of its last
    member in the Python mirror as the C compiler gives it."""
    import ctypes as C
    import subprocess
    from spirula_studio_amd import lib
    pairs = [("ssr_world", lib.World), ("ssr_screen", lib.Screen), ("ssr_sh_quant", lib.ShQuant), ("ssr_camera", lib.Camera),
             ("ssr_projection_fwd_params", lib.ProjectionFwdParams), ("ssr_projection_packed_params", lib.ProjectionPackedParams),
             ("ssr_raster_fwd_params", lib.RasterFwdParams), ("ssr_raster_bwd_params", lib.RasterBwdParams),
             ("ssr_projection_bwd_params", lib.ProjectionBwdParams), ("ssr_fpbo_params", lib.FpboParams)]
    src = tmp_path / "sizes.c"
    body = "".join(f'    printf("%zu %zu\\n", sizeof({c}), offsetof({c}, {py._fields_[-1][0]}));\n' for c, py in pairs)
    src.write_text('#include <stdio.h>\n#include <stddef.h>\n#include "ssr_backend.h"\nint main(void) {\n' + body + "    return 0;\n}\n")
    exe = tmp_path / "sizes"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split("\n")
    for (c, py), line in zip(pairs, out):
        size, off = [int(v) for v in line.split()]
        assert C.sizeof(py) == size, (c, C.sizeof(py), size)
        assert getattr(py, py._fields_[-1][0]).offset == off, (c, py._fields_[-1][0])
