"""The 3dgs rows of the reference's backend parity tools on their own inputs (src/backend/tests/render_parity.cpp,
raster_bwd_parity.cpp, accum_weight_map.cpp), one camera of the tools' two-camera batch per run: the GPU path
through the C ABI against the oracle, and accum_weight_map's own expectations on the GPU path."""
import numpy as np
import pytest

import reference_tools as R
from gpu_pipeline import GpuRun, world_grad_check
from test_gpu_parity import _compare, _compare_packed, gpu  # noqa: F401  (gpu: module fixture)

pytestmark = pytest.mark.gpu

PINHOLE, FISHEYE, EQUISOLID, EQUIRECT = 0, 1, 2, 3
NONE, OPENCV, THIN_PRISM, RATIONAL = 0, 1, 2, 3


# render_parity.cpp:186-196, rows with prim == 0 (3dgs) and 1 (mip): (mip, packed, camera model, tier, dist_type, median)
@pytest.mark.parametrize("mip,packed,model,tier,dist_type,median", [(False, False, PINHOLE, OPENCV, 2, True), (True, False, PINHOLE, NONE, 2, True),
                                                                  (False, False, FISHEYE, THIN_PRISM, 1, False),
                                                                  (False, True, EQUIRECT, NONE, 0, False)])
@pytest.mark.parametrize("cam", [0, 1])
def test_render_parity_rows(gpu, oracle, mip, packed, model, tier, dist_type, median, cam):
    sc, _ = R.tool_scene(gpu, R.SEED_RENDER, cam, model, tier, mip=mip)
    z3, z1 = np.zeros((sc.height, sc.width, 3), np.float32), np.zeros((sc.height, sc.width), np.float32)
    va = dict(dist_type=dist_type, median=median, v_dist_rgb=z3, v_dist_depth=z1, v_median=z1)
    label = f"render_parity model {model} tier {tier} cam {cam}"
    if packed:
        _compare_packed(gpu, oracle, sc, label, fused_count=True, variant=va)
    else:
        _compare(gpu, oracle, sc, label, fused_count=True, use_list=True, use_packed=True, variant=va)


# raster_bwd_parity.cpp:176-181, rows with prim == 0: (packed, camera model, tier, dist_type, median, accumulation mode)
@pytest.mark.parametrize("packed,model,tier,dist_type,median,accum", [(False, PINHOLE, NONE, 0, False, 0), (False, PINHOLE, OPENCV, 2, True, 1),
                                                                    (True, FISHEYE, THIN_PRISM, 1, False, 2),
                                                                    (True, FISHEYE, THIN_PRISM, 1, False, 3)])
@pytest.mark.parametrize("cam", [0, 1])
def test_raster_bwd_parity_rows(gpu, oracle, packed, model, tier, dist_type, median, accum, cam):
    _, rng = R.tool_world(R.SEED_RASTER_BWD)
    ct = R.raster_bwd_cotangents(rng)
    sc, _ = R.tool_scene(gpu, R.SEED_RASTER_BWD, cam, model, tier, cotangents=ct)
    va = dict(dist_type=dist_type, median=median, accum_mode=accum, v_dist_rgb=ct["v_dist_rgb"][cam], v_dist_depth=ct["v_dist_depth"][cam],
              v_median=ct["v_median"][cam], accum_map=ct["accum_map"][cam])
    label = f"raster_bwd_parity model {model} tier {tier} dist {dist_type} accum {accum} cam {cam}"
    if packed:
        _compare_packed(gpu, oracle, sc, label, fused_count=True, use_packed=True, variant=va)
    else:
        _compare(gpu, oracle, sc, label, fused_count=True, use_list=True, use_packed=True, use_vrows=True, variant=va)


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("mode", [1, 2, 3])
def test_accum_weight_map_reaches_the_right_splats(gpu, oracle, packed, mode):
    """accum_weight_map.cpp run_mode(): known loss maps planted on the real forward chain, the per-splat score read back."""
    centres = {}
    runs = {}
    for cam in (0, 1):
        sc, _ = R.tool_scene(gpu, R.SEED_RASTER_BWD, cam)
        g = GpuRun(gpu, sc, use_packed=True, packed_projection=packed)
        g.projection_fwd(fused_count=True)
        g.tiles(fused_count=True)
        g.raster_fwd()
        xy = np.full((sc.n, 2), -1e9, np.float32)
        if packed:   # packed rows go back through gaussian_ids, the mapping under test
            xy[g.host("gaussian_ids")[:g.nnz]] = g.host("xy")[:g.nnz]
        else:
            aabb = g.host("aabb")
            vis = aabb[:, 2] > aabb[:, 0]
            xy[vis] = g.host("xy")[vis]
        centres[cam], runs[cam] = xy, g
    for cam in (0, 1):
        g, sc = runs[cam], runs[cam].sc

        def run(amap):
            g.variant = dict(accum_mode=mode, accum_map=amap)
            g.raster_bwd()
            return R.accum_finalize(g.host("accum_weight"), sc.n, mode)
        R.accum_weight_map_checks(run, centres[cam], centres[1 - cam], mode, f"gpu {'packed' if packed else 'plain'} mode {mode} cam {cam}")


# fpbo_parity.cpp:160-162, the two fp32-state 3dgs rows: PINHOLE without a lens and with the OpenCV tier, all five
# non-SH world gradients present, densify score on, two consecutive steps (10, then 11)
@pytest.mark.parametrize("row,tier", [(0, NONE), (1, OPENCV)])
@pytest.mark.parametrize("cam", [0, 1])
def test_fpbo_parity_rows(gpu, oracle, row, tier, cam):
    sc, rng = R.tool_scene(gpu, R.SEED_FPBO, cam, PINHOLE, tier, n=R.N_FPBO)
    for _ in range(row + 1):   # row 1 draws after row 0
        vs2, v_world, g1, g2 = R.fpbo_row_inputs(rng)
    vs = {k: np.ascontiguousarray(v[cam]) for k, v in vs2.items()}
    g = GpuRun(gpu, sc)
    g.projection_fwd()
    D = gpu.lib.DeviceArray
    for k, v in vs.items():
        g.d[k] = D.from_host(v)
    aabb = g.host("aabb")
    assert 100 < (aabb[:, 2] > aabb[:, 0]).sum() < sc.n
    P = {k: np.ascontiguousarray(getattr(sc, k), np.float32).copy() for k in oracle.WORLD_KEYS}
    o1 = {k: v.copy() for k, v in g1.items()}
    o2 = {k: v.copy() for k, v in g2.items()}
    h = R.FPBO_HYPER
    lrs = dict(means="lr_means", quats="lr_quats", log_scales="lr_scales", opacity_logits="lr_opacs",
               features_dc="lr_features_dc", features_sh="lr_features_sh")
    d1, d2 = g1, g2
    for step in (10, 11):
        dP, d1, d2, dscore = g.fused_optimizer(d1, d2, h, step=step, v_in=v_world)
        score = oracle.fused_projection_bwd_optimizer(sc, aabb, vs, P, o1, o2, h, step=step, v_in=v_world)
        for k in oracle.WORLD_KEYS:
            a, b = d1[k].reshape(sc.n, -1).astype(np.float64), o1[k].reshape(sc.n, -1).astype(np.float64)
            assert (np.abs(a - b) <= 1e-3 * np.abs(b) + 1e-4 * (np.abs(b).max(axis=1, keepdims=True) + 1e-12)).all(), ("g1", k, step)
            a, b = d2[k].reshape(sc.n, -1).astype(np.float64), o2[k].reshape(sc.n, -1).astype(np.float64)
            assert (np.abs(a - b) <= 2e-3 * np.abs(b) + 1e-12).all(), ("g2", k, step)
            a, b = dP[k].astype(np.float64), P[k].astype(np.float64)
            assert np.abs(a - b).max() <= 0.02 * h[lrs[k]] * 40 + 1e-6, (k, step, float(np.abs(a - b).max()))
        assert np.allclose(dscore, score, rtol=1e-3, atol=1e-9)
    assert np.abs(P["means"] - sc.means).max() > 1e-5   # two steps did move the splats


# projection_parity.cpp:120-160 with prim == 0: every camera model at SH degree 0 without a lens and at degree 3 with
# each of its compiled tiers
@pytest.mark.parametrize("model", [PINHOLE, FISHEYE, EQUISOLID, EQUIRECT])
@pytest.mark.parametrize("cam", [0, 1])
@pytest.mark.parametrize("mip", [False, True])      # prim 0 and prim 1 of the tool's sweep
def test_projection_parity_rows(gpu, oracle, model, cam, mip):
    for deg, tiers in [(0, [NONE]), (3, R.COMPILED_TIERS[model])]:
        for tier in tiers:
            sc, _ = R.tool_scene(gpu, R.SEED_PROJ, cam, model, tier, mip=mip)
            want = oracle.projection_fwd(sc, deg)
            g = GpuRun(gpu, sc, sh_degree=deg)
            g.projection_fwd()
            got = g.proj_host()
            vis = want["aabb"][:, 2] > want["aabb"][:, 0]
            print(f"[projection_parity model {model} tier {tier} degree {deg} cam {cam}] visible={int(vis.sum())}", flush=True)
            assert 50 < vis.sum() < sc.n
            for k in ["aabb", "sort_depth", "radii"]:
                assert np.array_equal(got[k].view(np.uint32), want[k].view(np.uint32)), (k, tier, deg)
            for k in ["xy", "depth", "conic", "opac", "rgb"]:
                assert np.array_equal(got[k][vis].view(np.uint32), want[k][vis].view(np.uint32)), (k, tier, deg)


# projection_parity.cpp:201-215 with prim == 0 (PINHOLE): 8- and 16-bit SH value codes, bounds per 256 cells and per
# 256 splats, the tier rotating through the four configurations
@pytest.mark.parametrize("cam", [0, 1])
def test_projection_parity_quantized_rows(gpu, oracle, cam):
    _, rng = R.tool_world(R.SEED_PROJ)
    q = R.projection_quant_inputs(rng)
    qcfg = 0
    for bits in (8, 16):
        for per_block in (0, 1):
            tier = R.COMPILED_TIERS[PINHOLE][qcfg % 4]
            qcfg += 1
            sc, _ = R.tool_scene(gpu, R.SEED_PROJ, cam, PINHOLE, tier)
            sc.sh_codec = 1 if bits == 8 else 2
            sc.sh_packed = q["q8"] if bits == 8 else q["q16"]
            sc.sh_bounds = q["bounds_block"] if per_block else q["bounds_cell"]
            sc.sh_bounds_stride = 0 if per_block else 256      # 0: the fused optimizer's layout, as the tool passes it
            want = oracle.projection_fwd(sc, 3)
            g = GpuRun(gpu, sc)
            g.projection_fwd()
            got = g.proj_host()
            vis = want["aabb"][:, 2] > want["aabb"][:, 0]
            for k in ["aabb", "sort_depth", "radii"]:
                assert np.array_equal(got[k].view(np.uint32), want[k].view(np.uint32)), (k, bits, per_block)
            for k in ["xy", "depth", "conic", "opac", "rgb"]:
                assert np.array_equal(got[k][vis].view(np.uint32), want[k][vis].view(np.uint32)), (k, bits, per_block)
            # the colours do come from the codes: decode by the codec's definition and compare with an fp32 run
            stride = 256 * 45 if per_block else 256
            b = sc.sh_bounds[np.arange(sc.n * 45) // stride]
            qmax = np.float32(255.0 if bits == 8 else 65535.0)
            dec = (b[:, 0] + (b[:, 1] - b[:, 0]) * (sc.sh_packed.astype(np.float32) * (np.float32(1.0) / qmax))).astype(np.float32)
            sc32, _ = R.tool_scene(gpu, R.SEED_PROJ, cam, PINHOLE, tier)
            sc32.features_sh = dec.reshape(sc.n, 15, 3)
            w32 = oracle.projection_fwd(sc32, 3)
            assert np.array_equal(w32["rgb"][vis].view(np.uint32), want["rgb"][vis].view(np.uint32)), (bits, per_block)


def _k9_direct(gpu, oracle, sc, vs, label, packed=False, pose=False, sh_degree=3):
    """ssr_projection_bwd fed given screen gradients (rows: splats, or packed rows), against the oracle.
    pose: also the camera-pose gradient (the rows of the tool that ask for v_viewmats)."""
    g = GpuRun(gpu, sc, packed_projection=packed, sh_degree=sh_degree)
    g.projection_fwd()
    D = gpu.lib.DeviceArray
    aabb = g.host("aabb")
    if packed:
        ids = g.host("gaussian_ids")[:g.rows]
        full_aabb = np.zeros((sc.n, 4), np.float32)
        full_aabb[ids] = aabb[:g.rows]
        full_vs = {}
        for k, v in vs.items():
            assert v.shape[0] == g.rows
            full_vs[k] = np.zeros((sc.n,) + v.shape[1:], np.float32)
            full_vs[k][ids] = v
    else:
        full_aabb, full_vs = aabb, vs
    for k, v in vs.items():
        g.d[k] = D.from_host(np.ascontiguousarray(v))
    g.projection_bwd(pose=pose)
    want = oracle.projection_bwd(sc, full_aabb, full_vs, sh_degree=sh_degree, pose=pose)
    if pose:
        got_vm, want_vm = g.host("v_viewmat").astype(np.float64), want.pop("v_viewmat").astype(np.float64)
        print(f"[{label}] dL/dt = {want_vm[:3, 3]}", flush=True)
        assert not np.any(got_vm[3]) and np.abs(want_vm[:3]).min() > 0
        assert np.abs(got_vm - want_vm).max() <= 1e-3 * np.abs(want_vm).max(), (got_vm, want_vm)
        assert (np.abs(got_vm - want_vm) <= 5e-3 + 1e-3 * np.abs(want_vm)).all()     # the tool's band
    vis = full_aabb[:, 2] > full_aabb[:, 0]
    print(f"[{label}] visible={int(vis.sum())}", flush=True)
    assert 50 < vis.sum() < sc.n
    for k, o in [("w_means", "v_means"), ("w_quats", "v_quats"), ("w_log_scales", "v_scales"),
                 ("w_opacity_logits", "v_opacities"), ("w_features_dc", "v_dc"), ("w_features_sh", "v_sh")]:
        got, ref = g.host(k).astype(np.float64).reshape(sc.n, -1), want[o].astype(np.float64).reshape(sc.n, -1)
        world_grad_check(got, ref, sc.n, f"{label}/{k}")
        assert not np.any(got[~vis]), k
        # and inside the tool's own acceptance band (proj_bwd_parity.cpp:327)
        assert (np.abs(got - ref) <= 5e-3 + 1e-3 * np.abs(ref)).all(), k


# proj_bwd_parity.cpp:171-180, rows with prim == 0, the first two with the camera-pose gradient: screen gradients drawn by
# the tool, not produced by the compositing backward
@pytest.mark.parametrize("cam", [0, 1])
def test_proj_bwd_parity_rows(gpu, oracle, cam):
    n = R.N_TOOL
    _, rng = R.tool_world(R.SEED_PROJ_BWD)
    q = R.projection_quant_inputs(rng)          # the tool draws its codes and bounds before the rows (:126-142)
    # rows 0 and 1: PINHOLE without a lens / with the OpenCV tier, C * N rows each, camera-major
    for tier in (NONE, OPENCV):
        vs2 = R.screen_gradients(rng, R.C_TOOL * n)
        vs = {k: np.ascontiguousarray(v.reshape((R.C_TOOL, n) + v.shape[1:])[cam]) for k, v in vs2.items()}
        sc, _ = R.tool_scene(gpu, R.SEED_PROJ_BWD, cam, PINHOLE, tier)
        _k9_direct(gpu, oracle, sc, vs, f"proj_bwd_parity PINHOLE tier {tier} cam {cam}", pose=True)
    # row 2: the mip primitive, FISHEYE + thin prism, SH degree 2
    vs2 = R.screen_gradients(rng, R.C_TOOL * n)
    vs = {k: np.ascontiguousarray(v.reshape((R.C_TOOL, n) + v.shape[1:])[cam]) for k, v in vs2.items()}
    sc, _ = R.tool_scene(gpu, R.SEED_PROJ_BWD, cam, FISHEYE, THIN_PRISM, mip=True)
    _k9_direct(gpu, oracle, sc, vs, f"proj_bwd_parity mip FISHEYE THIN_PRISM cam {cam}", sh_degree=2)
    # row 3: packed, EQUISOLID + OpenCV; the tool's rows are camera 0's visible splats, then camera 1's
    nnz = []
    for c in range(R.C_TOOL):
        sc_c, _ = R.tool_scene(gpu, R.SEED_PROJ_BWD, c, EQUISOLID, OPENCV)
        a = oracle.projection_fwd(sc_c)["aabb"]
        nnz.append(int(((a[:, 2] - a[:, 0] > np.float32(1e-3)) & (a[:, 3] - a[:, 1] > np.float32(1e-3))).sum()))
    vs2 = R.screen_gradients(rng, sum(nnz))
    lo = sum(nnz[:cam])
    vs = {k: np.ascontiguousarray(v[lo:lo + nnz[cam]]) for k, v in vs2.items()}
    sc, _ = R.tool_scene(gpu, R.SEED_PROJ_BWD, cam, EQUISOLID, OPENCV)
    _k9_direct(gpu, oracle, sc, vs, f"proj_bwd_parity packed EQUISOLID OPENCV cam {cam}", packed=True, pose=True)
    # row 6: 8-bit SH codes, bounds per 256 cells, thin-prism lens (two rows of another primitive draw in between:
    # the gradients here have the tool's ranges, not its exact stream)
    vs2 = R.screen_gradients(rng, R.C_TOOL * n)
    vs = {k: np.ascontiguousarray(v.reshape((R.C_TOOL, n) + v.shape[1:])[cam]) for k, v in vs2.items()}
    sc, _ = R.tool_scene(gpu, R.SEED_PROJ_BWD, cam, PINHOLE, THIN_PRISM)
    sc.sh_codec, sc.sh_packed, sc.sh_bounds, sc.sh_bounds_stride = 1, q["q8"], q["bounds_cell"], 256
    _k9_direct(gpu, oracle, sc, vs, f"proj_bwd_parity q8 THIN_PRISM cam {cam}")


# fpbo_parity.cpp:169, the quantized 3dgs row: packed projection, EQUISOLID + OpenCV, degree 3, quantization level 1
# with the non-SH moments quantized too, all five non-SH world gradients, two steps (10, 11) on one forward.
# The stream is followed through the four rows before it, so these are the tool's own codes, bounds and gradients.
@pytest.mark.parametrize("cam", [0, 1])
def test_fpbo_parity_quantized_row(gpu, oracle, cam):
    n, C_ = R.N_FPBO, R.C_TOOL
    _, rng = R.tool_world(R.SEED_FPBO, n=n)
    for row in range(4):
        rng.raw(C_ * n * (7 if row == 3 else 10))                 # screen gradients (the 3dgut row has 7 floats per row)
        rng.raw(n * {0: 14, 1: 14, 2: 0, 3: 10}[row])              # world gradients present in that row
        rng.raw(2 * n * (14 + 45))                                 # both moments of all six tensors
        if row == 2:
            rng.raw(n)                                             # per-splat steps
    cells, nb = n * 45, (n + 255) // 256
    b = (rng.raw(2 * cells) & np.uint32(0xFF)).astype(np.uint16)
    codes = np.ascontiguousarray(b[0::2] | (b[1::2] << np.uint16(8)))
    d = rng.raw(2 * nb).reshape(nb, 2)
    uf = lambda col, lo, hi: (np.float32(lo) + ((np.float32(hi) - np.float32(lo)) * (d[:, col] & np.uint32(0xFFFFFF)).astype(np.float32))
                              / np.float32(16777215.0)).astype(np.float32)
    vbounds = np.ascontiguousarray(np.stack([uf(0, -0.5, -0.1), uf(1, 0.1, 0.5)], axis=1), np.float32)

    def scene(c):
        sc, _ = R.tool_scene(gpu, R.SEED_FPBO, c, EQUISOLID, OPENCV, n=n)
        sc.sh_codec, sc.sh_packed, sc.sh_bounds, sc.sh_bounds_stride = 2, codes.copy(), vbounds.copy(), 256 * 45
        return sc
    nnz = []
    for c in range(C_):
        a = oracle.projection_fwd(scene(c))["aabb"]
        nnz.append(int(((a[:, 2] - a[:, 0] > np.float32(1e-3)) & (a[:, 3] - a[:, 1] > np.float32(1e-3))).sum()))
    vs_all = R.screen_gradients(rng, sum(nnz))
    lo = sum(nnz[:cam])
    vs_rows = {k: np.ascontiguousarray(v[lo:lo + nnz[cam]]) for k, v in vs_all.items()}
    shapes = dict(means=(n, 3), quats=(n, 4), log_scales=(n, 3), opacity_logits=(n,), features_dc=(n, 3))
    v_world = {k: rng.uf(int(np.prod(s)), -0.05, 0.05).reshape(s) for k, s in shapes.items()}
    sc = scene(cam)
    g = GpuRun(gpu, sc, packed_projection=True)
    g.projection_fwd()
    assert g.rows == nnz[cam] and 100 < g.rows < n
    D = gpu.lib.DeviceArray
    for k, v in vs_rows.items():
        g.d[k] = D.from_host(v)
    ids = g.host("gaussian_ids")[:g.rows]
    aabb = np.zeros((n, 4), np.float32)
    aabb[ids] = g.host("aabb")[:g.rows]
    vs = {}
    for k, v in vs_rows.items():
        vs[k] = np.zeros((n,) + v.shape[1:], np.float32)
        vs[k][ids] = v
    q = dict(state_packed=np.zeros(cells, np.uint16), state_bounds=np.zeros((nb, 4), np.float32), value_packed=codes.copy(),
             value_bounds=vbounds.copy(), num_sh_buffer=15)
    ns = oracle.zero_non_sh_state(n)
    P = {k: np.ascontiguousarray(getattr(sc, k), np.float32).copy() for k in oracle.WORLD_KEYS[:5]}
    h = R.FPBO_HYPER
    dq, dns = q, ns
    for step in (10, 11):
        dP, _, _, _, dq = g.fused_optimizer(None, None, h, step=step, v_in=v_world, quant_state=dq, non_sh=dns)
        dns = g.non_sh_out
        oracle.fused_projection_bwd_optimizer_q(sc, aabb, vs, P, q, None, None, h, step=step, v_in=v_world, non_sh=ns, densify=False)
        assert np.allclose(dq["value_bounds"], q["value_bounds"], rtol=1e-5, atol=1e-7), step
        assert np.allclose(dq["state_bounds"], q["state_bounds"], rtol=1e-4, atol=1e-6), step
        dv = np.abs(dq["value_packed"].astype(np.int64) - q["value_packed"].astype(np.int64))
        assert dv.max() <= 2 and (dv > 1).mean() < 0.02, (step, int(dv.max()))
        a, b = dq["state_packed"].astype(np.int64), q["state_packed"].astype(np.int64)
        # the tool's own acceptance is +-1 quantum per code (fpbo_parity.cpp:11)
        assert max(np.abs((a & 255) - (b & 255)).max(), np.abs((a >> 8) - (b >> 8)).max()) <= 1, step
        for t, k in enumerate(oracle.NON_SH_KEYS):
            assert np.allclose(dns["bounds"][t], ns["bounds"][t], rtol=1e-4, atol=1e-6), (k, step)
            a, b = dns["packed"][t].astype(np.int64), ns["packed"][t].astype(np.int64)
            du, ds = np.abs((a & 65535) - (b & 65535)), np.abs((a >> 16) - (b >> 16))
            assert (du > 2).mean() < 0.02 and (ds > 2).mean() < 0.02, (k, step, int(du.max()), int(ds.max()))
            assert np.abs(dP[k].astype(np.float64) - P[k]).max() <= 0.02 * 5e-2 * 40 + 1e-6, (k, step)
        # the second step starts from the device's state on both sides
        q = {k: (v.copy() if isinstance(v, np.ndarray) else v) for k, v in dq.items()}
        ns = dict(packed=[x.copy() for x in dns["packed"]], bounds=[x.copy() for x in dns["bounds"]])
        P = {k: v.copy() for k, v in dP.items()}


# fpbo_parity.cpp:163, the mip row: unpacked, FISHEYE + thin prism, SH degree 2, fp32 state, the scale-agnostic step of the
# means, no world gradients, per-splat steps (then step 11 for everyone on the second call), no densify score
@pytest.mark.parametrize("cam", [0, 1])
def test_fpbo_parity_mip_row(gpu, oracle, cam):
    n = R.N_FPBO
    sc, rng = R.tool_scene(gpu, R.SEED_FPBO, cam, FISHEYE, THIN_PRISM, n=n, mip=True)
    for _ in range(2):                      # rows 0 and 1 draw first
        R.fpbo_row_inputs(rng)
    vs2 = R.screen_gradients(rng, R.C_TOOL * n)
    vs = {k: np.ascontiguousarray(v.reshape((R.C_TOOL, n) + v.shape[1:])[cam]) for k, v in vs2.items()}
    keys = oracle.WORLD_KEYS
    shapes = [(n, 3), (n, 4), (n, 3), (n,), (n, 3), (n, 15, 3)]
    g1, g2 = {}, {}
    for k, s in zip(keys, shapes):          # no world gradients in this row (vw_mask 0): the moments follow directly
        g1[k] = rng.uf(int(np.prod(s)), -0.02, 0.02).reshape(s)
        g2[k] = rng.uf(int(np.prod(s)), 0.0, 4e-4).reshape(s)
    steps = (1 + rng.raw(n) % np.uint32(50)).astype(np.int32)
    g = GpuRun(gpu, sc, sh_degree=2)
    g.projection_fwd()
    D = gpu.lib.DeviceArray
    for k, v in vs.items():
        g.d[k] = D.from_host(v)
    aabb, radii = g.host("aabb"), g.host("radii")
    assert 100 < (aabb[:, 2] > aabb[:, 0]).sum() < n
    P = {k: np.ascontiguousarray(getattr(sc, k), np.float32).copy() for k in keys}
    o1 = {k: v.copy() for k, v in g1.items()}
    o2 = {k: v.copy() for k, v in g2.items()}
    h = R.FPBO_HYPER
    lrs = dict(means="lr_means", quats="lr_quats", log_scales="lr_scales", opacity_logits="lr_opacs",
               features_dc="lr_features_dc", features_sh="lr_features_sh")
    d1, d2 = g1, g2
    for call, st in enumerate([steps, None]):
        dP, d1, d2, _ = g.fused_optimizer(d1, d2, h, step=11, steps=st, scale_agnostic=True)
        oracle.fused_projection_bwd_optimizer(sc, aabb, vs, P, o1, o2, h, step=11, steps=st, sh_degree=2, radii=radii, densify=False)
        for k in keys:
            a, b = d1[k].reshape(n, -1).astype(np.float64), o1[k].reshape(n, -1).astype(np.float64)
            assert (np.abs(a - b) <= 1e-3 * np.abs(b) + 1e-4 * (np.abs(b).max(axis=1, keepdims=True) + 1e-12)).all(), ("g1", k, call)
            a, b = d2[k].reshape(n, -1).astype(np.float64), o2[k].reshape(n, -1).astype(np.float64)
            assert (np.abs(a - b) <= 2e-3 * np.abs(b) + 1e-12).all(), ("g2", k, call)
            far = np.abs(dP[k].astype(np.float64) - P[k]) > 0.02 * h[lrs[k]] + 1e-7
            assert far.mean() < 2e-3, (k, call, float(far.mean()))
        # the coefficients above degree 2 are left alone
        assert np.array_equal(dP["features_sh"][:, 8:], sc.features_sh[:, 8:])


@pytest.mark.parametrize("model,tier,dist_type,median,accum", [(PINHOLE, NONE, 0, False, 0), (PINHOLE, OPENCV, 2, True, 1),
                                                              (FISHEYE, THIN_PRISM, 1, False, 3)])
def test_raster_bwd_parity_rows_as_the_tool_batches_them(gpu, oracle, model, tier, dist_type, median, accum):
    """The tool's two cameras in ONE call, as raster_bwd_parity.cpp runs them (C = 2 viewmats, [C,H,W,..]
    cotangents, per-camera lens rows), through the host layer's reference-shaped launch functions; checked
    against the oracle run once per camera."""
    import dataclasses
    from spirula_studio_amd import host
    host.load()
    _, rng = R.tool_world(R.SEED_RASTER_BWD)
    ct = R.raster_bwd_cotangents(rng)
    scs = [R.tool_scene(gpu, R.SEED_RASTER_BWD, cam, model, tier, cotangents=ct)[0] for cam in (0, 1)]
    refs = []
    for cam, sc in enumerate(scs):
        va = dict(dist_type=dist_type, median=False, accum_mode=accum, v_dist_rgb=ct["v_dist_rgb"][cam],
                  v_dist_depth=ct["v_dist_depth"][cam], accum_map=ct["accum_map"][cam])
        refs.append(oracle.pipeline(sc, variant=va))
        assert refs[-1]["proj"]["visible"] > 100
    both = dataclasses.replace(scs[0], viewmat=np.stack([s.viewmat for s in scs]), intrins=np.stack([s.intrins for s in scs]),
                               dist_coeffs=np.stack([s.dist_coeffs for s in scs]), v_rgb=ct["v_rgb"], v_depth=ct["v_depth"], v_T=ct["v_T"])
    eng = host.Engine(both)
    eng.set_variants(dist_type=dist_type, median=median)
    eng.forward()
    eng.backward_with_variants(ct["v_dist_rgb"] if dist_type == 2 else None, ct["v_dist_depth"] if dist_type else None, None,
                               ct["accum_map"] if accum else None, accum_mode=accum)
    n, h, w = both.n, both.height, both.width
    tiles = ((w + 15) // 16) * ((h + 15) // 16)
    n0 = refs[0]["sorted_ids"].size
    assert np.array_equal(eng.cache("sorted_ids"), np.concatenate([refs[0]["sorted_ids"], refs[1]["sorted_ids"] + (np.int64(tiles) << 32)]))
    assert np.array_equal(eng.cache("sorted_flat"), np.concatenate([refs[0]["sorted_flat"], refs[1]["sorted_flat"] + n]))
    assert np.array_equal(eng.cache("offsets"), np.concatenate([refs[0]["offsets"].reshape(-1), refs[1]["offsets"].reshape(-1) + n0]))
    rgb, depth, T = eng.render()
    for cam in (0, 1):
        assert np.abs(rgb[cam] - refs[cam]["fwd"]["rgb"]).max() <= 1e-4
        assert np.abs(T[cam] - refs[cam]["fwd"]["T"]).max() <= 1e-4
        if dist_type:
            assert np.abs(eng.cache("dist_depth").reshape(2, h, w)[cam] - refs[cam]["fwd"]["dist_depth"]).max() <= 1e-4
    if accum:
        a0, a1 = (r["vscreen"]["accum_weight"] for r in refs)
        assert np.allclose(eng.cache("accum_weight"), np.maximum(a0, a1) if accum == 1 else a0 + a1, rtol=1e-3, atol=1e-6)
    for key, v in eng.grads().items():
        r = sum(ref["grads"][key].astype(np.float64) for ref in refs).reshape(n, -1)
        scale = sum(np.abs(ref["grads"][key].astype(np.float64)).reshape(n, -1).max(axis=1, keepdims=True) for ref in refs)
        assert (np.abs(v.reshape(n, -1) - r) <= 2e-3 * scale + 2e-5 * (np.abs(r).mean() + 1e-12)).all(), key
