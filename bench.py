#!/usr/bin/env python3
"""Benchmark of the splat-raster hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2]

One step = one forward+backward iteration of the path on a seeded synthetic scene whose inputs
and pixel cotangents are already resident in HBM: zero radii -> projection+SH (with the tile
count fused) -> int64 scan (the first iteration reads the 16 bytes of counts back as the reference
does, later ones leave them on the device; --blocking-counts reads them every time) -> key write ->
64-bit radix sort -> tile offsets -> compositing forward -> zero the gradient rows -> compositing
backward -> projection backward. After the headline configuration the other four run briefly in the
same process (all_configs).
Prints ONE JSON line: the benchmark's metric (forward+backward iterations/s), a `roofline` object for the
kernel that takes the most time, and a `cpu_baseline` object (the CPU oracle timed on this host).
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0   # MI355X published HBM3E peak


def algorithmic_bytes(N, V, K, K_f, K_b, P, T, S, sort_sweeps):
    """Minimum HBM bytes per stage for one iteration: every array an algorithm of this shape must
    read or write once. N splats, V visible, K splat-tile pairs, K_f / K_b pairs the forward /
    backward actually need, P pixels, T tiles, S bytes of higher-order SH storage per splat;
    sort_sweeps = 8-bit digits of the whole sort key (32 depth bits + the tile bits): the figure the
    metric is defined on, whatever the sort does -- the tile-segmented sort moves the array only once per
    digit of the tile bits plus once in the per-tile sorts, and is still divided by this figure."""
    return {
        "K1": N * (44 + 20) + V * (12 + S + 40 + 4),
        "K2": N * 16 + V * (24 + 8) + (N - V) * 8,
        "K3": N * 16,
        "K4": N * 16 + V * (24 + 4 + 16) + K * 12,
        "K5": sort_sweeps * K * 24,
        "K6": K * 8 + T * 4,
        "K7": K_f * 44 + P * 24,
        "K8": P * 32 + K_b * 44 + K_b * 40 + N * 40,
        "K9": N * 16 + V * (56 + S + 40) + V * 236 + N * 236,
    }


def done_bytes(ab, N, V, K, T, S, sort_sweeps_done, fused_count, tile_sort, listed, packed, k9_all_rows, world_rows):
    """The same table for the work this build's stage order really does (the contract figures above price the
    reference's stage order): the key array swept `sort_sweeps_done` times, no separate count pass when the projection
    counts tiles itself, K4 and K9 over the visible rows only when a work list or the packed rows drive them, and K9's
    gradient rows written once -- all N of them when the launch covers every splat (it stores zeros for culled
    ones, so nothing is zero-filled beforehand), else the V visible ones plus as many re-zeroed from the iteration
    before."""
    d = dict(ab)
    if fused_count:
        d["K2"] = 0
    rows = V if packed else N                      # rows the scan and the key write run over
    d["K3"] = rows * 16
    d["K4"] = (V * (4 if listed else 0) + (V if (listed or packed) else N) * 16 + V * 44 + K * 12)
    d["K5"] = sort_sweeps_done * K * 24 + (K * 8 + T * 4 if tile_sort else 0)
    if tile_sort:
        d["K6"] = 0
    reads = (V * (4 if listed else 0) if (listed or packed) else N * 16) + V * (56 + S + 40)
    if packed and world_rows:
        reads += 0                                 # the parameter planes replace the gathers one for one
    d["K9"] = reads + (N * 236 if k9_all_rows else V * 236 * 2)
    return d


def tile_need(offsets, last_ids, n_isects, width, height):
    """K_b: per tile, (largest last_id over its pixels) - range start + 1, summed over tiles."""
    import numpy as np
    tw, th = (width + 15) // 16, (height + 15) // 16
    pad = np.full((th * 16, tw * 16), -1, np.int64)
    pad[:height, :width] = last_ids.reshape(height, width)
    tmax = pad.reshape(th, 16, tw, 16).max(axis=(1, 3)).reshape(-1)
    start = offsets.astype(np.int64)
    end = np.concatenate([start[1:], [n_isects]])
    need = np.clip(np.minimum(tmax, end - 1) - start + 1, 0, None)
    need[end <= start] = 0
    return int(need.sum())


def _time_oracle(oracle_lib, sc, threads, min_iters, budget_s):
    """Seconds per iteration of the CPU oracle's forward+backward on `threads` threads, and its last result."""
    oracle_lib.lib().or_set_num_threads(threads)
    t0 = time.time()
    iters, res = 0, None
    while iters < min_iters or (time.time() - t0 < budget_s and iters < 20):
        res = oracle_lib.pipeline(sc)
        iters += 1
        if time.time() - t0 > 3 * budget_s:
            break
    return (time.time() - t0) / iters, iters, res


def lavapipe_status():
    """The baseline the benchmark definition asks for is the reference's Vulkan path on Mesa lavapipe. It needs the reference
    tree, slangc and a Vulkan loader with the lavapipe ICD on this host; say what is missing instead of a number."""
    import glob
    import shutil
    missing = []
    if not os.path.isdir("/root/reference/src/backend/vulkan"):
        missing.append("the reference source tree (only this repository travels to the GPU box)")
    if not shutil.which("slangc"):
        missing.append("slangc (the reference compiles its shaders to SPIR-V at build time and commits none)")
    if not (glob.glob("/usr/lib/x86_64-linux-gnu/libvulkan.so*") or glob.glob("/usr/lib64/libvulkan.so*")):
        missing.append("a Vulkan loader")
    if not (glob.glob("/usr/share/vulkan/icd.d/lvp_icd*.json") or glob.glob("/etc/vulkan/icd.d/lvp_icd*.json")):
        missing.append("the lavapipe ICD")
    return "unavailable: missing " + "; ".join(missing) if missing else "present but not driven by this harness"


def cpu_baseline(pkg, cfg, sc):
    """The CPU oracle (this repository's restatement, not the reference implementation) on this host's cores, on
    the stated workload itself: whole iterations of configuration `cfg` on every core; for the headline
    configuration also one iteration on a single thread and configuration 1 on every core. Returns the JSON
    object and K_f, the number of (splat, tile) pairs the forward needs, which only the oracle records."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib
    L = oracle_lib.lib()
    cores = L.or_num_threads()
    dt, iters, res = _time_oracle(oracle_lib, sc, cores, 3 if sc.n <= 1_000_000 else 1, 10.0)
    out = {"value": 1.0 / dt, "unit": "iters/s", "cores": cores, "kind": "port",
           "sample": f"{iters} whole iteration(s) of config {cfg} (N={sc.n}, {sc.width}x{sc.height}) on {cores} threads: "
                     f"{dt * 1e3:.0f} ms each; own CPU oracle, not the reference implementation",
           "lavapipe": lavapipe_status()}
    if cfg == 2:
        dt1, it1, _ = _time_oracle(oracle_lib, sc, 1, 1, 0.0)
        out["single_thread"] = {"value": 1.0 / dt1, "unit": "iters/s", "cores": 1, "sample": f"{it1} iteration(s), {dt1 * 1e3:.0f} ms each"}
        sc1 = pkg.scenes.make_scene(1)
        dtc, itc, _ = _time_oracle(oracle_lib, sc1, cores, 3, 3.0)
        out["config1"] = {"value": 1.0 / dtc, "unit": "iters/s", "cores": cores, "sample": f"{itc} iteration(s) of config 1, {dtc * 1e3:.0f} ms each"}
    L.or_set_num_threads(cores)
    return out, int(res["fwd"]["K_f"])


def run_config(args, pkg, host, lib, np, with_cpu):
    """One configuration: builds the scene, times args.steps iterations, and returns the JSON object."""
    L = lib.load()
    cfg = args.config
    # config 4 looks out from inside the scene and sees an eighth of it: the reference's packed projection (compacted
    # nnz-row outputs) is its mode for such views and the faster one here, so it is this config's default
    if cfg == 4 and not (args.dense_projection or args.reference_order or args.cameras > 1):
        args.packed_projection = True
        # ... and its visible splats are scattered over the parameter arrays: the packed projection keeps their
        # parameters for the projection backward (not with the fused optimizer, which reads them where they live)
        args.packed_world_rows = not (args.fused_optimizer or args.no_packed_world_rows)
    t_gen = time.time()
    sc = pkg.scenes.make_scene(cfg, n=args.n)
    if args.fused_optimizer and args.quantization_level == 1:
        if sc.sh_codec != 0:
            sc = pkg.scenes.make_scene(cfg, n=args.n, sh_codec=0)
        pkg.scenes.apply_sh_codec(sc, 2, bounds_stride=256 * 45)
    if args.fisheye:
        sc.camera_model = pkg.scenes.CAM_FISHEYE
        f = sc.width / math.pi
        sc.intrins = np.array([f, f, sc.width / 2.0, sc.height / 2.0], np.float32)
    if args.lens != "none":
        sc = pkg.scenes.with_lens(sc, ["none", "opencv", "thin_prism", "rational"].index(args.lens))
    if args.mip:
        sc.antialiased = True
    ncam = args.cameras
    if ncam > 1:
        if args.packed_projection or args.fused_optimizer or args.dist_type or args.median or args.accum_mode:
            sys.exit("bench.py: --cameras runs the plain forward + backward only")
        vms = []
        for k in range(ncam):   # the same view, each camera a little further along x
            vm = np.array(sc.viewmat, np.float32).copy()
            vm[0, 3] += 0.05 * k
            vms.append(vm)
        sc.viewmat = np.stack(vms)
        sc.intrins = np.stack([np.asarray(sc.intrins, np.float32)] * ncam)
        if getattr(sc, "dist_coeffs", None) is not None:
            sc.dist_coeffs = np.stack([np.asarray(sc.dist_coeffs, np.float32)] * ncam)
        for name in ("v_rgb", "v_depth", "v_T"):
            setattr(sc, name, np.ascontiguousarray(np.stack([np.asarray(getattr(sc, name), np.float32)] * ncam)))
    t_gen = time.time() - t_gen
    native = not args.reference_order
    deferred = native and not args.whole_key_sort and not args.blocking_counts and ncam == 1   # needs the tile-segmented sort
    eng = host.Engine(sc, fuse_tile_count=native, visible_list=native and not args.packed_projection, packed_rows=native,
                      overwrite_world_grads=native, packed_projection=args.packed_projection, packed_vscreen=native,
                      tile_sort=native and not args.whole_key_sort, deferred_counts=deferred,
                      packed_world_rows=args.packed_world_rows,
                      backward_schedule={"auto": -1, "rows": 0, "lanes": 1}[args.backward_schedule])

    hyper = dict(lr_means=1.6e-6, lr_quats=1e-5, lr_scales=5e-5, lr_opacs=5e-4, lr_features_dc=2.5e-5, lr_features_sh=1.25e-6)
    adam_step = [0]

    # the accumulation of the loss map rides with the fused optimizer as the trainer's step does; alone, or with
    # distortion / median, it goes through the variants' backward
    fused_accum = bool(args.fused_optimizer and args.accum_mode and not (args.dist_type or args.median))
    variants = (args.dist_type or args.median or args.accum_mode) and not fused_accum
    if fused_accum:
        amap_dev = lib.DeviceArray.from_host(np.random.default_rng(1).uniform(0, 1, (ncam, sc.height, sc.width)).astype(np.float32))
        eng.set_loss_map(amap_dev.ptr, args.accum_mode)
    if variants:
        rng = np.random.default_rng(1)
        eng.set_variants(args.dist_type, args.median)
        u = lambda *shape: lib.DeviceArray.from_host(rng.uniform(-1, 1, shape).astype(np.float32))
        vcot = dict(rgb=u(sc.height, sc.width, 3), depth=u(sc.height, sc.width), med=u(sc.height, sc.width),
                    amap=lib.DeviceArray.from_host(rng.uniform(0, 1, (sc.height, sc.width)).astype(np.float32)))

    def backward():
        if variants:
            host.check(eng.h.ssrh_backward_with_variants(eng.d_vrgb.ptr, eng.d_vdepth.ptr, eng.d_vT.ptr, vcot["rgb"].ptr,
                                                         vcot["depth"].ptr, vcot["med"].ptr if args.median else None,
                                                         vcot["amap"].ptr if args.accum_mode else None, args.accum_mode))
        elif args.fused_optimizer:
            adam_step[0] += 1
            eng.backward_fused_optimizer(hyper, adam_step[0], scale_agnostic_mean=args.scale_agnostic_mean,
                                         quantization_level=args.quantization_level, non_sh_optim_bits=args.non_sh_optim_bits)
        else:
            eng.backward()

    def run(iters):
        if not (args.fused_optimizer or variants):
            return eng.time_iterations(iters)
        out = np.zeros(iters, np.float32)
        for i in range(iters):
            t = time.perf_counter()
            eng.forward()
            backward()
            lib.check(L.ssr_device_synchronize())
            out[i] = (time.perf_counter() - t) * 1e3
        return out

    run(max(args.warmup, 1))
    lib.check(L.ssr_device_synchronize())
    t0 = time.perf_counter()
    ms = run(args.steps)
    lib.check(L.ssr_device_synchronize())
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps

    # per-stage device times, outside the timed region (events around every stage)
    eng.set_stage_profiling(True)
    acc = {}
    reps = 5
    for _ in range(reps):
        eng.forward()
        backward()
        for k, v in eng.stage_times().items():
            acc[k] = acc.get(k, 0.0) + v / reps
    eng.set_stage_profiling(False)

    # problem sizes from the device results
    aabb = eng.cache("aabb").reshape(-1, 4)
    V = int((aabb[:, 2] > aabb[:, 0]).sum())   # packed form: every one of its nnz rows
    K = eng.n_isects
    P1, T1 = sc.width * sc.height, sc.tile_w * sc.tile_h
    P, T = ncam * P1, ncam * T1    # several cameras: C images of pixels and of tiles, C*N projected rows
    offs, last = eng.cache("offsets"), eng.cache("last_ids")
    K_b = 0
    for c in range(ncam):   # positions in offsets and last_ids are absolute, so each image is taken with its own end
        end = int(offs[(c + 1) * T1]) if c + 1 < ncam else K
        K_b += tile_need(offs[c * T1:(c + 1) * T1], last[c * P1:(c + 1) * P1], end, sc.width, sc.height)
    # K_f, the pairs the forward needs (it also reads the splat that ends a pixel), is recorded by the CPU oracle only:
    # taken from the cpu_baseline leg when that runs on this very scene, else bounded below by K_b
    K_f, cpu = K_b, None
    plain_scene = not (args.fisheye or args.lens != "none" or args.mip or ncam > 1 or args.n)
    if with_cpu:
        if plain_scene and not (args.fused_optimizer and args.quantization_level == 1):
            cpu, K_f = cpu_baseline(pkg, cfg, sc)
        else:
            cpu, _ = cpu_baseline(pkg, cfg, pkg.scenes.make_scene(cfg))
    S = 180 if sc.sh_codec == 0 else (47 if sc.sh_codec == 3 else 45 + 8 * 45 / 256)
    tile_bits = max(T - 1, 0).bit_length()
    tile_sort = native and not args.whole_key_sort
    sort_sweeps = (32 + tile_bits + 7) // 8
    sort_sweeps_done = (tile_bits + 7) // 8 + 1 if tile_sort else sort_sweeps
    ab = algorithmic_bytes(ncam * sc.n, V, K, K_f, K_b, P, T, S, sort_sweeps)
    if tile_sort:   # the tile-segmented sort writes the offsets itself; its K6 slot times the launch-order kernels
        ab["K5"] += ab["K6"]
        ab["K6"] = 0
    total_bytes = sum(ab.values())
    # ... and what this stage order really moves (done_bytes): K9 covers every row when the engine says its launch
    # overwrites them all (store mode, not packed, no list or a list holding half the splats)
    listed = native and not args.packed_projection
    k9_all_rows = (not native) or (not args.packed_projection and V * 2 >= ncam * sc.n)
    abd = done_bytes(ab, ncam * sc.n, V, K, T, S, sort_sweeps_done, fused_count=native, tile_sort=tile_sort, listed=listed,
                     packed=args.packed_projection, k9_all_rows=k9_all_rows, world_rows=args.packed_world_rows) if native else dict(ab)
    total_done = sum(abd.values())
    dom = max(acc, key=acc.get)
    dom_gbs = abd[dom] / (acc[dom] * 1e-3) / 1e9 if acc[dom] > 0 else 0.0
    traffic = None
    valu_inst = None     # profiled VALU wavefront instructions per launch of the dominant kernel
    prof = {}
    # the profiles were taken with this script's default arguments for each config: they describe no other variant
    default_run = (native and ncam == 1 and tile_sort and args.packed_projection == (cfg == 4) and
                   args.packed_world_rows == (cfg == 4) and not args.n and args.backward_schedule == "auto" and
                   not (variants or args.fused_optimizer or args.lens != "none" or args.fisheye or args.mip))
    tpath = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    prof, traffic, valu_inst, valu_busy, gpu_cycles = {}, None, None, None, None
    if default_run and os.path.exists(tpath):
        try:
            prof = json.load(open(tpath))
            traffic = prof.get(f"config{cfg}", {}).get(dom)
            valu_inst = prof.get(f"config{cfg}_valu_wave_instructions", {}).get(dom)
            valu_busy = prof.get(f"config{cfg}_valu_busy_cycles_per_simd", {}).get(dom)
            gpu_cycles = prof.get(f"config{cfg}_gpu_cycles", {}).get(dom)
        except Exception:
            prof, traffic, valu_inst, valu_busy, gpu_cycles = {}, None, None, None, None
    # What the sort really does, beside the charged figure of stage_algorithmic_GBs (which prices the reference's
    # whole-key sweeps): pairs per second through the whole stage, the sweeps done, and the HBM bytes the profile saw
    sort_ms = acc.get("K5", 0.0) + (0.0 if tile_sort else acc.get("K6", 0.0))   # sort + tile offsets
    sort_info = {"pairs": K, "ms": sort_ms,
                 "Gpairs_per_s": K / (sort_ms * 1e-3) / 1e9 if sort_ms > 0 else None,
                 "key_sweeps_done": sort_sweeps_done, "key_sweeps_charged": sort_sweeps,
                 "hbm_bytes_profiled": prof.get(f"config{cfg}", {}).get("K5"),
                 "hbm_GBs_profiled": (prof[f"config{cfg}"]["K5"] / (acc["K5"] * 1e-3) / 1e9
                                      if prof.get(f"config{cfg}", {}).get("K5") and acc.get("K5", 0.0) > 0 else None)}
    at = prof.get(f"config{cfg}_l2_atomic_requests", {})
    atomic_info = {"l2_atomic_requests_profiled": at or None,
                   "K8_G_atomic_requests_per_s": (at["K8"] / (acc["K8"] * 1e-3) / 1e9 if at.get("K8") and acc.get("K8", 0.0) > 0 else None),
                   "note": "K8 adds a fragment's ten gradient floats as one or two row requests (TCC_ATOMIC_sum counts requests, not floats)"}

    out = {
        "metric": "fwd+bwd raster iters/sec at 1M SH3 1080p; % of HBM roofline",
        "value": args.steps / wall,
        "unit": "iters/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"config {cfg}: {sc.name}, N={sc.n}, {sc.width}x{sc.height}, "
                               f"{['pinhole', 'fisheye', 'equisolid', 'equirectangular'][sc.camera_model]}"
                               f"{'' if not sc.distortion else ' + ' + args.lens + ' lens'}, SH3 "
                               f"{['fp32', 'ref-q8', 'ref-q16', 'int8*fp16scale'][sc.sh_codec]}, tile 16x16, seed {pkg.scenes.CONFIGS[cfg]['seed']:#x}",
                   "visible": V, "n_isects": K, "K_f": K_f, "K_b": K_b, "tiles": T, "pixels": P,
                   "stage_order": ("fused tile count, visible-splat work list, packed fragment rows, packed gradient rows, plain-store gradients"
                                   + (", tile-segmented sort" if tile_sort else "")
                                   + (", intersection count left on the device after the first iteration" if deferred else "") if native else "reference order")
                                  + (", antialiased (mip) primitive" if args.mip else "")
                                  + (f", {ncam} cameras per iteration in one call" if ncam > 1 else "")
                                  + (", packed projection outputs" if args.packed_projection else "")
                                  + (", parameter rows of the visible splats kept for the projection backward" if args.packed_world_rows else "")
                                  + (", projection backward fused with Adam" + ((" (quantized SH state" + (" and non-SH moments)" if args.non_sh_optim_bits == 16 else ")")) if args.quantization_level else "")
                                     if args.fused_optimizer else "")
                                  + (f", compositing variants dist_type={args.dist_type} median={int(args.median)} accum_mode={args.accum_mode}" if variants else "")
                                  + (f", loss map accumulated per splat (accum_mode={args.accum_mode})" if fused_accum else ""),
                   "device_ms_per_iter_median": float(np.median(ms))},
        # two byte counts: the contract's (the reference's stage order: whole-key sort sweeps, a separate count pass,
        # zero-filled gradient buffers) and the bytes of the work this stage order does; each over the same time
        "hbm_roofline_frac_whole_iteration": total_bytes / (float(np.median(ms)) * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "hbm_roofline_frac_whole_iteration_done": total_done / (float(np.median(ms)) * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "algorithmic_bytes_per_iter": total_bytes,
        "algorithmic_bytes_done": total_done,
        "stage_algorithmic_bytes_done": {k: int(abd[k]) for k in acc},
        "sort_sweeps": {"charged": sort_sweeps, "done": sort_sweeps_done},
        "sort": sort_info,
        "atomics": atomic_info,
        "stage_ms": {k: round(v, 4) for k, v in acc.items()},
        "stage_algorithmic_GBs": {k: round(abd[k] / (acc[k] * 1e-3) / 1e9, 1) if acc[k] > 0 and abd[k] > 0 else None for k in acc},
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": dom_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": dom_gbs / HBM_PEAK_GBS, "traffic": traffic,
                     "algorithmic_bytes_per_launch": abd[dom], "avg_launch_ms": acc[dom]},
    }
    if valu_inst and valu_busy and gpu_cycles:
        # The dominant kernel is bound by vector-instruction issue, which neither "hbm" nor "mfma" names. From the
        # committed profile of this configuration: wavefront instructions per launch, the SIMD cycles they occupy by
        # instruction class (fp32 add/mul/fma 2.7, transcendental 7.8, the rest 4.1 cycles: measured rates,
        # profiles/valu_issue_rates.md) spread over the 1024 SIMDs, and the kernel's own cycle count
        # (GRBM_GUI_ACTIVE / 8) in the same profiling run. A model, and a lower bound where DPP forms are many.
        out["roofline"]["valu_issue"] = {"wave_instructions_per_launch": valu_inst,
                                         "modelled_busy_cycles_per_simd": valu_busy, "kernel_cycles": gpu_cycles,
                                         "frac_of_issue_cycles": valu_busy / gpu_cycles}
    if cpu is not None:
        out["cpu_baseline"] = cpu   # one camera of the configuration
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", type=int, default=2, help="1..5 (the five benchmark configurations; 2 is the headline)")
    ap.add_argument("--n", type=int, default=None, help="override the number of Gaussians")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--reference-order", action="store_true",
                    help="run the stages exactly as the reference does (separate count pass, atomic K9 into zero-filled buffers)")
    ap.add_argument("--backward-schedule", choices=["auto", "rows", "lanes"], default="auto",
                    help="cut of the compositing backward: chosen from the tiles per visible splat, or forced")
    ap.add_argument("--whole-key-sort", action="store_true",
                    help="six whole-array digit passes + the offsets kernel instead of the tile-segmented sort")
    ap.add_argument("--lens", choices=["none", "opencv", "thin_prism", "rational"], default="none",
                    help="widened row: the scene's camera with a lens-distortion tier (mild preset coefficients)")
    ap.add_argument("--fisheye", action="store_true",
                    help="widened row: view the scene through an equidistant fisheye spanning 180 degrees of the image width")
    ap.add_argument("--packed-projection", action="store_true",
                    help="run the packed form of the projection (compacted nnz-row outputs; the reference's training default)")
    ap.add_argument("--dense-projection", action="store_true",
                    help="config 4: keep the [N]-row projection outputs instead of the packed rows its sparse view defaults to")
    ap.add_argument("--fused-optimizer", action="store_true",
                    help="backward = compositing backward + projection backward fused with the Adam step "
                         "(the reference's FPBO mode); K9 then includes the optimizer's 1.4 kB/splat of traffic")
    ap.add_argument("--quantization-level", type=int, default=0, choices=[0, 1],
                    help="with --fused-optimizer: 1 = SH values as 16-bit codes and their Adam moments as 8-bit cells "
                         "(the reference's default level); the scene's SH is then stored at 16 bits, one bound per 256 splats")
    ap.add_argument("--scale-agnostic-mean", action="store_true", help="with --fused-optimizer: the scale-agnostic step of the means")
    ap.add_argument("--mip", action="store_true", help="the antialiased primitive (blur 0.1, opacity compensation)")
    ap.add_argument("--non-sh-optim-bits", type=int, default=32, choices=[32, 16],
                    help="with --quantization-level 1: 16 = the moments of the non-SH tensors as 16-bit cells too (what the reference's trainer sets)")
    ap.add_argument("--dist-type", type=int, default=0, help="compositing variant: 1 depth distortion, 2 rgb + depth distortion")
    ap.add_argument("--median", action="store_true", help="compositing variant: also render the median depth and back-propagate it")
    ap.add_argument("--accum-mode", type=int, default=0, help="compositing variant: accumulate a pixel weight map per splat (1 max, 2 sum, 3 avg)")
    ap.add_argument("--packed-world-rows", action="store_true",
                    help="with the packed projection: keep the visible splats' parameters (64 bytes each) for the projection backward")
    ap.add_argument("--no-packed-world-rows", action="store_true", help="config 4: gather the parameters in the projection backward")
    ap.add_argument("--blocking-counts", action="store_true",
                    help="wait for the intersection count between the scan and the key write in every iteration, as the reference "
                         "does. Default: only the first iteration reads it; after that the key arrays are sized from the previous "
                         "count, the count follows asynchronously, and an overflow is refused before the backward uses anything")
    ap.add_argument("--cameras", type=int, default=1,
                    help="render C cameras per iteration in one call ([C,N] layout, plain path only); an iteration is then C images")
    ap.add_argument("--no-all-configs", action="store_true",
                    help="headline run only: leave out the short runs of the other four configurations (all_configs)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run device copies / fills of known size (for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus must be 1 (the path has no multi-GPU part)", file=sys.stderr)
        sys.exit(2)

    import numpy as np

    import ssr_pkg
    pkg = ssr_pkg.load()
    from spirula_studio_amd import host, lib

    if args.copy_calibration:
        L = lib.load()
        lib.check(L.ssr_init(0))
        nbytes = 1 << 30
        a, b = lib.DeviceArray((nbytes,), np.uint8), lib.DeviceArray((nbytes,), np.uint8)
        for _ in range(5):
            lib.check(L.ssr_fill_u32(a.ptr, 1, nbytes // 4, None))          # writes 1 GiB
            lib.check(L.ssr_memcpy(b.ptr, a.ptr, nbytes, lib.D2D, None, 1))  # reads 1 GiB, writes 1 GiB
        lib.check(L.ssr_device_synchronize())
        print(json.dumps({"copy_calibration_bytes": nbytes, "launches": 5}))
        return

    default_plain = not (args.reference_order or args.whole_key_sort or args.lens != "none" or args.fisheye or args.packed_projection
                         or args.dense_projection or args.fused_optimizer or args.mip or args.dist_type or args.median
                         or args.accum_mode or args.packed_world_rows or args.no_packed_world_rows or args.blocking_counts
                         or args.cameras != 1 or args.n)
    out = run_config(args, pkg, host, lib, np, with_cpu=not args.no_cpu_baseline)
    if default_plain and not args.no_all_configs:
        # the other four benchmark configurations, a short run each in this same process (no CPU leg; K_f then
        # stands at its lower bound K_b): iterations/s and both roofline fractions per configuration
        import copy
        rows = []
        for c in [1, 2, 3, 4, 5]:
            if c == args.config:
                r = out
            else:
                a2 = copy.copy(args)
                a2.config, a2.steps, a2.warmup = c, min(args.steps, 20), min(args.warmup, 5)
                r = run_config(a2, pkg, host, lib, np, with_cpu=False)
            dom = r["roofline"]["kernel"]
            rows.append({"workload": r["config"]["workload"], "ms_per_step": r["ms_per_step"], "iters_per_s": r["value"],
                         "steps": r["steps"], "frac_contract": r["hbm_roofline_frac_whole_iteration"],
                         "frac_done": r["hbm_roofline_frac_whole_iteration_done"], "dominant_kernel": dom,
                         "dominant_kernel_ms": r["stage_ms"][dom], "dominant_kernel_frac": r["roofline"]["frac"]})
        out["all_configs"] = rows
    print(json.dumps(out))


if __name__ == "__main__":
    main()
