"""Tile-skip map (compute_tile_active, the tile_active argument of the tile stage;
src/kernels/tile/IntersectTile.cu:309-368 and :62,76-80,95-98,225,240), oracle side."""
import numpy as np
import pytest


def _active_numpy(mask, w, h):
    """Independent restatement: nearest-sample the mask to the render size
    (src/core/Interpolation.cuh:108-120), dilate by one pixel, reduce over 16x16 tiles."""
    hm, wm = mask.shape
    xs = np.arange(w, dtype=np.float32)
    ys = np.arange(h, dtype=np.float32)
    u = ((xs + np.float32(0.5)) * np.float32(wm)) / np.float32(w) - np.float32(0.5)
    v = ((ys + np.float32(0.5)) * np.float32(hm)) / np.float32(h) - np.float32(0.5)
    sx = np.clip(np.floor(u + np.float32(0.5)).astype(np.int64), 0, wm - 1)
    sy = np.clip(np.floor(v + np.float32(0.5)).astype(np.int64), 0, hm - 1)
    full = mask[sy][:, sx].astype(bool)
    grown = full.copy()
    for dy in (-1, 0, 1):
        for dx in (-1, 0, 1):
            sh = np.zeros_like(full)
            ys0, ys1 = max(dy, 0), h + min(dy, 0)
            xs0, xs1 = max(dx, 0), w + min(dx, 0)
            sh[ys0:ys1, xs0:xs1] = full[ys0 - dy:ys1 - dy, xs0 - dx:xs1 - dx]
            grown |= sh
    th, tw = (h + 15) // 16, (w + 15) // 16
    pad = np.zeros((th * 16, tw * 16), bool)
    pad[:h, :w] = grown
    return pad.reshape(th, 16, tw, 16).any(axis=(1, 3)).astype(np.int32).reshape(-1)


@pytest.mark.parametrize("w,h,wm,hm", [(100, 70, 100, 70), (100, 70, 37, 23), (64, 48, 200, 150), (33, 17, 5, 3)])
def test_compute_tile_active(oracle, w, h, wm, hm):
    rng = np.random.default_rng(w * 7 + hm)
    for density in (0.0, 0.002, 0.05, 1.0):
        mask = (rng.random((hm, wm)) < density).astype(np.uint8)
        assert np.array_equal(oracle.compute_tile_active(mask, w, h), _active_numpy(mask, w, h)), density


def test_single_pixel_reaches_neighbour_tiles_through_the_one_pixel_pad(oracle):
    w = h = 64
    mask = np.zeros((h, w), np.uint8)
    mask[16, 16] = 1          # first pixel of tile (1,1): tiles (0,0), (0,1), (1,0) see it through the pad
    a = oracle.compute_tile_active(mask, w, h).reshape(4, 4)
    want = np.zeros((4, 4), np.int32)
    want[:2, :2] = 1
    assert np.array_equal(a, want)
    mask[:] = 0
    mask[20, 20] = 1          # interior pixel: its own tile only
    a = oracle.compute_tile_active(mask, w, h).reshape(4, 4)
    want[:] = 0
    want[1, 1] = 1
    assert np.array_equal(a, want)


def test_masked_tile_stage_is_the_unmasked_one_with_dead_tiles_removed(pkg, oracle):
    sc = pkg.scenes.tiny_scene(n=900, width=160, height=96, seed=41)
    sc.log_scales[::9] += 1.5     # some splats spanning many tiles, both enumeration orders
    rng = np.random.default_rng(5)
    live = (rng.random(sc.tile_w * sc.tile_h) < 0.6).astype(np.int32)
    u = oracle.pipeline(sc, backward=False)
    m = oracle.pipeline(sc, backward=False, tile_active=live)
    assert m["pads"] == 0
    tile_of = (u["isect_ids"] >> 32).astype(np.int64)
    keep = live[tile_of] != 0
    assert 0 < keep.sum() < keep.size
    assert np.array_equal(m["isect_ids"], u["isect_ids"][keep])
    assert np.array_equal(m["flatten_ids"], u["flatten_ids"][keep])
    assert np.array_equal(m["counts"], np.bincount(u["flatten_ids"][keep], minlength=sc.n))
    # dead tiles get an empty range: background there, and live tiles render exactly as before
    T = m["fwd"]["T"]
    ty, tx = np.divmod(np.arange(live.size), sc.tile_w)
    for t in range(live.size):
        ys, xs = slice(ty[t] * 16, ty[t] * 16 + 16), slice(tx[t] * 16, tx[t] * 16 + 16)
        if live[t]:
            assert np.array_equal(m["fwd"]["rgb"][ys, xs], u["fwd"]["rgb"][ys, xs])
            assert np.array_equal(T[ys, xs], u["fwd"]["T"][ys, xs])
        else:
            assert np.all(T[ys, xs] == 1.0) and not np.any(m["fwd"]["rgb"][ys, xs])
