"""Lane statistics of the compositing backward on the oracle's forward (CPU): of the pixels a (splat,
pixel-block) visit covers, how many composite the splat, for blocks of 8x8 (one wavefront per visit), 4x4 and
2x2 pixels. Run with -s to print the table; LANE_STATS_FULL=1 runs benchmark configurations 2 and 5 at full size
(tens of seconds), otherwise reduced copies that keep the splat footprint in pixels."""
import os

import numpy as np
import pytest


def _stats(oracle, sc):
    r = oracle.pipeline(sc, backward=False)
    st = oracle.raster_lane_stats(r["proj"], sc.width, sc.height, r["offsets"], r["sorted_flat"], r["fwd"]["last_ids"])
    st["K"] = int(r["isect_ids"].size)
    st["K_b"] = r["fwd"]["K_b"]
    st["visits_bwd"] = r["fwd"]["visits_bwd"]
    return st


@pytest.mark.parametrize("cfg", [2, 5])
def test_lane_utilisation(pkg, oracle, cfg):
    full = os.environ.get("LANE_STATS_FULL") == "1"
    if full:
        sc = pkg.scenes.make_scene(cfg)
    else:   # same camera and splat sizes on a smaller image with proportionally fewer splats
        sc = pkg.scenes.make_scene(cfg, n=60000 if cfg == 2 else 100000)
    st = _stats(oracle, sc)
    v, u, p = st["visits"], st["utilisation"], st["productive"]
    print(f"\n[lane stats cfg{cfg} N={sc.n} {sc.width}x{sc.height}] K={st['K']} K_b={st['K_b']} compositing pairs={st['pairs']}")
    for bs in (8, 4, 2):
        print(f"  block {bs}x{bs}: visits {v[bs]:>11d}  with >=1 compositing pixel {p[bs] / max(1, v[bs]):6.1%}  "
              f"lanes compositing {u[bs]:6.1%}  lane slots {v[bs] * bs * bs:>12d}")
    assert v[8] == st["visits_bwd"]                      # the same visit count the forward statistics give
    assert st["pairs"] > 0 and 0.0 < u[8] < u[4] < u[2] <= 1.0
    assert v[8] * 64 >= v[4] * 16 >= v[2] * 4 >= st["pairs"]   # finer blocks never cover more lane slots
