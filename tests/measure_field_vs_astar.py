"""CPU measurement (not collected by pytest): how far is the goal-rooted distance-field
formulation of the geodesic from the reference's own value?

The reference measures geodesic(goal -> agent) with Detour's A* (PathFinder.cpp:485-541,
DetourNavMeshQuery.cpp:945-1137), whose corridor depends on the agent's position through the
heuristic and on the order in which polygons were first reached
(DetourNavMeshQuery.cpp:1052-1058).  A distance field rooted at the goal has one corridor per
polygon, whatever the agent's position.  For goal -> agent queries of the second and fourth
benchmark configurations this script string-pulls both corridors with the same funnel and
prints the distribution of the relative difference.

    python tests/measure_field_vs_astar.py [queries per configuration, default 12000]
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

from bps_nav_amd import scenes  # noqa: E402
from oracle import bpo  # noqa: E402


def measure(lib, config, num_scenes, goals_per_scene, agents_per_goal, dmin, dmax, seed):
    """goal -> agent queries: for every goal, agents spread over the scene; pairs whose reference
    distance lies in [dmin, dmax] (the configuration's episode range, shrinking as the agent
    approaches) are kept."""
    f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
    u32p = np.ctypeslib.ndpointer(np.uint32, flags="C_CONTIGUOUS")
    lib.L.bpo_nav_geodesic_field.argtypes = [bpo.C.c_void_p, f32p, u32p, f32p, u32p, bpo.C.c_uint32, f32p]
    rel_all, ref_all = [], []
    for si in range(num_scenes):
        blob = scenes.config_scene(config, si)
        nav = bpo.Nav(lib, blob)
        pts = scenes.sample_points(blob, seed + si, goals_per_scene * (1 + agents_per_goal))
        x, r = nav.snap(pts)
        ok = r != 0
        x, r = x[ok], r[ok]
        goals, gref = x[:goals_per_scene], r[:goals_per_scene]
        rest, rref = x[goals_per_scene:], r[goals_per_scene:]
        for g in range(len(goals)):
            a = rest[g * agents_per_goal:(g + 1) * agents_per_goal]
            ar = rref[g * agents_per_goal:(g + 1) * agents_per_goal]
            if not len(a):
                continue
            gs = np.repeat(goals[g:g + 1], len(a), 0)
            gr = np.repeat(gref[g:g + 1], len(a))
            d_ref = nav.geodesic(gs, gr, a, ar)
            d_fld = np.zeros(len(a), np.float32)
            lib.L.bpo_nav_geodesic_field(nav.h, np.ascontiguousarray(gs), np.ascontiguousarray(gr), np.ascontiguousarray(a),
                                         np.ascontiguousarray(ar), len(a), d_fld)
            keep = np.isfinite(d_ref) & (d_ref >= 0.5) & (d_ref <= dmax)
            both = keep & np.isfinite(d_fld)
            rel_all.append(np.abs(d_fld[both].astype(np.float64) - d_ref[both]) / d_ref[both])
            ref_all.append(d_ref[both])
            lost = int((keep & ~np.isfinite(d_fld)).sum())
            if lost:
                rel_all.append(np.full(lost, np.inf))
                ref_all.append(d_ref[keep & ~np.isfinite(d_fld)])
        nav.close()
    return np.concatenate(rel_all), np.concatenate(ref_all)


def summary(name, rel):
    fin = rel[np.isfinite(rel)]
    q = lambda p: float(np.quantile(fin, p))  # noqa: E731
    return (f"{name}: {len(rel)} queries; relative difference median {q(0.5):.2e}, p90 {q(0.9):.2e}, p99 {q(0.99):.2e}, "
            f"max {fin.max():.2e}; identical bits {100 * (rel == 0).mean():.1f} %; above 1e-3: {100 * (rel > 1e-3).mean():.1f} %; "
            f"above 1e-2: {100 * (rel > 1e-2).mean():.1f} %; field corridor over the 256-polygon limit: {int(np.isinf(rel).sum())}")


def main():
    target = int(sys.argv[1]) if len(sys.argv) > 1 else 12000
    lib = bpo.load_oracle()
    lines = []
    for name, config, dmin, dmax in (("C2 (rooms, ~2k polygons)", 2, 1.0, 30.0), ("C4 (corridor maze, ~30k polygons)", 4, 1.0, 40.0)):
        num_scenes, goals = 4, 12
        per_goal = max(8, target // (num_scenes * goals))
        # maze-wide pairs mostly exceed the range (or Detour's node pool): oversample
        rel, ref = measure(lib, config, num_scenes, goals, per_goal * (14 if config == 4 else 1), dmin, dmax, 500 + config)
        lines.append(summary(name, rel))
        print(lines[-1], flush=True)
    return lines


if __name__ == "__main__":
    main()
