"""Shared builders for the tests: scenes of the benchmark configurations at reduced agent
counts, with episode tables measured by the CPU oracle."""
import numpy as np

from bps_nav_amd import episodes, scenes
from oracle import bpo

# config -> (geodesic range of the episodes, forward probability of the action stream)
CONFIGS = {1: (1.0, 10.0, None), 2: (1.0, 30.0, 0.6), 3: (1.0, 30.0, 0.7), 4: (15.0, 40.0, 0.8)}


def oracle_geodesic_fn(nav):
    def f(s, g):
        sx, sr = nav.snap(s)
        gx, gr = nav.snap(g)
        return nav.geodesic(sx, sr, gx, gr)
    return f


def build_scenes(oracle, config, num_scenes, episodes_per_scene=64):
    """[(navmesh bytes, episodes f32[E,10])] for scenes 0..num_scenes-1 of a configuration."""
    dmin, dmax, _ = CONFIGS[config]
    out = []
    for i in range(num_scenes):
        blob = scenes.config_scene(config, i)
        nav = bpo.Nav(oracle, blob)
        eps = episodes.make_episodes(blob, 2000 + i, episodes_per_scene, dmin, dmax, oracle_geodesic_fn(nav))
        nav.close()
        out.append((blob, eps))
    return out


def action_stream(config, steps, n):
    rng = np.random.default_rng(3000 + config)
    return [episodes.random_actions(rng, n, CONFIGS[config][2]) for _ in range(steps)]


def bits(a):
    a = np.ascontiguousarray(a)
    return a.view(np.uint32) if a.dtype == np.float32 else a
