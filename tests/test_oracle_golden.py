"""CPU: the oracle (independent restatement) against the golden vectors written by the
compiled reference (tests/golden/make_golden.py).  Everything is compared bit for bit."""
import glob
import os
import zlib

import numpy as np
import pytest

from bps_nav_amd import scenes
from oracle import bpo
from tests import common
from tests.golden import meshes

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def check_queries(nav, g):
    sx, sr = nav.snap(g["snap_in"])
    assert np.array_equal(sr, g["snap_ref"])
    assert np.array_equal(common.bits(sx), common.bits(g["snap_xyz"]))
    assert (sr[:4] == 0).all() and np.isnan(sx[:4]).all()  # far outside: PathFinder's NaN/0 convention
    tx, tr = nav.try_step(g["step_start"], g["snap_ref"], g["step_end"])
    assert np.array_equal(tr, g["step_ref"])
    assert np.array_equal(common.bits(tx), common.bits(g["step_xyz"]))
    p = g["geo_perm"]
    gd = nav.geodesic(g["step_start"], g["snap_ref"], g["step_start"][p], g["snap_ref"][p])
    assert np.array_equal(common.bits(gd), common.bits(g["geo_dist"]))
    return gd


@pytest.mark.parametrize("name", sorted(meshes.ALL))
def test_handmade_mesh_queries(oracle, name):
    g = np.load(os.path.join(GOLD, f"mesh_{name}.npz"))
    blob = g["blob"].tobytes()
    assert blob == meshes.ALL[name](), "the packer no longer reproduces the fixture's navmesh bytes"
    nav = bpo.Nav(oracle, blob)
    gd = check_queries(nav, g)
    if name == "islands":
        assert np.isinf(gd).any() and np.isfinite(gd).any()


@pytest.mark.parametrize("config", [1, 2, 4])
def test_generated_scene_queries(oracle, config):
    g = np.load(os.path.join(GOLD, f"scene_c{config}.npz"))
    blob = scenes.config_scene(config, 0)
    assert zlib.crc32(blob) == int(g["crc"][0]), "scene generator output changed: regenerate the golden vectors"
    check_queries(bpo.Nav(oracle, blob), g)


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLD, "trace_*.npz"))))
def test_simulator_traces(oracle, path):
    g = np.load(path)
    base = os.path.basename(path)
    config, mode = int(base[7]), int(base[-5])
    eps = g["episodes"]
    sc = [(scenes.config_scene(config, i), eps[i]) for i in range(len(eps))]
    n = g["actions"].shape[1]
    max_steps = {"trace_c1_mode0.npz": 40}.get(base, 60)
    sim = bpo.Sim(oracle, sc, n, reset_mode=mode, seed=21, max_steps=max_steps, threads=3)
    sim.reset()
    st = sim.state()
    assert np.array_equal(st["poly_ref"], g["reset_poly_ref"])
    assert np.array_equal(common.bits(st["position"]), common.bits(g["reset_position"]))
    for t, a in enumerate(g["actions"]):
        sim.step(a)
        o, s = sim.outputs(), sim.state()
        for k in ("rewards", "masks", "infos", "polars"):
            assert np.array_equal(o[k], g[k][t], equal_nan=True), f"{k} differs at step {t}"
        for k in ("position", "rotation", "poly_ref", "goal_ref", "step", "episode", "num_resets"):
            assert np.array_equal(s[k], g[k][t], equal_nan=True), f"{k} differs at step {t}"
    assert (g["masks"] == 0).sum() > 0


def test_random_point_in_convex_poly_golden(oracle):
    g = np.load(os.path.join(GOLD, "random_point.npz"))
    for row, (s, t), want in zip(g["polys"], g["st"], g["out"]):
        nv = int(row[0])
        pts = row[1:].reshape(6, 3)[:nv]
        got = oracle.random_point_in_convex_poly(pts, float(s), float(t))
        assert np.array_equal(common.bits(got), common.bits(want))
