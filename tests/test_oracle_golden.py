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


@pytest.mark.parametrize("config", [1, 2, 3, 4])
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


RECAST_FIXTURES = ("recast_room", "recast_two_floors")


def load_recast(name):
    with open(os.path.join(GOLD, name + ".navmesh"), "rb") as f:
        return f.read(), np.load(os.path.join(GOLD, name + ".npz"))


@pytest.mark.parametrize("name", RECAST_FIXTURES)
def test_recast_built_mesh_queries_and_traces(oracle, name):
    """Navmeshes made by the reference's own Recast (irregular polygons, detail meshes with extra
    height samples, islands on obstacles; two floors overlapping in xz joined by a ramp): queries
    and whole simulator traces of the compiled reference, bit for bit."""
    blob, g = load_recast(name)
    nav = bpo.Nav(oracle, blob)
    gd = check_queries(nav, g)
    assert np.isinf(gd).any() and np.isfinite(gd).any()       # box tops / unreachable parts are islands
    if name == "recast_two_floors":
        y = g["snap_xyz"][:, 1]
        assert (y[np.isfinite(y)] < 0.5).any() and (y[np.isfinite(y)] > 2.0).any()   # both floors are hit
    for mode in (0, 1):
        sim = bpo.Sim(oracle, [(blob, g["episodes"])], 24, reset_mode=mode, seed=33, max_steps=50, threads=2)
        sim.reset()
        assert np.array_equal(sim.state()["poly_ref"], g[f"sim{mode}_reset_poly_ref"])
        for t, a in enumerate(g[f"sim{mode}_actions"]):
            sim.step(a)
            o, s = sim.outputs(), sim.state()
            for k in ("rewards", "masks", "infos", "polars"):
                assert np.array_equal(o[k], g[f"sim{mode}_{k}"][t], equal_nan=True), f"{k} differs at step {t} (mode {mode})"
            for k in ("position", "rotation", "poly_ref", "goal_ref", "step", "episode", "num_resets"):
                assert np.array_equal(s[k], g[f"sim{mode}_{k}"][t], equal_nan=True), f"{k} differs at step {t} (mode {mode})"
        assert (g[f"sim{mode}_masks"] == 0).sum() > 0


def test_random_point_in_convex_poly_golden(oracle):
    g = np.load(os.path.join(GOLD, "random_point.npz"))
    for row, (s, t), want in zip(g["polys"], g["st"], g["out"]):
        nv = int(row[0])
        pts = row[1:].reshape(6, 3)[:nv]
        got = oracle.random_point_in_convex_poly(pts, float(s), float(t))
        assert np.array_equal(common.bits(got), common.bits(want))
