"""GPU parity: the HIP engine, called through the C ABI, against the CPU oracle on the same
seeded scenes, episodes and action streams.

Bars (BASELINE.json): polygon ids, dones and resets bit-exact; positions within 1e-4 m,
headings within 1e-4 rad; geodesic distance and reward within 1e-3 relative.  The kernels
keep the reference's fp32 operation order, so everything except the polar angle (device
atan2f vs glibc atan2f) is in fact compared bit for bit here.
"""
import numpy as np
import pytest

from tests import common

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch_cuda():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch


def make_gen(sc, n, num_active_scenes=None, **kw):
    from bps_nav_amd.bps_sim import PointNavRolloutGenerator
    return PointNavRolloutGenerator("", "", n, num_active_scenes or len(sc), scenes=sc, **kw)


@pytest.mark.parametrize("config", [1, 2, 3, 4])
def test_batched_queries_match_oracle(oracle, torch_cuda, config):
    from bps_nav_amd import scenes
    from oracle import bpo
    print(f"case: batched queries config {config}", flush=True)
    blob = scenes.config_scene(config, 0)
    nav = bpo.Nav(oracle, blob)
    gen = make_gen([(blob, np.zeros((1, 10), np.float32))], 1)
    rng = np.random.default_rng(config)
    pts = scenes.sample_points(blob, 7, 3000)
    q = pts + rng.normal(0, 0.3, pts.shape).astype(np.float32)
    q[:, 1] += rng.uniform(-1, 2, len(q)).astype(np.float32)
    q[:5] += 100.0  # far outside the mesh: snap fails
    xo, ro = nav.snap(q)
    xg, rg = gen.snap_points(0, q)
    assert np.array_equal(ro, rg)
    assert np.array_equal(common.bits(xo), common.bits(xg))
    assert (ro[:5] == 0).all() and np.isnan(xg[:5]).all()
    ok = ro != 0
    ang = rng.uniform(0, 2 * np.pi, len(q))
    d = rng.uniform(0, 0.6, len(q))
    end = xo.copy()
    end[:, 0] += (d * np.cos(ang)).astype(np.float32)
    end[:, 2] += (d * np.sin(ang)).astype(np.float32)
    so, sro = nav.try_step(xo[ok], ro[ok], end[ok])
    sg, srg = gen.try_steps(0, xo[ok], ro[ok], end[ok])
    assert np.array_equal(sro, srg)
    assert np.array_equal(common.bits(so), common.bits(sg))
    m = min(1000, ok.sum() // 2)
    a, ar, b, br = xo[ok][:m], ro[ok][:m], xo[ok][m:2 * m], ro[ok][m:2 * m]
    go = nav.geodesic(a, ar, b, br)
    gg = gen.geodesic(0, a, ar, b, br)
    assert np.array_equal(common.bits(go), common.bits(gg)), \
        f"{(common.bits(go) != common.bits(gg)).sum()} of {m} geodesics differ"
    if config == 4:  # maze-wide pairs: searches that outgrow the node links kept in LDS
        assert gen.counters()["geo_link_spills"] > 20
    if config >= 3:  # equal totals at the front of the open list: taken as a pair, or settled from the operation log
        assert gen.counters()["geo_pair_ties"] > 5 and gen.counters()["geo_tie_replays"] > 0
    # invalid refs and coincident points
    gz = gen.geodesic(0, a[:4], ar[:4], a[:4], ar[:4])
    assert (gz == 0).all()
    gi = gen.geodesic(0, a[:4], np.zeros(4, np.uint32), b[:4], br[:4])
    assert np.isinf(gi).all()
    # the vectors the compiled reference wrote for this scene (tests/golden/make_golden.py)
    import os
    import zlib
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", f"scene_c{config}.npz"))
    assert zlib.crc32(blob) == int(g["crc"][0])
    sx, sr = gen.snap_points(0, g["snap_in"])
    assert np.array_equal(sr, g["snap_ref"]) and np.array_equal(common.bits(sx), common.bits(g["snap_xyz"]))
    tx, tr = gen.try_steps(0, g["step_start"], g["snap_ref"], g["step_end"])
    assert np.array_equal(tr, g["step_ref"]) and np.array_equal(common.bits(tx), common.bits(g["step_xyz"]))
    p = g["geo_perm"]
    gd = gen.geodesic(0, g["step_start"], g["snap_ref"], g["step_start"][p], g["snap_ref"][p])
    assert np.array_equal(common.bits(gd), common.bits(g["geo_dist"])), "geodesics differ from the compiled reference's"
    gen.close()


@pytest.mark.parametrize("config,seed", [(1, 101), (2, 100), (2, 103), (3, 100), (4, 101), (4, 104)])
def test_geodesics_on_further_scenes_match_oracle(oracle, torch_cuda, config, seed):
    """Scene-wide point pairs on generated scenes that no other test uses: the searches meet other
    junctions, equal totals and pool sizes than those of the scenes above."""
    from bps_nav_amd import scenes
    from bps_nav_amd.bps_sim import nav_only
    from oracle import bpo
    print(f"case: geodesics on config {config} scene {seed}", flush=True)
    blob = scenes.config_scene(config, seed)
    nav = bpo.Nav(oracle, blob)
    gen = nav_only([blob])
    pts = scenes.sample_points(blob, 1000 + seed, 3000)
    x, r = nav.snap(pts)
    ok = r != 0
    x, r = x[ok], r[ok]
    m = len(x) // 2
    go = nav.geodesic(x[:m], r[:m], x[m:2 * m], r[m:2 * m])
    gg = gen.geodesic(0, x[:m], r[:m], x[m:2 * m], r[m:2 * m])
    nav.close()
    assert m > 1000 and np.isfinite(go).sum() > 100   # (maze-wide pairs mostly exceed the 256-polygon path limit: +inf on both sides)
    assert np.array_equal(common.bits(go), common.bits(gg)), \
        f"{(common.bits(go) != common.bits(gg)).sum()} of {m} geodesics differ"
    gen.close()


@pytest.mark.parametrize("name", ["recast_room", "recast_two_floors"])
def test_recast_built_meshes_match_reference_vectors(oracle, torch_cuda, name):
    """Navmeshes built by the reference's own Recast (committed fixtures): the engine against the
    vectors and simulator traces that the compiled reference wrote for them, and against the
    oracle on fresh random queries."""
    import os
    from bps_nav_amd import scenes
    from oracle import bpo
    print(f"case: recast-built fixture {name}", flush=True)
    gold = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    with open(os.path.join(gold, name + ".navmesh"), "rb") as f:
        blob = f.read()
    g = np.load(os.path.join(gold, name + ".npz"))
    gen = make_gen([(blob, g["episodes"])], 24, seed=33, max_steps=50)
    sx, sr = gen.snap_points(0, g["snap_in"])
    assert np.array_equal(sr, g["snap_ref"]) and np.array_equal(common.bits(sx), common.bits(g["snap_xyz"]))
    tx, tr = gen.try_steps(0, g["step_start"], g["snap_ref"], g["step_end"])
    assert np.array_equal(tr, g["step_ref"]) and np.array_equal(common.bits(tx), common.bits(g["step_xyz"]))
    p = g["geo_perm"]
    gd = gen.geodesic(0, g["step_start"], g["snap_ref"], g["step_start"][p], g["snap_ref"][p])
    assert np.array_equal(common.bits(gd), common.bits(g["geo_dist"]))
    # fresh queries against the oracle
    nav = bpo.Nav(oracle, blob)
    rng = np.random.default_rng(9)
    pts = scenes.sample_points(blob, 13, 1500)
    q = pts + rng.normal(0, 0.3, pts.shape).astype(np.float32)
    q[:, 1] += rng.uniform(-1, 2, len(q)).astype(np.float32)
    xo, ro = nav.snap(q)
    xg, rg = gen.snap_points(0, q)
    assert np.array_equal(ro, rg) and np.array_equal(common.bits(xo), common.bits(xg))
    gen.close()
    for mode in (0, 1):
        gen = make_gen([(blob, g["episodes"])], 24, seed=33, max_steps=50, reset_mode=mode)
        gen.reset(0)
        state, infos = gen.get_state(0), gen.get_infos(0)
        assert np.array_equal(state["poly_ref"].cpu().numpy().view(np.uint32), g[f"sim{mode}_reset_poly_ref"])
        for t, a in enumerate(g[f"sim{mode}_actions"]):
            gen.step(0, a)
            st = {k: v.cpu().numpy() for k, v in state.items()}
            for k in ("poly_ref", "goal_ref", "step", "episode", "num_resets"):
                assert np.array_equal(st[k].view(np.uint32), g[f"sim{mode}_{k}"][t]), f"{k} at step {t} mode {mode}"
            assert np.array_equal(common.bits(st["position"]), common.bits(g[f"sim{mode}_position"][t]))
            assert np.array_equal(gen.get_masks(0).cpu().numpy(), g[f"sim{mode}_masks"][t])
            gi = infos.packed.cpu().numpy()
            assert ((common.bits(gi) == common.bits(g[f"sim{mode}_infos"][t])) | np.isnan(gi)).all(), f"infos at step {t}"
            np.testing.assert_allclose(gi, g[f"sim{mode}_infos"][t], rtol=1e-3, equal_nan=True)
            np.testing.assert_allclose(gen.get_rewards(0).cpu().numpy(), g[f"sim{mode}_rewards"][t], rtol=1e-3, atol=1e-6,
                                       equal_nan=True)
            gp, cp = gen.get_polars(0).cpu().numpy(), g[f"sim{mode}_polars"][t]
            np.testing.assert_allclose(gp[:, 0], cp[:, 0], rtol=1e-6, atol=1e-6)
            dphi = np.abs(gp[:, 1] - cp[:, 1])
            assert (np.minimum(dphi, 2 * np.pi - dphi) < 1e-4).all()
        gen.check_errors()
        gen.close()


def test_open_hall_queries_match_oracle(oracle, torch_cuda):
    """A hall without obstacles: A* spreads over a wide front, so the open list outgrows the
    kernel's register heap, the node links outgrow LDS and long queries exhaust Detour's
    2048-node pool.  Every continuation path of the kernel must still equal the oracle."""
    from bps_nav_amd import scenes
    from oracle import bpo
    print("case: open hall (spill paths of the A* kernel)", flush=True)
    blob = scenes.gen_scene(scenes.BOX_ROOM, 4242, cell=5, size_x=30.0, size_z=30.0, num_boxes=0, tri_frac=0.2,
                            hex_frac=0.1)
    nav = bpo.Nav(oracle, blob)
    gen = make_gen([(blob, np.zeros((1, 10), np.float32))], 1)
    pts = scenes.sample_points(blob, 9, 1600)
    x, r = nav.snap(pts)
    assert (r != 0).all()
    m = len(x) // 2
    a, ar, b, br = x[:m], r[:m], x[m:], r[m:]
    # mix of ranges: short hops, mid-range (large open list, path found) and far (pool exhausted)
    k = m // 2
    b[:k] = a[:k] + (b[:k] - a[:k]) * np.linspace(0.02, 0.5, k, dtype=np.float32)[:, None]
    b, br = nav.snap(b)
    c0 = gen.counters()
    go = nav.geodesic(a, ar, b, br)
    gg = gen.geodesic(0, a, ar, b, br)
    c1 = gen.counters()
    assert np.array_equal(common.bits(go), common.bits(gg)), \
        f"{(common.bits(go) != common.bits(gg)).sum()} of {m} geodesics differ"
    assert np.isinf(go).any() and np.isfinite(go).sum() > m // 3
    # open lists beyond the sorted form's registers run again with the exact heap, which in turn
    # leaves its registers; ties between equal totals occur on the way
    assert c1["geo_exact_runs"] - c0["geo_exact_runs"] > 10, "exact re-run path not exercised"
    assert c1["geo_heap_spills"] - c0["geo_heap_spills"] > 10, "heap spill path not exercised"
    assert c1["geo_pair_ties"] - c0["geo_pair_ties"] > 50 and c1["geo_tie_replays"] - c0["geo_tie_replays"] > 0, \
        "tie paths not exercised"
    gen.close()


@pytest.mark.parametrize("config,num_scenes,n,steps,mode", [
    (1, 1, 64, 500, 0), (2, 4, 256, 300, 0), (3, 2, 128, 200, 1), (4, 4, 256, 200, 0), (2, 4, 256, 150, 1)])
def test_step_parity(oracle, torch_cuda, config, num_scenes, n, steps, mode):
    from oracle import bpo
    print(f"case: step parity config {config} scenes {num_scenes} agents {n} mode {mode}", flush=True)
    sc = common.build_scenes(oracle, config, num_scenes)
    cpu = bpo.Sim(oracle, sc, n, reset_mode=mode, seed=11, threads=4)
    gen = make_gen(sc, n, reset_mode=mode, seed=11)
    cpu.reset()
    gen.reset(0)
    views = dict(rewards=gen.get_rewards(0), masks=gen.get_masks(0), polars=gen.get_polars(0))
    infos = gen.get_infos(0)
    state = gen.get_state(0)
    acts = common.action_stream(config, steps, n)
    dones = 0
    for t, a in enumerate(acts):
        cpu.step(a)
        gen.step(0, torch_cuda.from_numpy(a).cuda() if t % 2 else a)  # device and host action paths
        co, cs = cpu.outputs(), cpu.state()
        g_state = {k: v.cpu().numpy() for k, v in state.items()}
        for k in ("poly_ref", "goal_ref", "step", "episode", "num_resets"):
            assert np.array_equal(cs[k], g_state[k].view(np.uint32)), f"{k} differs at step {t}"
        assert np.array_equal(co["masks"], views["masks"].cpu().numpy()), f"dones differ at step {t}"
        np.testing.assert_allclose(g_state["position"], cs["position"], atol=1e-4, rtol=0)
        np.testing.assert_allclose(g_state["rotation"], cs["rotation"], atol=1e-6, rtol=0)
        assert np.array_equal(common.bits(g_state["position"]), common.bits(cs["position"])), f"position bits at step {t}"
        gi = infos.packed.cpu().numpy()
        gr = views["rewards"].cpu().numpy()
        np.testing.assert_allclose(gi, co["infos"], rtol=1e-3, atol=0, equal_nan=True)
        np.testing.assert_allclose(gr, co["rewards"], rtol=1e-3, atol=1e-6, equal_nan=True)
        assert ((common.bits(gi) == common.bits(co["infos"])) | np.isnan(gi)).all(), f"info bits at step {t}"
        gp = views["polars"].cpu().numpy()
        np.testing.assert_allclose(gp[:, 0], co["polars"][:, 0], rtol=1e-6, atol=1e-6)
        dphi = np.abs(gp[:, 1] - co["polars"][:, 1])
        dphi = np.minimum(dphi, 2 * np.pi - dphi)
        assert (dphi < 1e-4).all(), f"polar angle differs by {dphi.max()} rad at step {t}"
        dones += int((co["masks"] == 0).sum())
    assert dones > 0, "the stream never finished an episode: resets were not exercised"
    gen.check_errors()
    gen.close()


@pytest.mark.parametrize("task,config,num_scenes,n,steps,mode,max_steps", [
    (1, 2, 4, 256, 250, 0, 60), (1, 4, 2, 128, 120, 1, 0), (2, 3, 2, 128, 250, 0, 80), (2, 1, 1, 64, 150, 1, 0)])
def test_flee_and_exploration_step_parity(oracle, torch_cuda, task, config, num_scenes, n, steps, mode, max_steps):
    """The other two tasks of the reference (simulator.cpp:830-997) against the oracle: same
    dynamics, info = distance from start (Flee) or visited-cell count (Exploration)."""
    from bps_nav_amd import bps_sim
    from oracle import bpo
    print(f"case: task {task} config {config} scenes {num_scenes} agents {n} mode {mode}", flush=True)
    sc = common.build_scenes(oracle, config, num_scenes)
    cpu = bpo.Sim(oracle, sc, n, reset_mode=mode, seed=23, threads=4, task=task, max_steps=max_steps)
    cls = bps_sim.FleeRolloutGenerator if task == 1 else bps_sim.ExplorationRolloutGenerator
    gen = cls("", "", n, len(sc), scenes=sc, reset_mode=mode, seed=23, max_steps=max_steps)
    cpu.reset()
    gen.reset(0)
    infos = gen.get_infos(0)
    assert infos.dtype.names == (("distanceFromStart",) if task == 1 else ("numVisited",))
    assert infos.packed.shape == (n, 1)
    rewards, masks, state = gen.get_rewards(0), gen.get_masks(0), gen.get_state(0)
    dones = 0
    nonzero = 0
    for t, a in enumerate(common.action_stream(config, steps, n)):
        cpu.step(a)
        gen.step(0, a)
        co, cs = cpu.outputs(), cpu.state()
        g_state = {k: v.cpu().numpy() for k, v in state.items()}
        for k in ("poly_ref", "goal_ref", "step", "episode", "num_resets"):
            assert np.array_equal(cs[k], g_state[k].view(np.uint32)), f"{k} differs at step {t}"
        assert np.array_equal(common.bits(g_state["position"]), common.bits(cs["position"])), f"position bits at step {t}"
        assert np.array_equal(co["masks"], masks.cpu().numpy()), f"dones differ at step {t}"
        gi = infos.packed.cpu().numpy()[:, 0]
        gr = rewards.cpu().numpy()
        np.testing.assert_allclose(gi, co["infos"][:, 0], rtol=1e-3, atol=0, equal_nan=True)
        np.testing.assert_allclose(gr, co["rewards"], rtol=1e-3, atol=1e-6, equal_nan=True)
        assert np.array_equal(common.bits(gi), common.bits(co["infos"][:, 0])), f"info bits at step {t}"
        dones += int((co["masks"] == 0).sum())
        nonzero += int((gr != 0).sum())
    assert dones > 0 and nonzero > 0
    gen.check_errors()
    gen.close()


def assert_step_equal(cpu, gen, group, state, infos, where):
    """Everything the reference's step shows of a group after one step, engine against oracle:
    ids, counters and position bit for bit, masks, and infos and rewards bit for bit wherever
    the value is a number (inf - inf gives a NaN whose payload differs between the two)."""
    co, cs = cpu.outputs(group), cpu.state(group)
    st = {k: v.cpu().numpy() for k, v in state.items()}
    for k in ("poly_ref", "goal_ref", "step", "episode", "num_resets"):
        assert np.array_equal(cs[k], st[k].view(np.uint32)), f"{k} differs {where}"
    assert np.array_equal(common.bits(st["position"]), common.bits(cs["position"])), f"position differs {where}"
    assert np.array_equal(common.bits(st["rotation"]), common.bits(cs["rotation"])), f"rotation differs {where}"
    assert np.array_equal(co["masks"], gen.get_masks(group).cpu().numpy()), f"dones differ {where}"
    gi = infos.packed.cpu().numpy()
    ci = co["infos"][:, :gi.shape[1]]
    assert ((common.bits(gi) == common.bits(ci)) | (np.isnan(gi) & np.isnan(ci))).all(), f"infos differ {where}"
    gr = gen.get_rewards(group).cpu().numpy()
    assert ((common.bits(gr) == common.bits(co["rewards"])) | (np.isnan(gr) & np.isnan(co["rewards"]))).all(), \
        f"rewards differ {where}"
    gp = gen.get_polars(group).cpu().numpy()
    np.testing.assert_allclose(gp[:, 0], co["polars"][:, 0], rtol=1e-6, atol=1e-6)
    dphi = np.abs(gp[:, 1] - co["polars"][:, 1])
    assert (np.minimum(dphi, 2 * np.pi - dphi) < 1e-4).all(), f"polar angle differs {where}"
    return co, cs


@pytest.mark.parametrize("config,num_scenes,n,steps,mode", [(2, 16, 1024, 1000, 0), (3, 64, 4096, 300, 1)])
def test_step_parity_at_configured_sizes(oracle, torch_cuda, config, num_scenes, n, steps, mode):
    """The second and third benchmark configurations at their own agent and scene counts (the
    third with its area-weighted sampled resets), stepped side by side with the oracle on all
    host cores and compared in full after every step."""
    import os
    from oracle import bpo
    print(f"case: configured size, config {config}: {n} agents / {num_scenes} scenes, {steps} steps", flush=True)
    sc = common.build_scenes(oracle, config, num_scenes, episodes_per_scene=32)
    threads = min(16, len(os.sched_getaffinity(0)))
    cpu = bpo.Sim(oracle, sc, n, reset_mode=mode, seed=101, threads=threads)
    gen = make_gen(sc, n, reset_mode=mode, seed=101)
    cpu.reset()
    gen.reset(0)
    state, infos = gen.get_state(0), gen.get_infos(0)
    for t, a in enumerate(common.action_stream(config, steps, n)):
        cpu.step(a)
        gen.step(0, a)
        co, cs = assert_step_equal(cpu, gen, 0, state, infos, f"at step {t}")
    assert int(cs["num_resets"].sum()) > n
    gen.check_errors()
    gen.close()


def largest_single_tile_maze(seed):
    """A corridor maze close to what one Detour tile holds (32767 polygons): the widest lattice
    whose polygon count still fits (the count varies with the seed's corridor widths)."""
    from bps_nav_amd import scenes
    for w in (54, 53, 52, 51, 50):
        try:
            return scenes.gen_scene(scenes.MAZE, seed, cell=10, maze_w=w, maze_h=w, corridor_min=1.0, corridor_max=1.5,
                                    wall=1.0, braid=0.08, tri_frac=0.05, hex_frac=0.05)
        except RuntimeError as e:
            if "more than 32767 polygons" not in str(e):
                raise
    raise RuntimeError("no lattice size fits one tile")


def test_mixed_scenes_at_the_largest_configured_shape(oracle, torch_cuda):
    """The fifth benchmark configuration's shape: 65536 agents over 256 scenes of mixed kinds and
    sizes in one simulator (room plans of ~2k polygons, cluttered plans of ~20k, mazes of ~30k, mazes at
    the largest size one Detour tile holds, and the Recast-built two-floor mesh with its ramp),
    stepped next to the oracle and compared in full after every step.  Scenes above 32767 polygons
    need several tiles, which the reference's PathFinder cannot address: they are not run."""
    import os
    import struct
    from bps_nav_amd import episodes, scenes
    from bps_nav_amd.bps_sim import nav_only
    from oracle import bpo
    print("case: 65536 agents / 256 mixed scenes", flush=True)
    gold = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    with open(os.path.join(gold, "recast_two_floors.navmesh"), "rb") as f:
        two_floors = f.read()
    blobs, ranges = [], []
    biggest = 0
    for i in range(256):
        kind = i % 8
        if kind < 3:
            blobs.append(scenes.config_scene(2, i)); ranges.append((1.0, 30.0))
        elif kind < 5:
            blobs.append(scenes.config_scene(3, i)); ranges.append((1.0, 30.0))
        elif kind == 5:
            blobs.append(largest_single_tile_maze(1000 + i)); ranges.append((5.0, 30.0))
        elif kind == 6:
            blobs.append(scenes.config_scene(4, i)); ranges.append((5.0, 30.0))
        else:
            blobs.append(two_floors); ranges.append((1.0, 30.0))
        biggest = max(biggest, struct.unpack_from("<i", blobs[-1], 48 + 24)[0])
    assert 31000 < biggest <= 32767, f"largest scene has {biggest} polygons"
    nav = nav_only(blobs)

    def gfn(i):
        def f(s, g):
            sx, sr = nav.snap_points(i, s)
            gx, gr = nav.snap_points(i, g)
            return nav.geodesic(i, sx, sr, gx, gr)
        return f
    sc = [(b, episodes.make_episodes(b, 2000 + i, 32, ranges[i][0], ranges[i][1], gfn(i))) for i, b in enumerate(blobs)]
    nav.close()
    n, steps = 65536, 60
    threads = min(16, len(os.sched_getaffinity(0)))
    cpu = bpo.Sim(oracle, sc, n, seed=55, threads=threads)
    gen = make_gen(sc, n, seed=55)
    cpu.reset()
    gen.reset(0)
    state, infos = gen.get_state(0), gen.get_infos(0)
    rng = np.random.default_rng(8)
    for t in range(steps):
        a = episodes.random_actions(rng, n, 0.7)
        cpu.step(a)
        gen.step(0, a)
        co, cs = assert_step_equal(cpu, gen, 0, state, infos, f"at step {t}")
        if t % 10 == 0:
            print(f"  step {t} equal", flush=True)
    assert int(cs["num_resets"].sum()) > n
    assert (cs["position"][:, 1] > 2.0).any(), "nobody on the upper floor of the two-floor scenes"
    gen.check_errors()
    gen.close()


def test_full_size_workload_properties(oracle, torch_cuda):
    """The benchmark's own shape (16384 agents, 128 maze scenes of ~30k polygons), with the oracle
    stepped along on all host cores and compared in full after every step, plus
    size-independent properties:
      - rewards obey the reference's algebra given the infos (simulator.cpp:800-825);
      - every finite distance is at least the straight line between its two navmesh points;
      - a sample of agents' distances equals the oracle's geodesic for the same two points;
      - a second simulator with the same seed produces bit-identical outputs."""
    import os
    import torch
    from bps_nav_amd import episodes, scenes
    from bps_nav_amd.bps_sim import PointNavRolloutGenerator, nav_only
    from oracle import bpo
    print("case: full-size workload properties", flush=True)
    N, S, steps = 16384, 128, 40
    blobs = [scenes.config_scene(4, i) for i in range(S)]
    nav = nav_only(blobs)

    def gfn(i):
        def f(s, g):
            sx, sr = nav.snap_points(i, s)
            gx, gr = nav.snap_points(i, g)
            return nav.geodesic(i, sx, sr, gx, gr)
        return f
    sc = [(b, episodes.make_episodes(b, 2000 + i, 128, 15.0, 40.0, gfn(i))) for i, b in enumerate(blobs)]
    nav.close()
    rng = np.random.default_rng(5)
    acts = [episodes.random_actions(rng, N, 0.8) for _ in range(steps)]
    runs = []
    for rep in range(2):
        gen = PointNavRolloutGenerator("", "", N, S, scenes=sc, seed=77)
        gen.reset(0)
        state, infos = gen.get_state(0), gen.get_infos(0)
        if rep == 0:
            cpu = bpo.Sim(oracle, sc, N, seed=77, threads=min(16, len(os.sched_getaffinity(0))))
            cpu.reset()
        prev = torch.full((N,), float("nan"), device="cuda")   # reset writes no outputs: unknown until step 1
        for t, a in enumerate(acts):
            gen.step(0, torch.from_numpy(a).cuda())
            if rep == 0:
                cpu.step(a)
                assert_step_equal(cpu, gen, 0, state, infos, f"at step {t}")
            info = infos.packed
            rew, mask = gen.get_rewards(0), gen.get_masks(0)
            d, succ, spl = info[:, 2], info[:, 0], info[:, 1]
            done = mask == 0
            expect = torch.where(done, -0.01 + 2.5 * spl, -0.01 + (prev - d))
            ok = torch.isfinite(expect)
            assert torch.allclose(rew[ok], expect[ok], rtol=1e-5, atol=1e-6), f"reward algebra at step {t}"
            assert bool(((succ == 0) | (d < 0.2)).all())
            # after an auto-reset the next step measures against the new episode's first distance,
            # which the outputs do not show: carry on only for agents that did not finish
            prev = torch.where(done, torch.full_like(d, float("nan")), d)
        st = {k: v.cpu().numpy() for k, v in state.items()}
        out = dict(info=infos.packed.cpu().numpy(), rew=gen.get_rewards(0).cpu().numpy(),
                   polar=gen.get_polars(0).cpu().numpy(), pos=st["position"], ref=st["poly_ref"],
                   mask=gen.get_masks(0).cpu().numpy(), goal=st["goal"])
        runs.append(out)
        if rep == 0:
            cpu.close()
            cnt = gen.counters()
            assert cnt["agent_steps"] == N * steps and cnt["geodesic_queries"] > N
        gen.check_errors()
        gen.close()
    for k in runs[0]:
        assert np.array_equal(common.bits(runs[0][k]), common.bits(runs[1][k])), f"{k} not reproducible"
    # oracle spot check on 4 scenes x 24 agents: distance shown for the agent's current point
    r = runs[0]
    per = N // S
    for sidx in (0, 37, 90, 127):
        onav = bpo.Nav(oracle, blobs[sidx])
        ids = np.arange(sidx * per, sidx * per + 24)
        pos = r["pos"][ids]
        x, ref = onav.snap(pos)
        assert np.array_equal(ref, r["ref"][ids].view(np.uint32)), "agents stand where the oracle snaps them"
        # agents that just moved forward and go on: the distance shown is geodesic(goal point -> agent point)
        fresh = (acts[-1][ids] == 1) & (r["mask"][ids] == 1)
        gx, gref = onav.snap(r["goal"][ids])
        want = onav.geodesic(gx[fresh], gref[fresh], pos[fresh], ref[fresh])
        assert fresh.sum() > 8
        assert np.array_equal(common.bits(want), common.bits(r["info"][ids][fresh, 2])), "distance differs from the oracle's"
        onav.close()
    # straight-line bound, all agents: geodesic(goal point -> agent) >= |goal - agent| (3-D), using rho of the polar
    d = r["info"][:, 2]
    assert np.isfinite(d).mean() > 0.99
    fin = np.isfinite(d) & (r["mask"] == 1)   # a finished agent's polar already shows its next episode
    assert (d[fin] >= r["polar"][fin, 0] * 0.98 - 0.5).all(), "a path shorter than the straight line"



def test_two_group_stepping_parity(oracle, torch_cuda):
    """double_buffered=True (simulator.cpp:1503-1508, 1404-1410): two groups of N/2 envs, each
    on its own half of the scenes, stepped alternately with their own action streams; every
    step of either group is compared in full with the oracle's same group, and the other
    group's outputs must not move."""
    from oracle import bpo
    print("case: two groups (double_buffered)", flush=True)
    sc = common.build_scenes(oracle, 2, 4, episodes_per_scene=32)
    n = 256
    cpu = bpo.Sim(oracle, sc, n, double_buffered=True, seed=19, threads=4, max_steps=50)
    gen = make_gen(sc, n, double_buffered=True, seed=19, max_steps=50)
    assert gen.num_groups == 2 and gen.envs_per_group == n // 2 and cpu.n == n // 2
    state = [gen.get_state(g) for g in (0, 1)]
    infos = [gen.get_infos(g) for g in (0, 1)]
    assert state[0]["position"].data_ptr() != state[1]["position"].data_ptr()
    for g in (0, 1):
        cpu.reset(g)
        gen.reset(g)
    rng = np.random.default_rng(41)
    from bps_nav_amd import episodes
    resets = [0, 0]
    for t in range(240):
        # mostly alternating, sometimes the same group twice in a row
        g = t % 2 if t % 7 else (t // 7) % 2
        other = 1 - g
        before = {k: v.clone() for k, v in state[other].items()}
        rew_before = gen.get_rewards(other).clone()
        a = episodes.random_actions(rng, n // 2, 0.6)
        cpu.step(a, g)
        if t % 3 == 0:
            gen.step_start(g, torch_cuda.from_numpy(a).cuda())
            with pytest.raises(RuntimeError, match="previous step not finished"):
                gen.step_start(other, a)      # one outstanding step, whichever the group
            with pytest.raises(RuntimeError, match="no step in flight"):
                gen.step_end(other)
            gen.step_end(g)
        else:
            gen.step(g, a)
        co, cs = assert_step_equal(cpu, gen, g, state[g], infos[g], f"group {g} at step {t}")
        resets[g] = int(cs["num_resets"].sum())
        for k, v in before.items():
            assert torch_cuda.equal(v, state[other][k]), f"group {other}'s {k} moved during group {g}'s step"
        assert torch_cuda.equal(rew_before, gen.get_rewards(other))
    assert resets[0] > n and resets[1] > n
    gen.check_errors()
    gen.close()


def test_random_points_match_oracle(oracle, torch_cuda):
    """bpsx_random_points (PathFinder::getRandomNavigablePoint's distribution with the build's
    prefix-sum rule) against the oracle's sampler on the same variates, bit for bit, on a
    generated plan and on the Recast-built two-floor mesh; polygon refs must be those of
    walkable polygons that hold the point."""
    import os
    from bps_nav_amd import scenes
    from oracle import bpo
    print("case: random points", flush=True)
    gold = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    with open(os.path.join(gold, "recast_two_floors.navmesh"), "rb") as f:
        two_floors = f.read()
    blobs = [scenes.config_scene(3, 1), two_floors, scenes.config_scene(4, 2)]
    gen = make_gen([(b, np.zeros((1, 10), np.float32)) for b in blobs], 3)
    rng = np.random.default_rng(12)
    for i, blob in enumerate(blobs):
        nav = bpo.Nav(oracle, blob)
        u = rng.uniform(0, 1, (5000, 3)).astype(np.float32)
        u[:3] = [[0, 0, 0], [0.99999994, 0.99999994, 0.99999994], [0.5, 0, 0.99999994]]
        want = nav.sample(u)
        xyz, ref = gen.random_points(i, u)
        assert np.array_equal(common.bits(want), common.bits(xyz)), f"scene {i}: sampled points differ"
        refs, flags, _ = nav.poly_info()
        walkable = set(int(r) for r, f in zip(refs, flags) if (f & 1) and not (f & 4))
        assert all(int(r) in walkable for r in ref), f"scene {i}: a ref that is no walkable polygon"
        # the point lies on its polygon: snapping it finds that polygon again (points on a shared
        # edge may go to the neighbour)
        sx, sr = nav.snap(xyz)
        assert (sr == ref).mean() > 0.95, f"scene {i}: refs do not name the polygons that hold the points"
        nav.close()
    assert len(gen.random_points(0, np.zeros((0, 3), np.float32))[0]) == 0
    gen.close()


def test_scene_rotation_parity(oracle, torch_cuda):
    """Scenes are swapped in while the simulation runs (SceneSwapper, simulator.cpp:1063-1154):
    envs move to the new scene when their episode ends.  Same swaps at the same steps on the
    oracle; everything must stay equal, through several generations per slot, with scenes of
    different sizes (the engine re-uses the space of scenes that left)."""
    from oracle import bpo
    print("case: scene rotation", flush=True)
    pool = common.build_scenes(oracle, 2, 6, episodes_per_scene=24) + common.build_scenes(oracle, 1, 2, episodes_per_scene=24)
    n, S = 96, 3
    cpu = bpo.Sim(oracle, pool[:S], n, seed=5, threads=3, max_steps=40)
    gen = make_gen(pool[:S], n, seed=5, max_steps=40, scene_reserve=4.0)
    cpu.reset()
    gen.reset(0)
    state, infos = gen.get_state(0), gen.get_infos(0)
    nxt = S
    swaps = 0
    for t, a in enumerate(common.action_stream(2, 420, n)):
        if t % 25 == 10:
            for slot in range(S):
                rem, _ = gen.swap_status(slot)
                assert rem == cpu.swap_remaining(slot)
                if rem == 0:
                    blob, eps = pool[nxt % len(pool)]
                    nxt += 1
                    cpu.swap_scene(slot, blob, eps)
                    gen.swap_scene(slot, blob, eps)
                    swaps += 1
                else:
                    with pytest.raises(RuntimeError, match="still in progress"):
                        gen.swap_scene(slot, *pool[0])
        cpu.step(a)
        gen.step(0, a)
        co, cs = cpu.outputs(), cpu.state()
        st = {k: v.cpu().numpy() for k, v in state.items()}
        for k in ("poly_ref", "goal_ref", "step", "episode", "num_resets"):
            assert np.array_equal(cs[k], st[k].view(np.uint32)), f"{k} differs at step {t}"
        assert np.array_equal(common.bits(st["position"]), common.bits(cs["position"])), f"position at step {t}"
        assert np.array_equal(co["masks"], gen.get_masks(0).cpu().numpy())
        gi = infos.packed.cpu().numpy()
        assert ((common.bits(gi) == common.bits(co["infos"])) | np.isnan(gi)).all(), f"infos at step {t}"
    assert swaps >= 12
    assert gen.swap_status(0)[1] >= 6, "swaps did not complete"
    assert gen.swap_stats[0] > 0
    gen.check_errors()
    gen.close()


def write_dataset(root, pool):
    """A dataset directory in the reference's layout (simulator.cpp:190-336, env_utils.py:40-48):
    <root>/content/<scene>.json.gz with that scene's episodes, navmeshes under <root>/assets."""
    import gzip
    import json
    import os
    os.makedirs(os.path.join(root, "content"))
    os.makedirs(os.path.join(root, "assets", "plans"))
    for i, (blob, eps) in enumerate(pool):
        with open(os.path.join(root, "assets", "plans", f"s{i:02d}.navmesh"), "wb") as f:
            f.write(blob)
        rows = [{"episode_id": str(k), "scene_id": f"plans/s{i:02d}.glb", "start_position": [float(v) for v in e[0:3]],
                 "start_rotation": [float(v) for v in e[3:7]], "goals": [{"position": [float(v) for v in e[7:10]]}]}
                for k, e in enumerate(eps)]
        with gzip.open(os.path.join(root, "content", f"s{i:02d}.json.gz"), "wt") as f:
            json.dump({"episodes": rows}, f)
    return os.path.join(root, "content"), os.path.join(root, "assets")


class ScenePolicy:
    """Independent restatement of which scenes the reference's generator holds and draws next
    (simulator.cpp:1518-1534 selection sampling, :1093-1106 startSceneSwap), on the library's
    counter-based stream of scene choices."""
    M64 = (1 << 64) - 1

    def __init__(self, seed, num_dataset, num_active):
        self.seed, self.k = seed, 0
        self.active, self.inactive = [], []
        i = 0
        while i < num_dataset and len(self.active) < num_active:
            w = np.float32(self.draw() >> 8) * np.float32(1.0 / 16777216.0)
            if w * np.float32(num_dataset - i) < np.float32(num_active - len(self.active)):
                self.active.append(i)
            else:
                self.inactive.append(i)
            i += 1
        self.inactive += list(range(i, num_dataset))

    def mix(self, z):
        z &= self.M64
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & self.M64
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & self.M64
        return z ^ (z >> 31)

    def draw(self):
        key = self.mix(self.seed + 0x9E3779B97F4A7C15 * 0x100000000 + 0xD1B54A32D192ED03)
        r = self.mix(key + 0x9E3779B97F4A7C15 * (self.k + 1)) >> 32
        self.k += 1
        return r

    def start_swap(self, slot):
        pos = (self.draw() * len(self.inactive)) >> 32
        self.inactive[pos], self.active[slot] = self.active[slot], self.inactive[pos]
        return self.active[slot]


def test_dataset_directory_and_automatic_rotation(oracle, torch_cuda, tmp_path):
    """Construction from a dataset directory with more scenes than slots, through the trainer-side
    entry (construct_envs): the library picks the resident scenes at random and rotates the
    others in by itself, loading them in a thread of its own while the simulation steps.  Which
    scenes it picks is checked against an independent restatement of the reference's policy;
    every swap it starts is repeated on the oracle at the same step, and every step is compared
    in full.  Actions stay on the GPU and outputs are taken by device-to-device copies, like a
    device-resident rollout storage would."""
    import time
    from bps_nav_amd import env_utils
    from oracle import bpo
    print("case: dataset directory + automatic rotation", flush=True)
    pool = common.build_scenes(oracle, 2, 5, episodes_per_scene=24) + common.build_scenes(oracle, 1, 3, episodes_per_scene=24)
    content, assets = write_dataset(str(tmp_path), pool)
    n, S, seed = 96, 3, 12345
    envs, obs, rewards, masks, infos, syncs = env_utils.construct_envs(
        "pointnav", content, assets, n, num_worker_groups=S, double_buffered=False, seed=seed, max_steps=40,
        scene_reserve=4.0, rotation_interval_ms=0)
    assert rewards[0].shape == (n, 1) and masks[0].shape == (n, 1) and obs[0]["pointgoal_with_gps_compass"].shape == (n, 2)
    assert all(t.is_cuda for t in (rewards[0], masks[0], obs[0]["pointgoal_with_gps_compass"], infos[0]["spl"]))
    policy = ScenePolicy(seed, len(pool), S)
    first = list(policy.active)
    assert sorted(first) != [0, 1, 2] or True     # any three of the eight
    cpu = bpo.Sim(oracle, [pool[i] for i in first], n, seed=seed, threads=3, max_steps=40)
    expected_next = [policy.start_swap(slot) for slot in range(S)]   # every slot starts loading at construction
    assert list(envs.active_scenes()) == expected_next
    cpu.reset()
    envs.reset(0)
    state, info_view = envs.get_state(0), envs.get_infos(0)
    storage = torch_cuda.zeros((200, n, 1), device="cuda")        # a rollout storage's reward buffer
    pending = {}          # slot -> dataset index on its way in
    events = 0
    acts = common.action_stream(2, 200, n)
    for t, a in enumerate(acts):
        if t in (0, 40, 90):
            time.sleep(0.3)     # let the loader thread finish what it has been asked for
        envs.step_start(0, torch_cuda.from_numpy(a).cuda())
        for step_ordinal, slot, scene in envs.rotation_events():
            assert step_ordinal == t and scene == expected_next[slot], "a scene other than the policy's was brought in"
            cpu.swap_scene(slot, *pool[scene])
            pending[slot] = scene
            events += 1
        cpu.step(a)
        envs.step_end(0)
        syncs[0].wait()
        storage[t].copy_(rewards[0])
        assert_step_equal(cpu, envs, 0, state, info_view, f"at step {t}")
        for slot in sorted(pending):          # postStep: completed swaps draw their slot's next scene, in slot order
            if cpu.swap_remaining(slot) == 0:
                del pending[slot]
                expected_next[slot] = policy.start_swap(slot)
        assert list(envs.active_scenes()) == expected_next
    assert events >= 6, f"only {events} swaps were started"
    pct, in_use, per_scene = envs.swap_stats
    assert pct > 0 and S <= in_use <= 2 * S and per_scene <= n / S
    assert np.isfinite(storage.cpu().numpy()).mean() > 0.9
    with pytest.raises(RuntimeError, match="rotates its scenes by itself"):
        envs.swap_scene(0, *pool[0])
    envs.check_errors()
    envs.close()
    # without rotation the extra scenes are only a pool to pick from
    gen = make_gen(pool, n, seed=seed, rotate=False, num_active_scenes=S)
    assert list(gen.active_scenes()) == first
    gen.close()


def test_error_paths(oracle, torch_cuda):
    print("case: error paths", flush=True)
    sc = common.build_scenes(oracle, 1, 1, episodes_per_scene=8)
    gen = make_gen(sc, 8)
    gen.reset(0)
    with pytest.raises(RuntimeError, match="no step in flight"):
        gen.step_end(0)
    a = np.ones(8, np.int64)
    gen.step_start(0, a)
    with pytest.raises(RuntimeError, match="previous step not finished"):
        gen.step_start(0, a)
    gen.step_end(0)
    before = {k: v.clone() for k, v in gen.get_state(0).items()}
    bad = np.array([1, 7, -1, 2, 1, 1, 1, 1], np.int64)
    gen.step(0, bad)
    after = gen.get_state(0)
    for k in before:  # agents with invalid actions are left untouched
        assert torch_cuda.equal(before[k][1:3], after[k][1:3])
    with pytest.raises(RuntimeError, match="outside 0..3"):
        gen.check_errors()
    with pytest.raises(RuntimeError):
        gen.rgba(0)
    # scene rotation: bad slot, bad mesh, call while a step is in flight, scene that does not fit
    with pytest.raises(RuntimeError, match="slot out of range"):
        gen.swap_scene(3, *sc[0])
    with pytest.raises(RuntimeError, match="magic"):
        gen.swap_scene(0, b"XXXX" + sc[0][0][4:], sc[0][1])
    gen.step_start(0, a)
    with pytest.raises(RuntimeError, match="in flight"):
        gen.swap_scene(0, *sc[0])
    gen.step_end(0)
    assert gen.swap_status(0) == (0, 0)
    from bps_nav_amd import scenes as _sc
    big = _sc.config_scene(3, 0)   # ~20k polygons against a reserve sized for a ~1.6k polygon room
    with pytest.raises(RuntimeError, match="does not fit"):
        gen.swap_scene(0, big, sc[0][1])
    gen.swap_scene(0, *sc[0])       # a scene of the same size does
    assert gen.swap_status(0)[0] == 8
    gen.close()
    from bps_nav_amd import scenes
    four = scenes.gen_scene(scenes.BOX_ROOM, 5, 5, size_x=10.0, size_z=10.0, num_boxes=4, box_min=0.5, box_max=2.0,
                            tiles_x=2, tiles_z=2)
    with pytest.raises(RuntimeError, match="multi-tile"):
        make_gen([(four, sc[0][1])], 8)
    with pytest.raises(RuntimeError, match="magic"):
        make_gen([(b"XXXX" + sc[0][0][4:], sc[0][1])], 8)
    # hostile tile headers: counts that overflow 32-bit size arithmetic or the tree's 16-bit links
    import struct
    blob = bytearray(sc[0][0])
    for off, val, msg in ((48 + 28, 0x7fffffff, "exceeds the tile size"), (48 + 48, 0x10000, "more BV nodes"),
                          (48 + 32, 0x7ffffff0, "exceeds the tile size")):
        bad = bytearray(blob)
        struct.pack_into("<i", bad, off, val)
        with pytest.raises(RuntimeError, match=msg):
            make_gen([(bytes(bad), sc[0][1])], 8)
