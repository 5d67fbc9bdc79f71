"""CPU: what the mathematics fixes, independent of any implementation — closed-form
geodesics on hand-made meshes, the reference's own known-answer vectors
(Tests/Detour/Tests_Detour.cpp:5-33), the step state machine's algebra, brute force and
distribution checks."""
import math

import numpy as np
import pytest

from bps_nav_amd import episodes, scenes
from oracle import bpo
from tests.golden import meshes


def nav_of(oracle, name):
    return bpo.Nav(oracle, meshes.ALL[name]())


def geo(nav, a, b):
    ax, ar = nav.snap(np.array([a], np.float32))
    bx, br = nav.snap(np.array([b], np.float32))
    assert ar[0] and br[0]
    return float(nav.geodesic(ax, ar, bx, br)[0])


def test_detour_known_answer_vectors(oracle):
    # Tests_Detour.cpp:9-31: triangle (0,0,0),(0,0,1),(1,0,0)
    tri = np.array([[0, 0, 0], [0, 0, 1], [1, 0, 0]], np.float32)
    for s, t, want in ((0.0, 1.0, (0, 0, 1)), (0.5, 1.0, (0.5, 0, 0.5)), (1.0, 1.0, (1, 0, 0))):
        got = oracle.random_point_in_convex_poly(tri, s, t)
        assert np.allclose(got, want, atol=1e-6)


def test_l_shape_geodesics(oracle):
    nav = nav_of(oracle, "l_shape")
    # same convex region: straight line
    assert geo(nav, (9, 0, 1), (1, 0, 4)) == pytest.approx(math.hypot(8, 3), rel=1e-6)
    # around the inner corner (5,5), both directions
    bent = 2 * math.sqrt(32)
    assert geo(nav, (9, 0, 1), (1, 0, 9)) == pytest.approx(bent, rel=1e-6)
    assert geo(nav, (1, 0, 9), (9, 0, 1)) == pytest.approx(bent, rel=1e-6)
    # coincident points and a snap far outside
    assert geo(nav, (2, 0, 2), (2, 0, 2)) == 0.0
    x, r = nav.snap(np.array([[50, 0, 50]], np.float32))
    assert r[0] == 0 and np.isnan(x).all()


def test_u_shape_geodesic(oracle):
    nav = nav_of(oracle, "u_shape")
    want = 2 * math.hypot(1.5, 5) + 3
    assert geo(nav, (1.5, 0, 8), (7.5, 0, 8)) == pytest.approx(want, rel=1e-6)


def test_two_rooms_goes_through_the_door(oracle):
    nav = nav_of(oracle, "two_rooms")
    # door spans x 4..4.5, z 1.5..2.5; from (1,·,3.5) to (7.5,·,3.5) the path bends at (4,2.5),(4.5,2.5)
    want = math.hypot(3, 1) + 0.5 + math.hypot(3, 1)
    assert geo(nav, (1, 0, 3.5), (7.5, 0, 3.5)) == pytest.approx(want, rel=1e-6)


def test_ramp_height_and_3d_length(oracle):
    nav = nav_of(oracle, "ramp")
    x, r = nav.snap(np.array([[6, 1.3, 2]], np.float32))  # just above the ramp midpoint, where y = 1
    assert r[0] and x[0, 1] == pytest.approx(1.0, abs=1e-5)
    # the funnel adds no vertex where the slope changes, so the length the reference reports is
    # the 3-D chord between the end points (pathLength, PathFinder.cpp:473-482), not 2+sqrt(20)+2
    want = math.sqrt(64 + 4)
    assert geo(nav, (2, 0, 2), (10, 2, 2)) == pytest.approx(want, rel=1e-5)


def test_islands_are_unreachable(oracle):
    nav = nav_of(oracle, "islands")
    assert math.isinf(geo(nav, (1, 0, 1), (5, 0, 1)))
    refs, flags, isl = nav.poly_info()
    assert len(set(isl.tolist())) == 2


def test_try_step_free_wall_and_slide(oracle):
    nav = nav_of(oracle, "l_shape")
    sx, sr = nav.snap(np.array([[1, 0, 1]], np.float32))
    # free move
    x, r = nav.try_step(sx, sr, np.array([[1.2, 0, 1.1]], np.float32))
    assert np.allclose(x[0], (1.2, 0, 1.1), atol=1e-6) and r[0] == sr[0]
    # straight into the x = 0 wall: clamped onto it
    x, r = nav.try_step(sx, sr, np.array([[-0.5, 0, 1]], np.float32))
    assert np.allclose(x[0], (0, 0, 1), atol=1e-6)
    # oblique push: slides along the wall to the projection of the target
    x, r = nav.try_step(sx, sr, np.array([[-0.3, 0, 1.4]], np.float32))
    assert np.allclose(x[0], (0, 0, 1.4), atol=1e-6)
    # crossing a shared edge changes the polygon
    sx2, sr2 = nav.snap(np.array([[4.9, 0, 1]], np.float32))
    x, r = nav.try_step(sx2, sr2, np.array([[5.1, 0, 1]], np.float32))
    assert r[0] != sr2[0] and np.allclose(x[0], (5.1, 0, 1), atol=1e-6)
    # an invalid start polygon never moves (PathFinder.cpp:556-558)
    x, r = nav.try_step(sx, np.zeros(1, np.uint32), np.array([[1.2, 0, 1.1]], np.float32))
    assert r[0] == 0 and np.array_equal(x, sx)


def test_nearest_poly_matches_brute_force(oracle):
    blob = scenes.config_scene(1, 3)
    nav = bpo.Nav(oracle, blob)
    rng = np.random.default_rng(0)
    pts = scenes.sample_points(blob, 1, 300) + rng.normal(0, 0.4, (300, 3)).astype(np.float32)
    pts[:, 1] = 0.1
    x, r = nav.snap(pts)
    # flat mesh at y = 0, query within climb height: the snapped point is the nearest point of the
    # walkable area in xz; brute force = dense sampling of the walkable polygons
    dense = scenes.sample_points(blob, 2, 200000)
    for i in range(0, 300, 10):
        d_snap = np.hypot(x[i, 0] - pts[i, 0], x[i, 2] - pts[i, 2])
        d_brute = np.hypot(dense[:, 0] - pts[i, 0], dense[:, 2] - pts[i, 2]).min()
        assert d_snap <= d_brute + 1e-5, "a nearer walkable point exists than the one snapPoint returned"
        assert d_brute <= d_snap + 0.05


def test_geodesic_invariants(oracle):
    blob = scenes.config_scene(2, 1)
    nav = bpo.Nav(oracle, blob)
    p = scenes.sample_points(blob, 3, 600)
    x, r = nav.snap(p)
    a, ar, b, br, c, cr = x[:200], r[:200], x[200:400], r[200:400], x[400:], r[400:]
    ab, ba = nav.geodesic(a, ar, b, br), nav.geodesic(b, br, a, ar)
    bc, ac = nav.geodesic(b, br, c, cr), nav.geodesic(a, ar, c, cr)
    fin = np.isfinite(ab) & np.isfinite(bc) & np.isfinite(ac) & np.isfinite(ba)
    assert fin.sum() > 50
    eu = np.linalg.norm(a - b, axis=1)
    assert (ab[fin] >= eu[fin] - 1e-4).all(), "a path shorter than the straight line"
    # the string-pulled corridor is not the exact shortest path, but detours stay small
    assert (ac[fin] <= (ab[fin] + bc[fin]) * 1.15 + 1e-3).all()
    assert np.allclose(ab[fin], ba[fin], rtol=0.1)


def test_area_weighted_sampling_distribution(oracle):
    blob = scenes.config_scene(1, 2)
    nav = bpo.Nav(oracle, blob)
    refs, flags, isl = nav.poly_info()
    rng = np.random.default_rng(9)
    n = 60000
    pts = nav.sample(rng.uniform(0, 1, (n, 3)).astype(np.float32))
    x, r = nav.snap(pts)
    assert (r != 0).all() and np.allclose(x, pts, atol=1e-4), "sampled points must lie on the mesh"
    # chi-square of counts per polygon against polygon areas (areas via a huge uniform sample
    # would be circular; instead use cell counts: every generated polygon is 1, 0.5 or 2 cells)
    counts = np.bincount((r - refs[0]).astype(np.int64), minlength=len(refs)).astype(float)
    # polygon areas from vertex data of the packed tile
    areas = poly_areas(blob)
    exp = areas / areas.sum() * n
    chi2 = ((counts - exp) ** 2 / exp).sum()
    dof = len(refs) - 1
    assert chi2 < dof + 6 * math.sqrt(2 * dof), f"chi2 {chi2:.0f} for {dof} dof"


def poly_areas(blob):
    """xz areas of the polygons of a single-tile MSET blob, from the on-disk layout."""
    import struct
    t = 48
    np_, nv = struct.unpack_from("<ii", blob, t + 24)
    verts = np.frombuffer(blob, np.float32, nv * 3, t + 100).reshape(nv, 3)
    polys = np.frombuffer(blob, np.uint8, np_ * 32, t + 100 + nv * 12).reshape(np_, 32)
    out = np.zeros(np_)
    for i in range(np_):
        idx = polys[i, 4:16].view(np.uint16)
        k = polys[i, 30]
        p = verts[idx[:k]][:, [0, 2]].astype(np.float64)
        out[i] = 0.5 * abs(np.dot(p[:, 0], np.roll(p[:, 1], -1)) - np.dot(p[:, 1], np.roll(p[:, 0], -1)))
    return out


def test_sampling_matches_reference_distribution(oracle, reflib):
    if reflib is None:
        pytest.skip("compiled reference not available outside the development container")
    blob = scenes.config_scene(1, 2)
    no, nr = bpo.Nav(oracle, blob), bpo.Nav(reflib, blob)
    n = 40000
    rx = np.zeros((n, 3), np.float32)
    rr = np.zeros(n, np.uint32)
    reflib.L.bpo_nav_find_random_points(nr.h, 123, n, rx, rr)
    rng = np.random.default_rng(10)
    ox = no.sample(rng.uniform(0, 1, (n, 3)).astype(np.float32))
    # two-sample check on a coarse 8 x 8 grid over the room
    def hist(p):
        h, _, _ = np.histogram2d(p[:, 0], p[:, 2], bins=8, range=[[0, 10], [0, 10]])
        return h.reshape(-1)
    ho, hr = hist(ox), hist(rx)
    m = (ho + hr) > 0
    chi2 = (((ho - hr) ** 2) / (ho + hr))[m].sum()
    dof = m.sum() - 1
    assert chi2 < dof + 6 * math.sqrt(2 * dof), f"chi2 {chi2:.0f} for {dof} dof"


# ---------------------------------------------------------------- state machine algebra
def one_room_sim(oracle, n=1, max_steps=0, start=(2, 0, 2), goal=(2, 0, 8), yaw=0.0, task=0):
    blob = meshes.l_shape()
    ep = np.concatenate([start, episodes.yaw_quat(np.array(yaw)), goal]).astype(np.float32)[None]
    return bpo.Sim(oracle, [(blob, ep)], n, max_steps=max_steps, task=task)


def test_forward_moves_along_heading_and_rewards_progress(oracle):
    # yaw 0 looks down -z; yaw pi looks up +z towards the goal at (2, 8)
    sim = one_room_sim(oracle, yaw=math.pi)
    sim.reset()
    p0 = sim.state()["position"][0].copy()
    sim.step(np.array([1]))
    s, o = sim.state(), sim.outputs()
    assert np.allclose(s["position"][0] - p0, (0, 0, 0.25), atol=1e-6)
    # reward = -slack + (previous distance - new distance) = -0.01 + 0.25
    assert o["rewards"][0] == pytest.approx(0.24, abs=1e-5)
    assert o["masks"][0] == 1 and o["infos"][0, 2] == pytest.approx(5.75, abs=1e-5)
    # polar: goal straight ahead at 5.75 m
    assert o["polars"][0, 0] == pytest.approx(5.75, abs=1e-5) and abs(o["polars"][0, 1]) < 1e-5


def test_thirty_six_left_turns_are_identity_and_turn_reward_is_slack(oracle):
    sim = one_room_sim(oracle, yaw=0.3)
    sim.reset()
    q0 = sim.state()["rotation"][0].copy()
    for _ in range(36):
        sim.step(np.array([2]))
        assert sim.outputs()["rewards"][0] == pytest.approx(-0.01, abs=1e-7)
    q = sim.state()["rotation"][0]
    assert np.allclose(q, -q0, atol=1e-5) or np.allclose(q, q0, atol=1e-5)  # 360 degrees = -q
    # left then right cancels
    sim.step(np.array([2])); sim.step(np.array([3]))
    assert np.allclose(np.abs(sim.state()["rotation"][0]), np.abs(q), atol=1e-6)


def test_polar_of_goal_to_the_left_and_right(oracle):
    # facing -z (yaw 0) at (2,2) with the goal at (2,8): goal is directly behind
    sim = one_room_sim(oracle, yaw=0.0)
    sim.reset()
    o = sim.outputs()
    assert o["polars"][0, 0] == pytest.approx(6.0, abs=1e-5)
    assert abs(abs(o["polars"][0, 1]) - math.pi) < 1e-5
    # facing +x (yaw -pi/2): goal along +z is on the agent's right => phi negative => output -phi positive
    sim = one_room_sim(oracle, yaw=-math.pi / 2)
    sim.reset()
    assert sim.outputs()["polars"][0, 1] == pytest.approx(-math.pi / 2, abs=1e-5) or \
        sim.outputs()["polars"][0, 1] == pytest.approx(math.pi / 2, abs=1e-5)


def test_stop_ends_episode_with_spl_and_success(oracle):
    # start 0.1 m from the goal: stop => success, spl = init / max(init, 0) = 1, reward = -0.01 + 2.5
    sim = one_room_sim(oracle, start=(2, 0, 2), goal=(2, 0, 2.1))
    sim.reset()
    sim.step(np.array([0]))
    o = sim.outputs()
    assert o["masks"][0] == 0 and o["infos"][0, 0] == 1.0 and o["infos"][0, 1] == pytest.approx(1.0)
    assert o["rewards"][0] == pytest.approx(2.49, abs=1e-6)
    assert sim.state()["step"][0] == 1 and sim.state()["num_resets"][0] == 2  # auto-reset in the same step
    # far from the goal: stop => failure, reward = -0.01
    sim = one_room_sim(oracle)
    sim.reset()
    sim.step(np.array([0]))
    o = sim.outputs()
    assert o["masks"][0] == 0 and o["infos"][0, 0] == 0.0 and o["rewards"][0] == pytest.approx(-0.01)


def test_episode_ends_at_max_steps_and_reward_sum_telescopes(oracle):
    sim = one_room_sim(oracle, max_steps=12, yaw=math.pi)
    sim.reset()
    init = 6.0
    total, t, last_d = 0.0, 0, None
    while True:
        sim.step(np.array([1]))
        t += 1
        o = sim.outputs()
        total += float(o["rewards"][0])
        if o["masks"][0] == 0:
            last_d = float(o["infos"][0, 2])
            break
    # step_ starts at 1 and the episode ends when it reaches max_steps: max_steps - 1 actions
    assert t == 11
    # sum of rewards = (init - d_before_last) - 0.01 * T  (+ 2.5 * spl = 0 on failure); the terminal
    # step pays no progress term
    assert last_d == pytest.approx(init - 0.25 * 11, abs=1e-4)
    assert total == pytest.approx((init - (init - 0.25 * 10)) - 0.01 * 11, abs=1e-4)


def test_flee_distance_from_start_and_reward(oracle):
    # Flee (simulator.cpp:830-887): info = geodesic(start point -> agent), refreshed on forward
    # moves only; reward = its change, no slack, no success bonus
    sim = one_room_sim(oracle, yaw=math.pi, task=1, max_steps=9)
    sim.reset()
    assert sim.outputs()["infos"][0, 0] == 0.0
    for k in range(1, 5):
        sim.step(np.array([1]))
        o = sim.outputs()
        assert o["infos"][0, 0] == pytest.approx(0.25 * k, abs=1e-5)   # one convex room: straight line
        assert o["rewards"][0] == pytest.approx(0.25, abs=1e-5) and o["masks"][0] == 1
    sim.step(np.array([2]))      # a turn: distance kept, reward 0
    o = sim.outputs()
    assert o["infos"][0, 0] == pytest.approx(1.0, abs=1e-5) and o["rewards"][0] == 0.0
    sim.step(np.array([3])); sim.step(np.array([3]))
    sim.step(np.array([0]))      # stop: done, distance kept (not recomputed), reward 0, then reset
    o = sim.outputs()
    assert o["masks"][0] == 0 and o["infos"][0, 0] == pytest.approx(1.0, abs=1e-5) and o["rewards"][0] == 0.0
    assert sim.state()["num_resets"][0] == 2 and sim.state()["step"][0] == 1
    sim.step(np.array([1]))      # new episode measures from the new start: prev = 0
    assert sim.outputs()["rewards"][0] == pytest.approx(0.25, abs=1e-5)


def test_exploration_counts_cells_of_the_start_frame(oracle):
    # Exploration (simulator.cpp:889-997): 1 m cells of the start pose's frame, int() truncation,
    # so walking straight ahead along -z' enters a new cell when the path length reaches 1, 2, ...
    for yaw in (math.pi, math.pi - 0.3):
        sim = one_room_sim(oracle, yaw=yaw, task=2, start=(2, 0, 2.5))
        sim.reset()
        assert sim.outputs()["infos"][0, 0] == 0.0
        seen = []
        for k in range(1, 15):
            sim.step(np.array([1]))
            o = sim.outputs()
            seen.append(o["infos"][0, 0])
            if k % 4 != 0:     # away from the exact cell boundaries
                assert o["infos"][0, 0] == float(k // 4), (yaw, k, seen)
        assert seen[-1] == 3.0
        # rewards: 0.25 per new cell, summed = 0.25 * cells
        # turning on the spot or revisiting adds nothing
        for a in (2, 2, 3, 3):
            sim.step(np.array([a]))
            assert sim.outputs()["rewards"][0] == 0.0 and sim.outputs()["infos"][0, 0] == 3.0
    # 18 left turns then forward: back over visited cells, count unchanged
    for _ in range(18):
        sim.step(np.array([2]))
    for _ in range(6):
        sim.step(np.array([1]))
        assert sim.outputs()["infos"][0, 0] == 3.0
    sim.step(np.array([0]))
    assert sim.outputs()["masks"][0] == 0 and sim.outputs()["infos"][0, 0] == 3.0
    sim.step(np.array([1]))
    assert sim.outputs()["infos"][0, 0] == 0.0 and sim.outputs()["rewards"][0] == 0.0


def test_exploration_reward_is_quarter_per_new_cell(oracle):
    sim = one_room_sim(oracle, yaw=math.pi, task=2, start=(2, 0, 2.4))
    sim.reset()
    total = 0.0
    for _ in range(13):
        sim.step(np.array([1]))
        total += sim.outputs()["rewards"][0]
    assert total == pytest.approx(0.25 * sim.outputs()["infos"][0, 0]) and sim.outputs()["infos"][0, 0] == 3.0


def test_scene_rotation_moves_envs_when_their_episode_ends(oracle):
    # SceneSwapper / swapReady / swapScene (simulator.cpp:1063-1154, 1284-1310, 1636-1642): after a
    # swap is started, an env changes scene exactly when its episode ends; an explicit reset does not.
    room = meshes.l_shape()
    other = meshes.two_rooms()
    ep_room = np.concatenate([(2, 0, 2), episodes.yaw_quat(np.array(0.0)), (2, 0, 8)]).astype(np.float32)[None]
    ep_other = np.concatenate([(1, 0, 1), episodes.yaw_quat(np.array(0.0)), (1, 0, 2)]).astype(np.float32)[None]
    sim = bpo.Sim(oracle, [(room, ep_room)], 4, max_steps=6)
    sim.reset()
    sim.swap_scene(0, other, ep_other)
    assert sim.swap_remaining(0) == 4
    with pytest.raises(RuntimeError, match="in progress"):
        sim.swap_scene(0, other, ep_other)
    sim.reset()                                   # not an episode end: nobody moves
    assert sim.swap_remaining(0) == 4
    assert np.allclose(sim.state()["position"], (2, 0, 2), atol=1e-5)
    sim.step(np.array([2, 0, 2, 2]))              # env 1 stops: it alone moves to the new scene
    assert sim.swap_remaining(0) == 3
    pos = sim.state()["position"]
    assert np.allclose(pos[1], (1, 0, 1), atol=1e-5) and np.allclose(pos[[0, 2, 3]], (2, 0, 2), atol=1e-5)
    for _ in range(5):                            # the others run into max_steps
        sim.step(np.array([2, 2, 2, 2]))
    assert sim.swap_remaining(0) == 0
    assert np.allclose(sim.state()["position"], (1, 0, 1), atol=1e-5)
    sim.swap_scene(0, room, ep_room)              # and back again: allowed now
    assert sim.swap_remaining(0) == 4


def test_invalid_action_is_flagged_and_agent_untouched(oracle):
    sim = one_room_sim(oracle)
    sim.reset()
    before = sim.state()
    sim.step(np.array([7]))
    after = sim.state()
    assert sim.bad_action()
    for k in before:
        assert np.array_equal(before[k], after[k])


def test_reset_stream_is_deterministic_and_thread_independent(oracle):
    blob = scenes.config_scene(1, 0)
    nav = bpo.Nav(oracle, blob)
    from tests import common
    eps = episodes.make_episodes(blob, 5, 32, 1.0, 10.0, common.oracle_geodesic_fn(nav))
    rng = np.random.default_rng(1)
    acts = [episodes.random_actions(rng, 32, None) for _ in range(60)]
    runs = []
    for threads in (1, 4):
        sim = bpo.Sim(oracle, [(blob, eps)], 32, seed=42, threads=threads)
        sim.reset()
        for a in acts:
            sim.step(a)
        runs.append((sim.state(), sim.outputs()))
    for k in runs[0][0]:
        assert np.array_equal(runs[0][0][k], runs[1][0][k], equal_nan=True)
    for k in runs[0][1]:
        assert np.array_equal(runs[0][1][k], runs[1][1][k], equal_nan=True)
