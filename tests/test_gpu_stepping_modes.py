"""GPU parity of the ways a caller may drive the engine besides reset-then-step: a reset of a
group after stepping has begun (simulator.cpp:1377-1380), stream-ordered stepping (step_end
that leaves the waiting to the stream), and automatic scene rotation with two groups, under
stream-ordered stepping, and with a pool whose later scenes are larger than the first ones.
Everything is compared with the CPU oracle, bit for bit except the polar angle.
"""
import time

import numpy as np
import pytest

from tests import common
from tests.test_gpu_parity import ScenePolicy, assert_step_equal, make_gen, write_dataset

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch_cuda():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch


def test_reset_of_a_group_in_mid_run(oracle, torch_cuda):
    """reset(group) after 40 steps: first distances of the episodes begun in the last step are
    still to be measured and both sets of queues have been in use.  The group starts over like
    the oracle's, and 110 further steps stay equal."""
    from oracle import bpo
    print("case: reset of a group in mid-run (one group)", flush=True)
    sc = common.build_scenes(oracle, 2, 4, episodes_per_scene=32)
    n = 256
    cpu = bpo.Sim(oracle, sc, n, seed=29, threads=4, max_steps=60)
    gen = make_gen(sc, n, seed=29, max_steps=60)
    cpu.reset()
    gen.reset(0)
    state, infos = gen.get_state(0), gen.get_infos(0)
    acts = common.action_stream(2, 190, n)
    for t, a in enumerate(acts):
        if t in (40, 41, 97):       # also twice in a row, and once more later
            cpu.reset()
            gen.reset(0)
            cs = cpu.state()
            st = {k: v.cpu().numpy() for k, v in state.items()}
            for k in ("poly_ref", "goal_ref", "step", "episode", "num_resets"):
                assert np.array_equal(cs[k], st[k].view(np.uint32)), f"{k} differs after the reset before step {t}"
            assert np.array_equal(common.bits(st["position"]), common.bits(cs["position"]))
            gp, cp = gen.get_polars(0).cpu().numpy(), cpu.outputs()["polars"]
            np.testing.assert_allclose(gp[:, 0], cp[:, 0], rtol=1e-6, atol=1e-6)   # a reset writes the polar only
        cpu.step(a)
        gen.step(0, torch_cuda.from_numpy(a).cuda() if t % 2 else a)
        co, cs = assert_step_equal(cpu, gen, 0, state, infos, f"at step {t}")
    assert int(cs["num_resets"].sum()) > 4 * n
    gen.check_errors()
    gen.close()


def test_reset_of_one_group_between_the_other_groups_steps(oracle, torch_cuda):
    """double_buffered=True: group 0 is reset in mid-run between two steps of group 1 (and later
    group 1 between steps of group 0); both groups stay equal to the oracle's for 100 more steps
    each."""
    from bps_nav_amd import episodes
    from oracle import bpo
    print("case: reset of a group in mid-run (two groups)", flush=True)
    sc = common.build_scenes(oracle, 2, 4, episodes_per_scene=32)
    n = 256
    cpu = bpo.Sim(oracle, sc, n, double_buffered=True, seed=31, threads=4, max_steps=50)
    gen = make_gen(sc, n, double_buffered=True, seed=31, max_steps=50)
    state = [gen.get_state(g) for g in (0, 1)]
    infos = [gen.get_infos(g) for g in (0, 1)]
    for g in (0, 1):
        cpu.reset(g)
        gen.reset(g)
    rng = np.random.default_rng(43)
    for t in range(280):
        g = t % 2
        if t in (61, 150):          # t odd: group 1 steps next, group 0 stepped last; t even: the other way round
            r = 1 - g
            cpu.reset(r)
            gen.reset(r)
        a = episodes.random_actions(rng, n // 2, 0.6)
        cpu.step(a, g)
        gen.step(g, torch_cuda.from_numpy(a).cuda())
        co, cs = assert_step_equal(cpu, gen, g, state[g], infos[g], f"group {g} at step {t}")
    gen.check_errors()
    gen.close()


class Recorder:
    """Takes a group's outputs and state after every step with device-to-device copies on the
    current stream, like a device-resident rollout storage: nothing waits for the device."""
    KEYS = ("poly_ref", "goal_ref", "step", "episode", "num_resets", "position", "rotation")

    def __init__(self, torch, gen, group, steps):
        self.gen, self.group = gen, group
        self.src = dict(rewards=gen.get_rewards(group), masks=gen.get_masks(group), infos=gen.get_infos(group).packed,
                        polars=gen.get_polars(group))
        st = gen.get_state(group)
        self.src.update({k: st[k] for k in self.KEYS})
        self.buf = {k: torch.empty((steps,) + tuple(v.shape), dtype=v.dtype, device=v.device) for k, v in self.src.items()}

    def take(self, t):
        for k, v in self.src.items():
            self.buf[k][t].copy_(v, non_blocking=True)

    def host(self):
        return {k: v.cpu().numpy() for k, v in self.buf.items()}


def compare_recorded(cpu, rec, t, where, group=0):
    """Step t of a recording against the oracle's state and outputs, as assert_step_equal does."""
    co, cs = cpu.outputs(group), cpu.state(group)
    for k in ("poly_ref", "goal_ref", "step", "episode", "num_resets"):
        assert np.array_equal(cs[k], rec[k][t].view(np.uint32)), f"{k} differs {where}"
    assert np.array_equal(common.bits(rec["position"][t]), common.bits(cs["position"])), f"position differs {where}"
    assert np.array_equal(common.bits(rec["rotation"][t]), common.bits(cs["rotation"])), f"rotation differs {where}"
    assert np.array_equal(co["masks"], rec["masks"][t]), f"dones differ {where}"
    gi, ci = rec["infos"][t], co["infos"]
    assert ((common.bits(gi) == common.bits(ci)) | (np.isnan(gi) & np.isnan(ci))).all(), f"infos differ {where}"
    gr = rec["rewards"][t]
    assert ((common.bits(gr) == common.bits(co["rewards"])) | (np.isnan(gr) & np.isnan(co["rewards"]))).all(), \
        f"rewards differ {where}"
    gp = rec["polars"][t]
    np.testing.assert_allclose(gp[:, 0], co["polars"][:, 0], rtol=1e-6, atol=1e-6)
    dphi = np.abs(gp[:, 1] - co["polars"][:, 1])
    assert (np.minimum(dphi, 2 * np.pi - dphi) < 1e-4).all(), f"polar angle differs {where}"
    return co, cs


@pytest.mark.parametrize("config,num_scenes,n,steps,groups", [(4, 4, 256, 260, 1), (2, 4, 256, 240, 2)])
def test_stream_ordered_stepping_parity(oracle, torch_cuda, config, num_scenes, n, steps, groups):
    """bpsx_set_stream_ordered: step_end does not wait, the host runs ahead of the device, and a
    consumer on the same stream (device-to-device copies after every step) sees every step
    complete.  All recorded steps are compared with the oracle afterwards."""
    torch = torch_cuda
    from oracle import bpo
    print(f"case: stream-ordered stepping, config {config}, {groups} group(s)", flush=True)
    sc = common.build_scenes(oracle, config, num_scenes, episodes_per_scene=32)
    gen = make_gen(sc, n, seed=37, double_buffered=groups == 2, stream_ordered=True)
    per = n // groups
    for g in range(groups):
        gen.reset(g)
    acts = common.action_stream(config, steps, per)
    dev_acts = torch.from_numpy(np.stack(acts)).cuda()
    recs = [Recorder(torch, gen, g, steps) for g in range(groups)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for t in range(steps):
        g = t % groups
        gen.step_start(g, dev_acts[t])
        gen.step_end(g)
        recs[g].take(t)
    enqueued = time.perf_counter() - t0
    gen.synchronize()
    torch.cuda.synchronize()
    total = time.perf_counter() - t0
    print(f"  {steps} steps enqueued in {enqueued * 1e3:.1f} ms, complete after {total * 1e3:.1f} ms", flush=True)
    host = [r.host() for r in recs]
    cpu = bpo.Sim(oracle, sc, n, double_buffered=groups == 2, seed=37, threads=4)
    for g in range(groups):
        cpu.reset(g)
    for t in range(steps):
        g = t % groups
        cpu.step(acts[t], g)
        co, cs = compare_recorded(cpu, host[g], t, f"at step {t}", g)
    assert int(cs["num_resets"].sum()) > per
    gen.check_errors()
    # back to host-synchronous stepping on the same simulator: still equal
    gen.set_stream_ordered(False)
    state, infos = gen.get_state(0), gen.get_infos(0)
    for t, a in enumerate(common.action_stream(config, 8, per)):
        cpu.step(a, 0)
        gen.step(0, a)     # host-side actions
        assert_step_equal(cpu, gen, 0, state, infos, f"at host-synchronous step {t}")
    gen.close()


def rotation_pool(oracle):
    return common.build_scenes(oracle, 2, 5, episodes_per_scene=24) + common.build_scenes(oracle, 1, 3, episodes_per_scene=24)


def test_stream_ordered_stepping_with_automatic_rotation(oracle, torch_cuda, tmp_path):
    """Scene rotation while the host runs ahead of the device: completed swaps are noticed from
    the counts that earlier steps brought back, never by waiting.  The swaps the library started
    (rotation log) are repeated on the oracle at the same steps afterwards; the scenes must be the
    ones the policy draws, in the order in which the swaps completed, and every step must be equal."""
    torch = torch_cuda
    from bps_nav_amd import env_utils
    from oracle import bpo
    print("case: stream-ordered stepping + automatic rotation", flush=True)
    pool = rotation_pool(oracle)
    content, assets = write_dataset(str(tmp_path), pool)
    n, S, seed, steps = 96, 3, 777, 320
    envs, obs, rewards, masks, infos, syncs = env_utils.construct_envs(
        "pointnav", content, assets, n, num_worker_groups=S, double_buffered=False, seed=seed, max_steps=40,
        rotation_interval_ms=0, stream_ordered=True)
    policy = ScenePolicy(seed, len(pool), S)
    first = list(policy.active)
    expected_next = [policy.start_swap(slot) for slot in range(S)]
    envs.reset(0)
    acts = common.action_stream(2, steps, n)
    dev_acts = torch.from_numpy(np.stack(acts)).cuda()
    rec = Recorder(torch, envs, 0, steps)
    events = {}
    for t in range(steps):
        if t % 40 == 0:
            time.sleep(0.05)     # lets the loader thread and the device catch up now and then
        envs.step_start(0, dev_acts[t])
        for step_ordinal, slot, scene in envs.rotation_events():
            assert step_ordinal == t
            events.setdefault(t, []).append((slot, scene))
        envs.step_end(0)
        rec.take(t)
    envs.synchronize()
    host = rec.host()
    cpu = bpo.Sim(oracle, [pool[i] for i in first], n, seed=seed, threads=3, max_steps=40)
    cpu.reset()
    pending = {}
    for t in range(steps):
        for slot, scene in events.get(t, []):
            assert scene == expected_next[slot], f"step {t}: slot {slot} got scene {scene}, the policy draws {expected_next[slot]}"
            cpu.swap_scene(slot, *pool[scene])
            pending[slot] = scene
        cpu.step(acts[t])
        compare_recorded(cpu, host, t, f"at step {t}")
        for slot in sorted(pending):
            if cpu.swap_remaining(slot) == 0:
                del pending[slot]
                expected_next[slot] = policy.start_swap(slot)
    assert sum(len(v) for v in events.values()) >= 6, "too few swaps were started"
    assert envs.swap_stats[0] > 0
    envs.check_errors()
    envs.close()


def test_two_group_automatic_rotation(oracle, torch_cuda, tmp_path):
    """construct_envs' default, double_buffered=True, with automatic rotation: the two groups share
    the loader thread, the scene choices and the side stream; a slot's swap is started by whichever
    group steps next and completed by the steps of the slot's own group."""
    from bps_nav_amd import env_utils
    from oracle import bpo
    print("case: automatic rotation with two groups", flush=True)
    pool = rotation_pool(oracle)
    content, assets = write_dataset(str(tmp_path), pool)
    n, S, seed = 128, 4, 4242
    envs, obs, rewards, masks, infos, syncs = env_utils.construct_envs(
        "pointnav", content, assets, n, num_worker_groups=S, double_buffered=True, seed=seed, max_steps=40,
        rotation_interval_ms=0)
    assert envs.num_groups == 2 and len(rewards) == 2
    policy = ScenePolicy(seed, len(pool), S)
    first = list(policy.active)
    cpu = bpo.Sim(oracle, [pool[i] for i in first], n, double_buffered=True, seed=seed, threads=4, max_steps=40)
    expected_next = [policy.start_swap(slot) for slot in range(S)]
    assert list(envs.active_scenes()) == expected_next
    state = [envs.get_state(g) for g in (0, 1)]
    info_view = [envs.get_infos(g) for g in (0, 1)]
    for g in (0, 1):
        cpu.reset(g)
        envs.reset(g)
    rng = np.random.default_rng(47)
    from bps_nav_amd import episodes
    pending, events = {}, 0
    for t in range(400):
        g = t % 2
        if t in (0, 60, 140, 220, 300):
            time.sleep(0.3)
        a = episodes.random_actions(rng, n // 2, 0.6)
        envs.step_start(g, torch_cuda.from_numpy(a).cuda())
        for step_ordinal, slot, scene in envs.rotation_events():
            assert step_ordinal == t and scene == expected_next[slot]
            cpu.swap_scene(slot, *pool[scene])
            pending[slot] = scene
            events += 1
        cpu.step(a, g)
        envs.step_end(g)
        assert_step_equal(cpu, envs, g, state[g], info_view[g], f"group {g} at step {t}")
        for slot in sorted(pending):
            if cpu.swap_remaining(slot) == 0:
                del pending[slot]
                expected_next[slot] = policy.start_swap(slot)
        assert list(envs.active_scenes()) == expected_next
    assert events >= 8, f"only {events} swaps were started"
    slots_seen = envs.swap_stats
    assert slots_seen[0] > 0 and S <= slots_seen[1] <= 2 * S
    envs.check_errors()
    envs.close()


def test_rotation_when_later_scenes_are_larger_than_the_first(oracle, torch_cuda):
    """A pool of three small rooms and three plans about ten times their size, started on the
    three small ones: the space for rotation is sized from the pool, not from the scenes that
    happen to start resident, so the large scenes come in, swaps keep completing, and no load
    fails.  Compared with the oracle at every step."""
    from bps_nav_amd.bps_sim import PointNavRolloutGenerator
    from oracle import bpo
    print("case: rotation into larger scenes", flush=True)
    small = common.build_scenes(oracle, 1, 3, episodes_per_scene=24)          # ~1.6k polygons
    large = [common.build_scenes(oracle, 3, 1, episodes_per_scene=24)[0]] * 1 + common.build_scenes(oracle, 4, 2, episodes_per_scene=24)
    pool = small + large
    n, S = 96, 3
    seed = next(s for s in range(1000) if sorted(ScenePolicy(s, len(pool), S).active) == [0, 1, 2])
    gen = PointNavRolloutGenerator("", "", n, S, scenes=pool, seed=seed, max_steps=30, rotate=True, rotation_interval_ms=0)
    policy = ScenePolicy(seed, len(pool), S)
    cpu = bpo.Sim(oracle, [pool[i] for i in policy.active], n, seed=seed, threads=3, max_steps=30)
    expected_next = [policy.start_swap(slot) for slot in range(S)]
    cpu.reset()
    gen.reset(0)
    state, infos = gen.get_state(0), gen.get_infos(0)
    pending, brought_in = {}, []
    for t, a in enumerate(common.action_stream(2, 300, n)):
        if t % 50 == 0:
            time.sleep(0.3)
        gen.step_start(0, a)
        for step_ordinal, slot, scene in gen.rotation_events():      # raises if the loader thread failed
            assert scene == expected_next[slot]
            cpu.swap_scene(slot, *pool[scene])
            pending[slot] = scene
            brought_in.append(scene)
        cpu.step(a)
        gen.step_end(0)                                               # raises if a load failed for good
        assert_step_equal(cpu, gen, 0, state, infos, f"at step {t}")
        for slot in sorted(pending):
            if cpu.swap_remaining(slot) == 0:
                del pending[slot]
                expected_next[slot] = policy.start_swap(slot)
    assert sum(1 for s in brought_in if s >= 3) >= 3, f"large scenes were not brought in: {brought_in}"
    assert len(brought_in) >= 6 and gen.swap_stats[0] > 0
    gen.check_errors()
    gen.close()
