"""GPU measurement (not collected by pytest): a benchmark configuration at its own agent and scene
counts, stepped side by side with the CPU oracle on all host cores for as many steps as asked for
and compared in full after every step (the comparison of tests/test_gpu_parity.py, on a longer run).

    python tests/measure_long_parity.py <configuration 2|3|4> <scenes> <agents> <steps> <reset mode 0|1>
    python tests/measure_long_parity.py 4 128 16384 400 0      # about 30 s on the MI355X box
"""
import os, sys, time
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))
import numpy as np, torch
import common
from test_gpu_parity import assert_step_equal
from bps_nav_amd import episodes, scenes
from bps_nav_amd.bps_sim import PointNavRolloutGenerator, nav_only
from oracle import bpo
config, S, N, steps, mode = (int(v) for v in sys.argv[1:6])
oracle = bpo.load_oracle()
blobs = [scenes.config_scene(config, i) for i in range(S)]
nav = nav_only(blobs)
def gfn(i):
    def f(s, g):
        sx, sr = nav.snap_points(i, s); gx, gr = nav.snap_points(i, g)
        return nav.geodesic(i, sx, sr, gx, gr)
    return f
dmin, dmax, pf = common.CONFIGS[config]
sc = [(b, episodes.make_episodes(b, 2000 + i, 128, dmin, dmax, gfn(i))) for i, b in enumerate(blobs)]
nav.close()
rng = np.random.default_rng(55)
gen = PointNavRolloutGenerator("", "", N, S, scenes=sc, seed=91, reset_mode=mode)
cpu = bpo.Sim(oracle, sc, N, seed=91, reset_mode=mode, threads=min(16, len(os.sched_getaffinity(0))))
gen.reset(0); cpu.reset()
state, infos = gen.get_state(0), gen.get_infos(0)
t0 = time.time()
for t in range(steps):
    a = episodes.random_actions(rng, N, pf)
    gen.step(0, torch.from_numpy(a).cuda()); cpu.step(a)
    assert_step_equal(cpu, gen, 0, state, infos, f"at step {t}")
    if t % 50 == 0: print(f"config {config}: step {t} equal, {time.time() - t0:.0f}s", flush=True)
c = gen.counters()
print(f"config {config}: {steps} steps x {N} agents equal to the oracle; replays {c['geo_tie_replays']}, pair ties {c['geo_pair_ties']}, exact runs {c['geo_exact_runs']}, link spills {c['geo_link_spills']}")
gen.check_errors(); gen.close(); cpu.close()
