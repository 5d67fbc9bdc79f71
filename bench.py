"""Benchmark of the batch environment step on one MI355X.

Workload (config.workload "C4"): 16384 agents over 128 corridor-maze scenes of about 30k
polygons each, episodes of 15-40 m geodesic, action stream with P(forward) = 0.8, auto-reset
on done — the configuration BASELINE.json's metric is quoted on.  One "step" is one
step_start/step_end of all agents.  The configuration runs 2000 steps: what is timed starts from
its stationary state (--settle untimed steps after the whole-group reset, then the warm-up
steps), on the GPU and on the CPU alike.  The headline times K steps of stream-ordered stepping
(step_end leaves the waiting to the stream, one device synchronization after the K steps); the
same K steps with a host wait in every step_end, and the steps right after a reset, are
reported beside it.  Prints ONE JSON line on stdout; progress goes to stderr.

    python bench.py --gpus 1 --steps 200 --warmup 20
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "agent env-steps/sec (1 GPU, 16384 agents) + % HBM roofline vs CPU ref"
HBM_PEAK_GBS = 8000.0
# Algorithmic bytes of the geodesic kernel per query (reference data-structure sizes): a corridor
# of L polygons costs L * (4 next-pointer + 32 dtPoly + 24 two portal vertices) and the two
# end polygons are read once more for the boundary clamp, 2 * (32 + 12 * nv) with nv = 4.
BYTES_PER_CORRIDOR_POLY = 60
BYTES_PER_QUERY_ENDS = 2 * (32 + 12 * 4)
# Counter figures of the dominant kernel (HBM bytes per launch, vector instructions per launch)
# are not measured by this script: they come from rocprofv3 --pmc runs of this file whose
# summary is tracked in profiles/.  That summary names the kernel sources it was measured on
# (a hash); the figures are printed only while the sources are still the same, otherwise null.
COUNTER_SUMMARY = os.path.join(ROOT, "profiles", "k_geodesic_c4_hbm_traffic.md")
KERNEL_SOURCES = ("device_types.h", "kernels.h", "nav_device.h", "geodesic_device.h", "kernels.hip")
# Instruction issue peak of either pipe: a CU issues one vector instruction of a wavefront per
# cycle (four SIMDs, four cycles per 64-lane instruction each) and one scalar-unit instruction
# per cycle; 256 CUs at 2.4 GHz.
ISSUE_PEAK = 256 * 2.4e9


def log(*a):
    print("[bench]", *a, file=sys.stderr, flush=True)


def kernel_source_hash():
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "bps_nav_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def tracked_counters():
    """{name: value} from the `measured:` line of the tracked counter summary, or {} when the
    summary is missing or was measured on other kernel sources."""
    try:
        with open(COUNTER_SUMMARY) as f:
            lines = [ln for ln in f if ln.startswith("measured:")]
    except OSError:
        return {}
    if not lines:
        return {}
    kv = dict(item.split("=", 1) for item in lines[-1].split()[1:])
    if kv.get("kernel_source_sha16") != kernel_source_hash():
        log(f"{os.path.relpath(COUNTER_SUMMARY, ROOT)} was measured on other kernel sources: counter figures not printed")
        return {}
    return kv


def gpu_geodesic_fn(nav, scene):
    def f(s, g):
        sx, sr = nav.snap_points(scene, s)
        gx, gr = nav.snap_points(scene, g)
        return nav.geodesic(scene, sx, sr, gx, gr)
    return f


def build_workload(num_scenes, episodes_per_scene):
    """Scenes 0..num_scenes-1 of configuration 4 with episode tables whose geodesic distances
    are measured by the engine's own batched queries."""
    from bps_nav_amd import episodes, scenes
    from bps_nav_amd.bps_sim import nav_only
    t0 = time.time()
    blobs = [scenes.config_scene(4, i) for i in range(num_scenes)]
    log(f"generated {num_scenes} scenes, {sum(len(b) for b in blobs) / 1e6:.0f} MB, {time.time() - t0:.1f}s")
    t0 = time.time()
    nav = nav_only(blobs)
    out = []
    for i, b in enumerate(blobs):
        out.append((b, episodes.make_episodes(b, 2000 + i, episodes_per_scene, 15.0, 40.0, gpu_geodesic_fn(nav, i))))
    nav.close()
    log(f"built episode tables ({episodes_per_scene} per scene) in {time.time() - t0:.1f}s")
    return out


def cpu_baseline(workload, agents_per_scene, seed, p_forward, budget_s=20.0, require_ref=False, threads=0, settle=100):
    """The CPU step on a bounded sample of the same workload: the first scenes of the list with
    the same number of agents per scene, the reference's threading model (one worker per core),
    the same `settle` untimed steps after the reset as the GPU leg, 20 warm-up steps, then timed
    steps.  Runs the compiled reference (oracle/_ref, built in the
    development container from the reference's own sources) when that library is present, else
    the restated oracle; which one is reported as `kind`."""
    import numpy as np

    from bps_nav_amd import episodes
    from oracle import bpo
    lib = bpo.load_ref()
    if lib is None:
        if require_ref:
            print("bench.py: --require-ref given but oracle/_ref/libbpsref.so is not there", file=sys.stderr)
            sys.exit(3)
        log("oracle/_ref/libbpsref.so is not there: the CPU leg runs the restated oracle (kind \"port\")")
        lib = bpo.load_oracle()
    affinity = len(os.sched_getaffinity(0))
    # a GPU box grants a job the CPU share of its GPU (16 cores of the host), whatever the
    # affinity mask shows; more threads than that would be timed on borrowed cores
    cores = threads if threads > 0 else min(affinity, 16)
    sample_scenes = min(len(workload), 16)
    n = sample_scenes * agents_per_scene
    t0 = time.time()
    sim = bpo.Sim(lib, workload[:sample_scenes], n, seed=seed, threads=cores)
    sim.reset()
    log(f"cpu baseline: {lib.path} (kind {lib.kind}); {sample_scenes} scenes, {n} agents, {cores} threads of {affinity} "
        f"cores in the affinity mask, setup {time.time() - t0:.1f}s")
    rng = np.random.default_rng(77)
    # the steps right after the reset, timed apart (the GPU leg reports them too)
    t0 = time.perf_counter()
    for _ in range(min(settle, 20)):
        sim.step(episodes.random_actions(rng, n, p_forward))
    after_reset = n * min(settle, 20) / (time.perf_counter() - t0) if settle > 0 else None
    for _ in range(max(0, settle - 20) + 20):
        sim.step(episodes.random_actions(rng, n, p_forward))
    steps, elapsed = 0, 0.0
    while steps < 400 and elapsed < budget_s:
        a = episodes.random_actions(rng, n, p_forward)
        t0 = time.perf_counter()
        sim.step(a)
        elapsed += time.perf_counter() - t0
        steps += 1
    sim.close()
    # the same step on one thread, on a smaller sample (2 scenes), for the per-core rate
    n1 = min(2, sample_scenes) * agents_per_scene
    sim = bpo.Sim(lib, workload[:min(2, sample_scenes)], n1, seed=seed, threads=1)
    sim.reset()
    for _ in range(settle + 5):
        sim.step(episodes.random_actions(rng, n1, p_forward))
    steps1, elapsed1 = 0, 0.0
    while steps1 < 200 and elapsed1 < budget_s / 4:
        a = episodes.random_actions(rng, n1, p_forward)
        t0 = time.perf_counter()
        sim.step(a)
        elapsed1 += time.perf_counter() - t0
        steps1 += 1
    sim.close()
    return {"value": n * steps / elapsed, "unit": "agent-steps/s", "cores": cores, "affinity_cores": affinity,
            "kind": lib.kind, "library": os.path.relpath(lib.path, ROOT),
            "sample": f"first {sample_scenes} of the {len(workload)} scenes, {n} agents, {settle} settle + 20 warm-up + {steps} timed steps",
            "value_first_steps_after_reset": after_reset,
            "single_thread_value": n1 * steps1 / elapsed1,
            "single_thread_sample": f"first 2 scenes, {n1} agents, {settle} settle + 5 warm-up + {steps1} timed steps"}


def measured_copy_bandwidth(torch):
    """Bytes read plus written per second by a 256 MiB device-to-device copy on this box, in GB/s:
    what the memory system delivers to a plain streaming kernel, next to the nominal peak."""
    src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device="cuda")
    dst = torch.empty_like(src)
    dst.copy_(src)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(10):
        dst.copy_(src)
    e1.record()
    torch.cuda.synchronize()
    return 10 * 2 * src.numel() * 4 / (e0.elapsed_time(e1) * 1e-3) / 1e9


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--settle", type=int, default=100,
                    help="steps taken after the whole-group reset and before the warm-up steps, untimed: configuration 4 "
                         "runs 2000 steps with auto-reset, so what is timed starts from its stationary mix of episode ages "
                         "(right after a reset every agent is at the start of an episode, 15 %% more of them move freely "
                         "and ask for a distance than later on)")
    ap.add_argument("--agents", type=int, default=16384)
    ap.add_argument("--scenes", type=int, default=128)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--require-ref", action="store_true",
                    help="exit with an error instead of timing the restated oracle when the compiled reference is missing")
    ap.add_argument("--cpu-threads", type=int, default=0, help="threads of the CPU leg (default: affinity cores, at most 16)")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy, so a counter profile of this command holds a "
                         "kernel of known traffic to scale FETCH_SIZE / WRITE_SIZE by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this engine runs on one GPU; --gpus must be 1 (agents are independent, so a "
              "multi-GPU run would be one such process per GPU on its own share of agents)", file=sys.stderr)
        sys.exit(2)
    import numpy as np
    import torch

    from bps_nav_amd.bps_sim import PointNavRolloutGenerator
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    N, S, K, W = args.agents, args.scenes, args.steps, args.warmup
    seed, p_forward = 3004, 0.8
    workload = build_workload(S, max(64, 2 * (N // S)))
    gen = PointNavRolloutGenerator("", "", N, S, gpu_id=0, scenes=workload, seed=seed)
    # action streams of configuration 4, resident in HBM before any timed region
    g = torch.Generator().manual_seed(3004)
    p_turn = (1.0 - p_forward - 0.04) / 2
    probs = torch.tensor([0.04, p_forward, p_turn, p_turn])

    def action_block(steps, generator):
        return torch.multinomial(probs.expand(max(1, steps), 4), N, replacement=True, generator=generator).to(torch.int64).cuda()
    actions = action_block(K + W, g)
    if args.calib_copy:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    copy_gbs = measured_copy_bandwidth(torch)

    def timed(block, first, count):
        """`count` steps from row `first` of an action block: (wall seconds between two device
        synchronizations, seconds between two HIP events on the stream the steps run on)."""
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record()
        for t in range(first, first + count):
            gen.step_start(0, block[t])
            gen.step_end(0)
        e1.record()
        torch.cuda.synchronize()
        return time.perf_counter() - t0, e0.elapsed_time(e1) * 1e-3

    gen.reset(0)
    after_reset = None
    if args.settle > 0:
        settle = action_block(args.settle, torch.Generator().manual_seed(3005))
        head = min(args.settle, 25)
        for t in range(min(5, head)):
            gen.step(0, settle[t])
        if head > 5:
            # steps 5..25 after the whole-group reset, host-synchronous: every agent near the start of an episode
            wall, _ = timed(settle, 5, head - 5)
            after_reset = {"ms_per_step": wall / (head - 5) * 1e3, "value": N * (head - 5) / wall,
                           "steps": f"steps 5..{head} after the whole-group reset, host-synchronous"}
        for t in range(head, args.settle):
            gen.step(0, settle[t])
        del settle
    # headline: K steps of stream-ordered stepping (step_end leaves the waiting to the stream; the
    # host runs at most four steps ahead), one device synchronization at the end
    gen.set_stream_ordered(True)
    for t in range(W):
        gen.step_start(0, actions[t])
        gen.step_end(0)
    elapsed, elapsed_events = timed(actions, W, K)
    gen.set_stream_ordered(False)
    gen.check_errors()
    # the same number of steps with a host wait in every step_end (the reference's calling pattern)
    sync_actions = action_block(K, g)
    for t in range(min(W, 5)):
        gen.step(0, sync_actions[t])
    sync_elapsed, _ = timed(sync_actions, 0, K)
    gen.check_errors()
    # a further pass with HIP events around every kernel (on the stream the kernels run on):
    # per-kernel durations and the counters the roofline uses
    P = min(K, 100)
    extra = action_block(P, g)
    c0 = gen.counters()
    gen.set_profiling(True)
    torch.cuda.synchronize()
    tp = time.perf_counter()
    for t in range(P):
        gen.step_start(0, extra[t])
        gen.step_end(0)
    torch.cuda.synchronize()
    profiled_elapsed = time.perf_counter() - tp
    gen.set_profiling(False)
    gen.check_errors()
    c1 = gen.counters()
    kt, profiled = gen.kernel_times()
    assert profiled == P
    d = {k: c1[k] - c0[k] for k in c1 if k != "phase_cycles"}
    if any(c1["phase_cycles"]):
        ph = [a - b for a, b in zip(c1["phase_cycles"], c0["phase_cycles"])]
        log("A* phase cycles per expanded node (diagnostic build): " + " ".join(f"{v / max(1, d['astar_pops']):.0f}" for v in ph))
    dist = gen.get_infos(0)["distanceToGoal"].cpu().numpy()
    log(f"timed {K} steps in {elapsed:.3f}s ({elapsed / K * 1e3:.3f} ms/step stream-ordered, {elapsed_events / K * 1e3:.3f} by HIP events; "
        f"{sync_elapsed / K * 1e3:.3f} ms/step host-synchronous); profiled pass: {P} steps, "
        f"{profiled_elapsed / P * 1e3:.3f} ms/step, per-kernel ms/step {json.dumps({k: round(v, 4) for k, v in kt.items()})}")
    log(f"per step: {d['geodesic_queries'] / P:.0f} geodesic queries, {d['astar_pops'] / max(1, d['geodesic_queries']):.0f} "
        f"A* pops/query, corridor {d['corridor_polys'] / max(1, d['geodesic_queries']):.1f} polys/query, "
        f"{d['resets'] / P:.1f} resets, {d.get('geo_link_spills', 0) / P:.0f} link spills, {d.get('geo_heap_spills', 0) / P:.0f} heap spills, {d.get('geo_long_path', 0) / P:.0f} on the large-LDS path, {d.get('geo_exact_runs', 0) / P:.0f} run again with the exact heap, {d.get('geo_pair_ties', 0) / P:.0f} tied pairs taken in one pass, {d.get('geo_tie_replays', 0) / P:.0f} ties resolved from the log; non-finite distances now: {int((~np.isfinite(dist)).sum())} of {N}")
    # roofline of the dominant kernel (geodesic over the step's queries), HIP-event timed; the
    # counters cover the profiled pass
    dominant = max(kt, key=kt.get)
    geo_bytes = BYTES_PER_CORRIDOR_POLY * d["corridor_polys"] + BYTES_PER_QUERY_ENDS * d["geodesic_queries"]
    geo_ms = kt["geodesic"]
    achieved = geo_bytes / P / (geo_ms * 1e-3) / 1e9 if geo_ms > 0 else 0.0
    tracked = tracked_counters() if (N, S) == (16384, 128) else {}
    expansions_per_launch = d["astar_pops"] / P
    expansions_per_s = expansions_per_launch / (geo_ms * 1e-3) if geo_ms > 0 else 0.0
    # HBM bytes per launch: the counters' bytes per expanded node (tracked summary) times the
    # expansions of this run's launches, so that it describes the same launch as the algorithmic bytes
    traffic = None
    if "hbm_bytes_per_expansion" in tracked:
        traffic = float(tracked["hbm_bytes_per_expansion"]) * expansions_per_launch
    roofline = {"bound": "hbm", "kernel": "k_geodesic", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": achieved / HBM_PEAK_GBS,
                "measured_copy_gbs": copy_gbs, "frac_of_measured_copy": achieved / copy_gbs,
                "traffic": traffic,
                "traffic_source": (os.path.relpath(COUNTER_SUMMARY, ROOT) + " @ " + tracked.get("commit", "?") +
                                   ": bytes per expanded node x this run's expanded nodes per launch") if traffic else None,
                "traffic_over_algorithmic": traffic / (geo_bytes / P) if traffic else None,
                "dominant_kernel_by_time": dominant,
                "kernel_ms_per_step": kt, "kernel_ms_steps": P, "algorithmic_bytes_per_step": geo_bytes / P,
                "expanded_nodes_per_launch": expansions_per_launch, "expanded_nodes_per_s": expansions_per_s}
    if "valu_insts_per_expansion" in tracked:
        # what actually bounds the kernel: instructions issued against what the chip can issue.  A CU
        # issues at most one vector instruction of a wavefront per cycle (four SIMDs, each taking four
        # cycles per 64-lane instruction) and at most one scalar-unit instruction (scalar ALU or branch).
        v = float(tracked["valu_insts_per_expansion"])
        roofline["valu_issue"] = {"insts_per_expanded_node": v, "achieved": expansions_per_s * v, "peak": ISSUE_PEAK,
                                  "unit": "wavefront instructions/s", "frac": expansions_per_s * v / ISSUE_PEAK}
        if "scalar_insts_per_expansion" in tracked:
            sc = float(tracked["scalar_insts_per_expansion"])
            roofline["scalar_issue"] = {"insts_per_expanded_node": sc, "achieved": expansions_per_s * sc, "peak": ISSUE_PEAK,
                                        "unit": "wavefront instructions/s (scalar ALU + branch)",
                                        "frac": expansions_per_s * sc / ISSUE_PEAK}
    gen.close()
    result = {
        "metric": METRIC, "value": N * K / elapsed, "unit": "agent-steps/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": elapsed / K * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"C4: {N} agents / {S} corridor-maze scenes (~30k polygons each), geodesic 15-40 m, "
                               f"P(forward)={p_forward}, auto-reset", "agents": N, "scenes": S,
                   "settle_steps": args.settle, "stepping": "stream-ordered (step_end does not wait; one device "
                                                            "synchronization after the timed steps)"},
        "ms_per_step_hip_events": elapsed_events / K * 1e3,
        "host_synchronous": {"ms_per_step": sync_elapsed / K * 1e3, "value": N * K / sync_elapsed,
                             "stepping": "step_end waits for the device in every step"},
        "after_reset": after_reset,
        "roofline": roofline,
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(workload, N // S, seed, p_forward, require_ref=args.require_ref,
                                              threads=args.cpu_threads, settle=args.settle)
        result["speedup_vs_cpu_baseline"] = result["value"] / result["cpu_baseline"]["value"]
        result["host_synchronous"]["speedup_vs_cpu_baseline"] = result["host_synchronous"]["value"] / result["cpu_baseline"]["value"]
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
