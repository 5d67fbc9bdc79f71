"""GPU measurement (not collected by pytest): what the path-search launch of a step waits for at
its end, on the benchmark workload (16384 agents / 128 maze scenes).

Needs the query-trace diagnostic build of the library, which records start, end, nodes expanded,
expected length and log replays of every search of a launch:

    make -C bps_nav_amd/csrc clean && make -C bps_nav_amd/csrc DIAG=-DBPSX_QUERY_TRACE OUT=../libbpsx_trace.so
    make -C bps_nav_amd/csrc clean && make -C bps_nav_amd/csrc         # the normal library again
    BPSX_LIBRARY=$PWD/bps_nav_amd/libbpsx_trace.so python tests/measure_launch_tail.py [steps, default 150]

Per step it takes the number of searches in flight over time (a wavefront serves one search at a
time, so this is the number of busy wavefronts) and prints, over the steps: the launch's length,
how long it ran with fewer than 10 % of its wavefronts busy, when the queue ran dry, and what the
last search to end was.
"""
import ctypes
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def main():
    import torch

    import bench
    from bps_nav_amd import _lib
    from bps_nav_amd.bps_sim import PointNavRolloutGenerator
    steps = int(sys.argv[1]) if len(sys.argv) > 1 else 150
    L = _lib.lib()
    if not hasattr(L, "bpsx_debug_trace"):
        print("this library has no query trace: build it with DIAG=-DBPSX_QUERY_TRACE and point BPSX_LIBRARY at it", file=sys.stderr)
        sys.exit(2)
    N, S, settle = 16384, 128, 120
    wl = bench.build_workload(S, 256)
    gen = PointNavRolloutGenerator("", "", N, S, gpu_id=0, scenes=wl, seed=3004)
    g = torch.Generator().manual_seed(3004)
    probs = torch.tensor([0.04, 0.8, 0.08, 0.08])
    acts = torch.multinomial(probs.expand(settle + steps, 4), N, replacement=True, generator=g).to(torch.int64).cuda()
    gen.reset(0)
    for t in range(settle):
        gen.step(0, acts[t])
    waves = None
    buf = np.zeros((1 << 17, 4), np.uint64)
    rows = []
    for t in range(settle, settle + steps):
        L.bpsx_debug_trace(None, 0)
        gen.step(0, acts[t])
        n = L.bpsx_debug_trace(ctypes.c_void_p(buf.ctypes.data), 1 << 17)
        tr = buf[:n].astype(np.int64)
        t0 = tr[:, 0].min()
        st, en = (tr[:, 0] - t0) / 100.0, (tr[:, 1] - t0) / 100.0      # microseconds (100 MHz clock)
        w = tr[:, 3]
        pred, rep = (w >> 8) & 0xffff, (w >> 24) & 0xfff
        pops = tr[:, 2]
        # searches in flight over time
        ev = np.concatenate([np.stack([st, np.ones(n)], 1), np.stack([en, -np.ones(n)], 1)])
        ev = ev[np.argsort(ev[:, 0], kind="stable")]
        busy = np.cumsum(ev[:, 1])
        if waves is None:
            waves = int(busy.max())
        end = en.max()
        below = busy < 0.1 * waves
        dt = np.diff(ev[:, 0], append=end)
        first_full = np.argmax(busy >= 0.9 * waves)
        under10 = float(dt[first_full:][below[first_full:]].sum())
        dry = float(st.max())                                        # the last search to begin: the queue is empty from here on
        k = int(np.argmax(en))
        ends = np.sort(en)
        rows.append((end, under10, dry, st[k], pops[k], pred[k], rep[k], ends[-2], ends[-10], ends[-50]))
    gen.close()
    R = np.array(rows, float)
    pct = lambda v: "mean %.0f, median %.0f, 90th percentile %.0f" % (v.mean(), np.median(v), np.percentile(v, 90))  # noqa: E731
    print(f"{steps} steps, {waves} wavefronts busy at most; microseconds from the launch's first search")
    print("launch length (first search begins -> last search ends): " + pct(R[:, 0]))
    print("of it with fewer than 10 % of the wavefronts busy: " + pct(R[:, 1]))
    print("queue dry (last search begins) at: " + pct(R[:, 2]))
    print("second-last, tenth-last, fiftieth-last search end before the last by: %.0f, %.0f, %.0f (means)"
          % ((R[:, 0] - R[:, 7]).mean(), (R[:, 0] - R[:, 8]).mean(), (R[:, 0] - R[:, 9]).mean()))
    replayed = R[:, 6] > 0
    print("last search to end replayed its operation log in %d of %d steps; those launches: %s; the others: %s"
          % (replayed.sum(), steps, pct(R[replayed, 0]) if replayed.any() else "-", pct(R[~replayed, 0]) if (~replayed).any() else "-"))
    under = (~replayed) & (R[:, 5] != 0xffff) & (R[:, 4] > R[:, 5] + 128)
    unknown = (~replayed) & (R[:, 5] == 0xffff)
    print("last search to end, where it did not replay: %d of unknown length, %d that expanded over 128 nodes more than expected, %d others"
          % (unknown.sum(), under.sum(), ((~replayed) & ~under & ~unknown).sum()))
    print("last search to end, where it replayed: began at %.0f, %.0f nodes (mean); where not: began at %.0f, %.0f nodes"
          % (R[replayed, 3].mean() if replayed.any() else 0, R[replayed, 4].mean() if replayed.any() else 0,
             R[~replayed, 3].mean() if (~replayed).any() else 0, R[~replayed, 4].mean() if (~replayed).any() else 0))
    print("time with fewer than a tenth of the wavefronts busy, launches whose last search replayed: %.0f (mean); the others: %.0f"
          % (R[replayed, 1].mean() if replayed.any() else 0, R[~replayed, 1].mean() if (~replayed).any() else 0))


if __name__ == "__main__":
    main()
