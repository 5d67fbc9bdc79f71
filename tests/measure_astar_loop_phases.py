"""Measurement (not collected by pytest): where the instructions and the cycles of the A* kernel's
sorted-list loop go, phase by phase.

Both parts use the phase-timing diagnostic build (-DBPSX_PHASE_TIMING), whose loop carries eleven
marks: 0 front of the list, 1 fetch of the edge records and the expanded nodes, 2 node lookup,
3 costs, 4 rows that stand, 5 closing, 6 new nodes, 7 stores, 8 front entries leave and the log,
9 list updates, 10 end of the pass.

    python tests/measure_astar_loop_phases.py
        No GPU needed.  Compiles kernels.hip to assembly with the Makefile's own options and counts,
        for the loop's most used instantiation (links in LDS, list in one register pair) inside
        k_geodesic, the instructions between consecutive marks in the order the compiler laid them
        out, by class: vector ALU, scalar ALU, branch, LDS, memory, waits.  Blocks that the compiler
        moved out of line (rare cases) are counted where they lie, and a loop inside a phase (the
        list updates, one per updated node) is counted once: the figures are those of the code,
        not of its execution.

    make -C bps_nav_amd/csrc clean && make -C bps_nav_amd/csrc DIAG=-DBPSX_PHASE_TIMING OUT=../libbpsx_phase.so
    make -C bps_nav_amd/csrc clean && make -C bps_nav_amd/csrc         # the normal library again
    BPSX_LIBRARY=$PWD/bps_nav_amd/libbpsx_phase.so python tests/measure_astar_loop_phases.py --cycles [steps, default 50]
        On the GPU: cycles per expanded node in each phase (the wavefront's own clock, so time spent
        waiting for the other wavefronts of its SIMD is included), on the benchmark workload.
"""
import os
import re
import subprocess
import sys
import tempfile

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "bps_nav_amd", "csrc")
PHASES = ["front of the list", "fetch", "node lookup", "costs", "rows that stand", "closing", "new nodes", "stores",
          "front leaves, log", "list updates (once)", "end of pass, loop top"]


def classify(line):
    s = line.strip()
    if not s or s.startswith(";") or s.startswith(".") or s.endswith(":"):
        return None
    op = s.split()[0]
    if op.startswith("s_cbranch") or op.startswith("s_branch"):
        return "branch"
    if op.startswith("s_waitcnt") or op.startswith("s_nop"):
        return "wait"
    if op.startswith("s_load") or op.startswith("s_buffer") or op.startswith("s_memtime") or op.startswith("s_memrealtime"):
        return "smem"
    if op.startswith("s_"):
        return "salu"
    if op.startswith("v_"):
        return "valu"
    if op.startswith("ds_"):
        return "lds"
    if op.split("_")[0] in ("global", "flat", "scratch", "buffer"):
        return "mem"
    return "other"


def static_counts():
    line = subprocess.run(["make", "-C", CSRC, "-n", "-B", "kernels.o", "DIAG=-DBPSX_PHASE_TIMING"], check=True,
                          capture_output=True, text=True).stdout
    cmd = [l for l in line.splitlines() if "hipcc" in l and "kernels.hip" in l][0].split()
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "kernels.s")
        i = cmd.index("-c")
        cmd = cmd[:i] + ["--cuda-device-only", "-S", os.path.join(CSRC, "kernels.hip"), "-o", out]
        subprocess.run(cmd, check=True, cwd=CSRC, stderr=subprocess.DEVNULL)
        text = open(out).read().split("\n")
    start = [i for i, l in enumerate(text) if re.match(r"_ZN4bpsx\S*10k_geodesicE\S*:", l)][0]
    end = start + [i for i, l in enumerate(text[start:]) if l.startswith(".Lfunc_end")][0]
    body = text[start:end]
    marks = {}
    for i, l in enumerate(body):
        m = re.search(r"; astar_fast spill=0 pairs=1 mark=(\d+)", l)
        if m:
            marks[int(m.group(1))] = i
    assert sorted(marks) == list(range(11)), "marks of the loop not found in the assembly"
    # the pass's end: from mark 10 to the loop's backward branch (the last branch to a label above mark 0
    # before the next instantiation's first mark), plus the loop top (from its header label to mark 0)
    header = max(i for i in range(marks[0]) if re.match(r"\.LBB\d+_\d+:.*Parent Loop", body[i]))
    rows = []
    for k in range(10):
        rows.append((PHASES[k], body[marks[k]:marks[k + 1]]))
    tail_end = marks[10]
    while tail_end < len(body) and "astar_fast spill" not in body[tail_end + 1]:
        tail_end += 1
        if re.match(r"\s*s_c?branch\S*\s+" + re.escape(body[header].split(":")[0]) + r"\b", body[tail_end]):
            break
    rows.append((PHASES[10], body[marks[10]:tail_end + 1] + body[header:marks[0]]))
    classes = ["valu", "salu", "branch", "lds", "mem", "smem", "wait"]
    print("instructions between the marks of astar_fast<links in LDS, one register pair> in k_geodesic, as laid out by the compiler")
    print("%-26s" % "phase" + "".join("%8s" % c for c in classes))
    total = dict.fromkeys(classes, 0)
    for name, lines in rows:
        c = dict.fromkeys(classes, 0)
        for l in lines:
            t = classify(l)
            if t in c:
                c[t] += 1
        for k in classes:
            total[k] += c[k]
        print("%-26s" % name + "".join("%8d" % c[k] for k in classes))
    print("%-26s" % "all" + "".join("%8d" % total[k] for k in classes))


def cycles(steps):
    import torch

    sys.path.insert(0, ROOT)
    import bench
    from bps_nav_amd.bps_sim import PointNavRolloutGenerator
    N, S, settle = 16384, 128, 120
    wl = bench.build_workload(S, 256)
    gen = PointNavRolloutGenerator("", "", N, S, gpu_id=0, scenes=wl, seed=3004)
    g = torch.Generator().manual_seed(3004)
    probs = torch.tensor([0.04, 0.8, 0.08, 0.08])
    acts = torch.multinomial(probs.expand(settle + steps, 4), N, replacement=True, generator=g).to(torch.int64).cuda()
    gen.reset(0)
    for t in range(settle):
        gen.step(0, acts[t])
    c0 = gen.counters()
    for t in range(settle, settle + steps):
        gen.step(0, acts[t])
    c1 = gen.counters()
    gen.close()
    d = [float(a - b) for a, b in zip(c1["phase_cycles"][:8], c0["phase_cycles"][:8])]
    if not sum(d):
        print("this library counts no phase cycles: build it with DIAG=-DBPSX_PHASE_TIMING and point BPSX_LIBRARY at it", file=sys.stderr)
        sys.exit(2)
    pops = float(c1["astar_pops"] - c0["astar_pops"])
    passes = d[7]
    names = ["front of the list (marks 0-1)", "fetch (1-2)", "node lookup (2-3)", "costs (3-4)", "rows that stand (4-5)",
             "closing, new nodes, stores (5-8)", "front leaves, log, list updates (8-10)"]
    print(f"{steps} steps: {pops / steps:.0f} nodes expanded per step in {passes / steps:.0f} passes ({pops / passes:.2f} nodes per pass)")
    tot = sum(d[:7])
    for n, v in zip(names, d[:7]):
        print(f"{n:42s} {v / passes:8.0f} cycles per pass {v / pops:8.0f} per node {100 * v / tot:6.1f} %")
    print(f"{'all (the loop top and the marks themselves excluded)':42s} {tot / passes:8.0f} cycles per pass {tot / pops:8.0f} per node")


if __name__ == "__main__":
    if len(sys.argv) > 1 and sys.argv[1] == "--cycles":
        cycles(int(sys.argv[2]) if len(sys.argv) > 2 else 50)
    else:
        static_counts()
