"""GPU: the allocation-free geodesic entry point (bpsx_geodesic_static) against bpsx_geodesic.

The entry point takes device pointers, enqueues on the caller's stream and keeps its queue and
A* node pools in an array that lives in the library's device image, so a caller that must not
allocate (graph capture, serving loops) can use it.  Its distances must equal bpsx_geodesic's
bit for bit, also on a second call with a smaller input that finds the previous call's
contents in the array.
"""
import numpy as np
import pytest

from tests import common

pytestmark = pytest.mark.gpu


def test_static_geodesic_matches_the_allocating_entry_point(oracle):
    import torch
    from bps_nav_amd import scenes
    from bps_nav_amd.bps_sim import PointNavRolloutGenerator
    from oracle import bpo
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    print("case: allocation-free geodesic entry point", flush=True)
    blobs = [scenes.config_scene(4, 3), scenes.config_scene(2, 1)]
    gen = PointNavRolloutGenerator("", "", 2, 2, scenes=[(b, np.zeros((1, 10), np.float32)) for b in blobs], seed=1)
    for scene, blob in enumerate(blobs):
        nav = bpo.Nav(oracle, blob)
        pts = scenes.sample_points(blob, 21 + scene, 2 * 3000)
        x, r = gen.snap_points(scene, pts)
        assert (r != 0).all()
        for call, m in enumerate((3000, 700)):       # the second call is smaller and finds the first one's scratch contents
            a, ar = x[:m], r[:m]
            b, br = x[3000:3000 + m], r[3000:3000 + m]
            if call == 1:
                a, b = a[::-1].copy(), b.copy()      # other pairs than the first call's
                ar = ar[::-1].copy()
            want = gen.geodesic(scene, a, ar, b, br)
            t = lambda v, dt: torch.from_numpy(np.ascontiguousarray(v).view(dt)).cuda()  # noqa: E731
            out = torch.full((m,), -1.0, device="cuda")
            got = gen.geodesic_static(scene, t(a, np.float32), t(ar, np.int32), t(b, np.float32), t(br, np.int32), out=out)
            torch.cuda.synchronize()
            got = got.cpu().numpy()
            assert np.array_equal(common.bits(want), common.bits(got)), \
                f"scene {scene} call {call}: {(common.bits(want) != common.bits(got)).sum()} of {m} distances differ"
            assert np.isfinite(got).sum() > 100 and (got[np.isfinite(got)] > 0).any()   # maze-wide pairs mostly exhaust the 2048-node pool: inf
            if call == 0 and scene == 1:
                ref = nav.geodesic(a[:500], ar[:500], b[:500], br[:500])
                assert np.array_equal(common.bits(ref), common.bits(got[:500])), "differs from the oracle"
        nav.close()
    # ---- what the entry point is for: no allocation, and usable under stream capture
    blob = blobs[1]
    pts = scenes.sample_points(blob, 99, 2 * 500)
    x, r = gen.snap_points(1, pts)
    t = lambda v, dt: torch.from_numpy(np.ascontiguousarray(v).view(dt)).cuda()  # noqa: E731
    a, ar, b, br = t(x[:500], np.float32), t(r[:500], np.int32), t(x[500:], np.float32), t(r[500:], np.int32)
    want = gen.geodesic(1, x[:500], r[:500], x[500:], r[500:])
    out = torch.full((500,), -1.0, device="cuda")
    gen.geodesic_static(1, a, ar, b, br, out=out)           # warm: everything the call touches exists
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    reserved0 = torch.cuda.memory_reserved()
    for _ in range(3):
        gen.geodesic_static(1, a, ar, b, br, out=out)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0, "device memory in use changed across allocation-free calls"
    assert torch.cuda.memory_reserved() == reserved0
    assert np.array_equal(common.bits(want), common.bits(out.cpu().numpy()))
    # captured once into a HIP graph, replayed three times with eager work and synchronizations in
    # between and other inputs in the same buffers: every replay equals the allocating entry point
    graph = torch.cuda.CUDAGraph()
    out.fill_(-1.0)
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        gen.geodesic_static(1, a, ar, b, br, out=out)
    for rep in range(3):
        perm = np.random.default_rng(rep).permutation(500)
        xa, ra = x[:500][perm], r[:500][perm]
        a.copy_(t(xa, np.float32))
        ar.copy_(t(ra, np.int32))
        want = gen.geodesic(1, xa, ra, x[500:], r[500:])    # eager work of the library between replays
        out.fill_(-1.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        assert np.array_equal(common.bits(want), common.bits(got)), f"graph replay {rep} differs"
    del graph
    # limits and empty input
    z3 = torch.zeros((gen.STATIC_MAX_QUERIES + 1, 3), device="cuda")
    zr = torch.zeros(gen.STATIC_MAX_QUERIES + 1, dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="exceeds BPSX_STATIC_MAX_QUERIES"):
        gen.geodesic_static(0, z3, zr, z3, zr)
    assert gen.geodesic_static(0, z3[:0], zr[:0], z3[:0], zr[:0]).numel() == 0
    full = gen.geodesic_static(0, z3[:-1], zr[:-1], z3[:-1], zr[:-1])    # the maximum itself is accepted
    torch.cuda.synchronize()
    assert bool((full == 0).all())      # coincident points: distance 0 (PathFinder.cpp:528-541)
    gen.check_errors()
    gen.close()
