"""CPU: the goal-rooted distance-field formulation of the geodesic (oracle side only, not the
reference's algorithm) against the reference's A*: equal where the mathematics says so, and
measurably different on the benchmark scenes, which is why the engine runs the A*."""
import numpy as np

from tests import common
from tests.golden import meshes
from tests.measure_field_vs_astar import measure


def field(oracle, nav, a, ar, b, br):
    import ctypes as C
    f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
    u32p = np.ctypeslib.ndpointer(np.uint32, flags="C_CONTIGUOUS")
    oracle.L.bpo_nav_geodesic_field.argtypes = [C.c_void_p, f32p, u32p, f32p, u32p, C.c_uint32, f32p]
    out = np.zeros(len(a), np.float32)
    oracle.L.bpo_nav_geodesic_field(nav.h, np.ascontiguousarray(a, np.float32), np.ascontiguousarray(ar, np.uint32),
                                    np.ascontiguousarray(b, np.float32), np.ascontiguousarray(br, np.uint32), len(a), out)
    return out


def test_field_equals_astar_where_the_corridor_is_forced(oracle):
    """On the hand-made L and U shapes every pair of points has one corridor: both formulations
    string-pull the same polygons and give the same bits.  Islands stay unreachable."""
    from oracle import bpo
    for name in ("l_shape", "u_shape", "islands"):
        blob = meshes.ALL[name]()
        nav = bpo.Nav(oracle, blob)
        from bps_nav_amd import scenes
        x, r = nav.snap(scenes.sample_points(blob, 3, 200))
        a, ar, b, br = x[:100], r[:100], x[100:], r[100:]
        want = nav.geodesic(a, ar, b, br)
        got = field(oracle, nav, a, ar, b, br)
        assert np.array_equal(np.isinf(want), np.isinf(got))
        fin = np.isfinite(want)
        assert np.allclose(got[fin], want[fin], rtol=1e-6), name
        if name != "islands":
            assert np.array_equal(common.bits(want), common.bits(got)), name


def test_field_differs_from_astar_on_benchmark_scenes(oracle):
    """On room plans and mazes most polygons can be reached through several corridors; the
    field's choice differs from A*'s for most goal -> agent pairs and the string-pulled lengths
    differ by percents: far above the 1e-3 the distance is allowed to be off."""
    for config, dmax in ((2, 30.0), (4, 40.0)):
        rel, _ = measure(oracle, config, 1, 6, 60 * (14 if config == 4 else 1), 1.0, dmax, 500 + config)
        assert len(rel) > 150
        assert (rel > 1e-3).mean() > 0.5, f"config {config}: only {(rel > 1e-3).mean():.2f} of the pairs differ by more than 1e-3"
        assert np.median(rel[np.isfinite(rel)]) > 2e-3
