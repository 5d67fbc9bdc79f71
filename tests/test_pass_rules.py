"""The rules by which the GPU kernel expands several open nodes of a path search in one pass
(bps_nav_amd/csrc/geodesic_device.h, astar_fast), checked on the CPU against the reference's
algorithm itself: the oracle's findPath (DetourNavMeshQuery.cpp:945-1137 restated, heap of
DetourNode.cpp:150-200) predicts before a pop which nodes its next pops will be and what their
expansions will write, by the kernel's rules and from the state as it is, and compares with
what it then does.  A rule that let a node through whose expansion depends on an earlier one's
would show as a wrong node or a wrong update."""
import numpy as np
import pytest

from bps_nav_amd import scenes
from oracle import bpo
from tests import common


@pytest.mark.parametrize("config,queries", [(1, 400), (2, 400), (3, 150), (4, 200)])
def test_predicted_passes_are_what_the_reference_does(oracle, config, queries):
    blob = scenes.config_scene(config, 0)
    nav = bpo.Nav(oracle, blob)
    pts = scenes.sample_points(blob, 11, 2 * queries)
    x, r = nav.snap(pts)
    ok = r != 0
    x, r = x[ok], r[ok]
    m = len(x) // 2
    plain = nav.geodesic(x[:m], r[:m], x[m:2 * m], r[m:2 * m])
    nav.pass_check(8)
    checked = nav.geodesic(x[:m], r[:m], x[m:2 * m], r[m:2 * m])
    st = nav.pass_check(0)
    nav.close()
    assert np.array_equal(common.bits(plain), common.bits(checked))   # the check changes nothing
    assert st["wrong_node"] == 0 and st["wrong_update"] == 0, st
    assert st["nodes"] > 50 * m and st["nodes"] > 2.2 * st["passes"], st     # the rules do let several nodes through
    if config >= 2:
        assert st["pairs"] > 0, st       # equal totals at the front occurred and were taken as pairs
    print(f"config {config}: {st}, {st['nodes'] / st['passes']:.2f} nodes per pass")


def test_single_row_is_the_plain_search(oracle):
    """With one row a pass is one pop: every prediction is the heap's minimum, ties are left alone."""
    blob = scenes.config_scene(2, 1)
    nav = bpo.Nav(oracle, blob)
    pts = scenes.sample_points(blob, 3, 200)
    x, r = nav.snap(pts)
    nav.pass_check(1)
    nav.geodesic(x[:100], r[:100], x[100:], r[100:])
    st = nav.pass_check(0)
    nav.close()
    assert st["wrong_node"] == 0 and st["wrong_update"] == 0 and st["pairs"] == 0
    assert st["nodes"] == st["passes"] > 0


@pytest.mark.parametrize("dropped,what", [(0x100, "wrong_node"), (0x200, "wrong_update")])
def test_each_rule_is_needed(oracle, dropped, what):
    """The check has teeth: without the rule on totals (an earlier row's update at or below a later
    row's total ends the pass there) the predicted nodes go wrong, and without the rule on
    polygons (no row reads what an earlier row writes) the predicted updates do."""
    blob = scenes.config_scene(2, 0)
    nav = bpo.Nav(oracle, blob)
    pts = scenes.sample_points(blob, 11, 400)
    x, r = nav.snap(pts)
    nav.pass_check(8 | dropped)
    nav.geodesic(x[:200], r[:200], x[200:], r[200:])
    st = nav.pass_check(0)
    nav.close()
    assert st[what] > 0, st
