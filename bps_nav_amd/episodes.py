"""Episode tables for synthetic scenes: rows of 10 floats {start xyz, start rotation xyzw,
goal xyz}, the layout of struct Episode (simulator.cpp:83-87).  Mirrors what the reference's
offline generator does with habitat-sim (create_gibson_large_dataset.py:44-49): random
navigable start/goal pairs kept when their geodesic distance lies in a range."""
import numpy as np

from . import scenes


def yaw_quat(yaw):
    """Rotation by `yaw` radians about +y as quaternion x,y,z,w (f32[n,4])."""
    yaw = np.asarray(yaw, np.float64)
    q = np.zeros(yaw.shape + (4,), np.float32)
    q[..., 1] = np.sin(yaw / 2)
    q[..., 3] = np.cos(yaw / 2)
    return q


def make_episodes(navmesh_bytes, seed, count, dmin, dmax, geodesic_fn, max_rounds=64):
    """Draws start/goal pairs by area-weighted sampling and keeps those with
    dmin <= geodesic <= dmax.  geodesic_fn(starts f32[k,3], goals f32[k,3]) -> f32[k]
    (inf where unreachable); it decides which implementation measures the distance."""
    rng = np.random.default_rng(seed)
    rows = []
    have = 0
    for r in range(max_rounds):
        k = max(256, 4 * count)
        pts = scenes.sample_points(navmesh_bytes, seed * 1000003 + r, 2 * k)
        s, g = pts[:k], pts[k:]
        # bias towards pairs whose straight-line distance can fall inside the range
        e = np.linalg.norm((s - g)[:, [0, 2]], axis=1)
        keep = (e <= dmax) & (e >= 0.25 * dmin)
        s, g = s[keep], g[keep]
        if len(s) == 0:
            continue
        d = geodesic_fn(s, g)
        ok = np.isfinite(d) & (d >= dmin) & (d <= dmax)
        s, g = s[ok], g[ok]
        yaw = rng.uniform(0, 2 * np.pi, len(s))
        ep = np.concatenate([s, yaw_quat(yaw), g], axis=1).astype(np.float32)
        rows.append(ep)
        have += len(ep)
        if have >= count:
            break
    if have < count:
        raise RuntimeError(f"only {have} of {count} episodes found in geodesic range [{dmin},{dmax}]")
    return np.ascontiguousarray(np.concatenate(rows)[:count])


def random_actions(rng, shape, p_forward=None):
    """Action ids int64: uniform over {0,1,2,3} when p_forward is None, otherwise
    forward with p_forward, stop with 0.04 and the rest split between the turns."""
    if p_forward is None:
        return rng.integers(0, 4, shape).astype(np.int64)
    p_turn = (1.0 - p_forward - 0.04) / 2
    return rng.choice(4, size=shape, p=[0.04, p_forward, p_turn, p_turn]).astype(np.int64)
