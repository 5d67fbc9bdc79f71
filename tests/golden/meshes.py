"""Hand-made navmeshes with closed-form answers, shared by the golden-vector generator and
the tests.  Coordinates are in voxels of 0.05 m (20 per metre)."""
import numpy as np

from bps_nav_amd import scenes

M = 20  # voxels per metre


def _rects_to_mesh(rects, heights=None):
    """rects: list of (x0, z0, x1, z1) in metres, edge-adjacent rectangles sharing full edges.
    heights: optional {(x, z) metres: y in voxels} for sloped vertices."""
    verts, vid, polys = [], {}, []

    def v(x, z):
        key = (round(x * M), round(z * M))
        if key not in vid:
            y = 0 if heights is None else heights.get((x, z), 0)
            vid[key] = len(verts)
            verts.append((key[0], y, key[1]))
        return vid[key]

    for (x0, z0, x1, z1) in rects:
        polys.append([v(x0, z0), v(x0, z1), v(x1, z1), v(x1, z0)])
    # neighbour = polygon owning the reversed edge
    edge = {}
    for i, p in enumerate(polys):
        for j in range(len(p)):
            edge[(p[j], p[(j + 1) % len(p)])] = i
    neis = [[edge.get((p[(j + 1) % len(p)], p[j]), -1) for j in range(len(p))] for p in polys]
    return scenes.navmesh_from_polys(np.array(verts), polys, neis)


def l_shape():
    """[0,10]x[0,5] + [0,5]x[5,10] as three 5 m squares; inner corner at (5, 5)."""
    return _rects_to_mesh([(0, 0, 5, 5), (5, 0, 10, 5), (0, 5, 5, 10)])


def u_shape():
    """Two 3 m x 9 m legs joined by a 3 m x 3 m bridge at the bottom; inner corners (3,3), (6,3)."""
    return _rects_to_mesh([(0, 0, 3, 3), (0, 3, 3, 9), (3, 0, 6, 3), (6, 0, 9, 3), (6, 3, 9, 9)])


def two_rooms():
    """Two 4 m rooms joined by a 1 m doorway through a 0.5 m wall; walls elsewhere."""
    return _rects_to_mesh([(0, 0, 4, 1.5), (0, 1.5, 4, 2.5), (0, 2.5, 4, 4), (4, 1.5, 4.5, 2.5),
                           (4.5, 0, 8.5, 1.5), (4.5, 1.5, 8.5, 2.5), (4.5, 2.5, 8.5, 4)])


def ramp():
    """Flat 4 m square, then a 4 m ramp rising 2 m, then a flat upper 4 m square."""
    h = {(8, 0): 40, (8, 4): 40, (12, 0): 40, (12, 4): 40}
    return _rects_to_mesh([(0, 0, 4, 4), (4, 0, 8, 4), (8, 0, 12, 4)], heights=h)


def islands():
    """Two disconnected 3 m squares 1 m apart."""
    return _rects_to_mesh([(0, 0, 3, 3), (4, 0, 7, 3)])


ALL = {"l_shape": l_shape, "u_shape": u_shape, "two_rooms": two_rooms, "ramp": ramp, "islands": islands}
