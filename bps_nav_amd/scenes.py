"""Synthetic floor plans and navmesh packing (host side of libbpsx).

These stand in for the Gibson/MP3D ".navmesh" files that the reference loads
(simulator.cpp:1712-1730); the bytes produced are the same MSET/Detour format.
"""
import ctypes as C

import numpy as np

from . import _lib

BOX_ROOM, ROOMS, MAZE = 0, 1, 2


def gen_scene(kind, seed, cell=5, **kw):
    """Returns the bytes of a single-tile ".navmesh". kw: fields of bpsx_scene_params."""
    L = _lib.lib()
    p = _lib.SceneParams()
    p.kind, p.seed, p.cell = kind, seed, cell
    origin = kw.pop("origin", (0.0, 0.0, 0.0))
    p.origin = (C.c_float * 3)(*origin)
    for k, v in kw.items():
        if not hasattr(p, k):
            raise TypeError(f"unknown scene parameter {k}")
        setattr(p, k, v)
    out, size = C.c_void_p(), C.c_size_t()
    _lib.check(L.bpsx_gen_scene(C.byref(p), C.byref(out), C.byref(size)))
    try:
        return C.string_at(out, size.value)
    finally:
        L.bpsx_free(out)


def sample_points(navmesh_bytes, seed, n):
    """Area-weighted random points on the walkable polygons: f32[n,3]."""
    out = np.zeros((n, 3), np.float32)
    _lib.check(_lib.lib().bpsx_sample_points(navmesh_bytes, len(navmesh_bytes), seed, n, out.ctypes.data))
    return out


def pack_tile(verts, polys, flags=None, areas=None, bmin=(0, 0, 0), bmax=None, cs=0.05, ch=0.05,
              walkable_height=0.88, walkable_radius=0.18, walkable_climb=0.2, nvp=6):
    """Packs one Detour tile from a quantised polygon soup (layout of dtNavMeshCreateParams)."""
    L = _lib.lib()
    verts = np.ascontiguousarray(verts, np.uint16).reshape(-1, 3)
    polys = np.ascontiguousarray(polys, np.uint16).reshape(-1, 2 * nvp)
    npoly = len(polys)
    flags = np.ascontiguousarray(flags if flags is not None else np.full(npoly, 1), np.uint16)
    areas = np.ascontiguousarray(areas if areas is not None else np.zeros(npoly), np.uint8)
    if bmax is None:
        bmax = (bmin[0] + float(verts[:, 0].max()) * cs, bmin[1] + float(verts[:, 1].max()) * ch + 1.0,
                bmin[2] + float(verts[:, 2].max()) * cs)
    d = _lib.TileDesc()
    d.verts, d.vert_count = verts.ctypes.data, len(verts)
    d.polys, d.poly_flags, d.poly_areas, d.poly_count = polys.ctypes.data, flags.ctypes.data, areas.ctypes.data, npoly
    d.nvp = nvp
    d.walkable_height, d.walkable_radius, d.walkable_climb = walkable_height, walkable_radius, walkable_climb
    d.bmin = (C.c_float * 3)(*bmin)
    d.bmax = (C.c_float * 3)(*bmax)
    d.cs, d.ch = cs, ch
    d.build_bv_tree = 1
    out, size = C.c_void_p(), C.c_size_t()
    _lib.check(L.bpsx_pack_tile(C.byref(d), C.byref(out), C.byref(size)))
    try:
        return C.string_at(out, size.value)
    finally:
        L.bpsx_free(out)


def pack_mset(tile, orig, tile_width, tile_height, max_polys):
    """Wraps one tile blob into MSET bytes the way a solo-mesh dtNavMesh saves it."""
    L = _lib.lib()
    buf = C.create_string_buffer(tile, len(tile))
    tiles = (C.c_void_p * 1)(C.cast(buf, C.c_void_p))
    sizes = (C.c_size_t * 1)(len(tile))
    o = (C.c_float * 3)(*orig)
    out, size = C.c_void_p(), C.c_size_t()
    _lib.check(L.bpsx_pack_mset(tiles, sizes, 1, o, tile_width, tile_height, 1, max_polys, C.byref(out), C.byref(size)))
    try:
        return C.string_at(out, size.value)
    finally:
        L.bpsx_free(out)


def navmesh_from_polys(verts_cells, polys, neis, bmin=(0.0, 0.0, 0.0), cs=0.05, ch=0.05, flags=None):
    """Hand-made single-tile navmesh: verts_cells int[nv,3] in voxel units, polys = lists of
    vertex ids (3..6 each), neis = per-polygon lists of neighbour polygon id or -1 per edge."""
    nvp = 6
    pk = np.full((len(polys), 2 * nvp), 0xFFFF, np.uint16)
    for i, (p, nb) in enumerate(zip(polys, neis)):
        for j, v in enumerate(p):
            pk[i, j] = v
            pk[i, nvp + j] = 0xFFFF if nb[j] < 0 else nb[j]
    verts_cells = np.asarray(verts_cells)
    bmax = (bmin[0] + float(verts_cells[:, 0].max()) * cs, bmin[1] + float(verts_cells[:, 1].max()) * ch + 1.0,
            bmin[2] + float(verts_cells[:, 2].max()) * cs)
    tile = pack_tile(verts_cells, pk, flags=flags, bmin=bmin, bmax=bmax, cs=cs, ch=ch)
    return pack_mset(tile, bmin, bmax[0] - bmin[0], bmax[2] - bmin[2], len(polys))


# The benchmark configurations, as scene-generator arguments.
def config_scene(config, scene_idx):
    """Scene `scene_idx` of benchmark configuration `config` (1..4)."""
    seed = 1000 + scene_idx
    if config == 1:
        return gen_scene(BOX_ROOM, seed, cell=5, size_x=10.0, size_z=10.0, num_boxes=8, box_min=0.5, box_max=2.0,
                         tri_frac=0.2, hex_frac=0.1)
    if config == 2:
        return gen_scene(ROOMS, seed, cell=6, rooms_min=4, rooms_max=8, room_min=3.0, room_max=6.0, door_width=0.9,
                         wall=0.3, clutter_frac=0.0, tri_frac=0.1, hex_frac=0.1)
    if config == 3:
        return gen_scene(ROOMS, seed, cell=4, rooms_min=10, rooms_max=25, room_min=5.0, room_max=7.0,
                         door_width=0.9, wall=0.2, clutter_frac=0.15, box_min=0.5, box_max=1.5, tri_frac=0.1,
                         hex_frac=0.1)
    if config == 4:
        # 0.5 m cells keep A* inside Detour's 2048-node pool and 256-polygon corridor limit for
        # the 15-40 m episodes of this configuration (finer cells make the reference return inf)
        return gen_scene(MAZE, seed, cell=10, maze_w=50, maze_h=50, corridor_min=1.0, corridor_max=1.5, wall=1.0,
                         braid=0.08, tri_frac=0.05, hex_frac=0.05)
    raise ValueError("config must be 1..4")
