"""CPU: the C-ABI library loads and exports every symbol include/bpsx.h declares; the
host-side pieces (packer, generator, dataset reader) behave; no GPU call is made."""
import ctypes
import gzip
import json
import os
import re
import struct
import subprocess
import zlib

import numpy as np
import pytest

from bps_nav_amd import _lib, scenes
from oracle import bpo
from tests import common
from tests.golden import meshes

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    hdr = open(os.path.join(ROOT, "include", "bpsx.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    names = set(re.findall(r"\b(bpsx_[a-z_0-9]+)\s*\(", hdr))
    assert len(names) >= 25
    L = ctypes.CDLL(_lib.LIB_PATH)
    missing = [n for n in sorted(names) if not hasattr(L, n)]
    assert not missing, f"libbpsx.so lacks {missing}"
    # ... and nothing else: no C++ internals, no template instantiations (one .so, C ABI only)
    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = {ln.split()[-1] for ln in out.splitlines() if ln.strip()}
    extra = sorted(exported - names)
    assert not extra, f"libbpsx.so exports symbols that include/bpsx.h does not declare: {extra[:10]}"


def test_generator_is_deterministic_and_seed_sensitive():
    a = scenes.config_scene(2, 5)
    assert a == scenes.config_scene(2, 5)
    assert a != scenes.config_scene(2, 6)
    # MSET container invariants: magic, one tile, maxPolys == polyCount (solo-mesh convention)
    magic, version, ntiles = struct.unpack_from("<iii", a, 0)
    assert magic == 0x4D534554 and version == 1 and ntiles == 1
    max_tiles, max_polys = struct.unpack_from("<ii", a, 32)
    poly_count = struct.unpack_from("<i", a, 48 + 24)[0]
    assert max_tiles == 1 and max_polys == poly_count
    tile_ref, size = struct.unpack_from("<Ii", a, 40)
    assert size == len(a) - 48 and tile_ref == 1 << (poly_count - 1).bit_length()


@pytest.mark.parametrize("config,lo,hi", [(1, 1200, 2400), (2, 500, 4000), (3, 5000, 30000), (4, 26000, 32767)])
def test_config_scene_sizes(config, lo, hi):
    n = struct.unpack_from("<i", scenes.config_scene(config, 1), 48 + 24)[0]
    assert lo <= n <= hi


def test_packer_rejects_bad_input():
    verts = np.array([[0, 0, 0], [0, 0, 10], [10, 0, 10]], np.uint16)
    poly = np.full((1, 12), 0xFFFF, np.uint16)
    poly[0, :3] = (0, 1, 2)
    scenes.pack_tile(verts, poly)  # fine
    bad = poly.copy()
    bad[0, 2] = 9
    with pytest.raises(RuntimeError, match="vertex index out of range"):
        scenes.pack_tile(verts, bad)
    bad = poly.copy()
    bad[0, 6] = 3
    with pytest.raises(RuntimeError, match="neighbour index out of range"):
        scenes.pack_tile(verts, bad)
    with pytest.raises(RuntimeError, match="fewer than 3"):
        two = poly.copy()
        two[0, 2] = 0xFFFF
        scenes.pack_tile(verts, two)
    with pytest.raises(RuntimeError, match="unknown kind"):
        scenes.gen_scene(9, 1)


def test_packer_matches_reference_builder_bytes(reflib):
    """bpsx_pack_tile against dtCreateNavMeshData (DetourNavMeshBuilder.cpp:280-658) on the same
    polygon soup: identical bytes, BV tree included."""
    if reflib is None:
        pytest.skip("compiled reference not available outside the development container")
    rng = np.random.default_rng(4)
    # a random conforming soup: grid of squares, some split into triangles, random heights
    nx, nz = 17, 13
    vid = lambda x, z: z * (nx + 1) + x  # noqa: E731
    verts = np.array([[x * 5, int(rng.integers(0, 6)), z * 5] for z in range(nz + 1) for x in range(nx + 1)], np.uint16)
    polys, owner = [], {}
    for z in range(nz):
        for x in range(nx):
            if rng.random() < 0.15:
                continue
            if rng.random() < 0.3:
                polys.append([vid(x, z), vid(x, z + 1), vid(x + 1, z + 1)])
                polys.append([vid(x, z), vid(x + 1, z + 1), vid(x + 1, z)])
            else:
                polys.append([vid(x, z), vid(x, z + 1), vid(x + 1, z + 1), vid(x + 1, z)])
    for i, p in enumerate(polys):
        for j in range(len(p)):
            owner[(p[j], p[(j + 1) % len(p)])] = i
    pk = np.full((len(polys), 12), 0xFFFF, np.uint16)
    for i, p in enumerate(polys):
        for j in range(len(p)):
            pk[i, j] = p[j]
            nb = owner.get((p[(j + 1) % len(p)], p[j]), -1)
            pk[i, 6 + j] = 0xFFFF if nb < 0 else nb
    flags = np.where(rng.random(len(polys)) < 0.9, 1, 4).astype(np.uint16)
    areas = rng.integers(0, 3, len(polys)).astype(np.uint8)
    bmin = np.array([1.5, -0.25, -3.0], np.float32)
    bmax = np.array([1.5 + nx * 5 * 0.05, 1.0, -3.0 + nz * 5 * 0.05], np.float32)
    mine = scenes.pack_tile(verts, pk, flags=flags, areas=areas, bmin=tuple(bmin), bmax=tuple(bmax), cs=0.05, ch=0.1)
    buf = np.zeros(len(mine) + 4096, np.uint8)
    size = reflib.L.bpo_ref_create_tile(verts.reshape(-1), len(verts), pk.reshape(-1), flags, areas, len(polys), 6,
                                        0.88, 0.18, 0.2, bmin, bmax, 0.05, 0.1, buf, len(buf))
    assert size == len(mine)
    assert bytes(buf[:size]) == mine


def test_packer_matches_reference_builder_with_portal_edges(reflib):
    """Tile-border portal codes (0x8000 | dir) go through the same neis mapping and link budget
    as dtCreateNavMeshData (DetourNavMeshBuilder.cpp:381-396, 497-515)."""
    if reflib is None:
        pytest.skip("compiled reference not available outside the development container")
    verts = np.array([[0, 0, 0], [0, 0, 20], [20, 0, 20], [20, 0, 0], [40, 0, 20], [40, 0, 0]], np.uint16)
    pk = np.full((2, 12), 0xFFFF, np.uint16)
    pk[0, :4] = (0, 1, 2, 3)
    pk[0, 6:10] = (0x8000, 0x8001, 1, 0x8003)      # x-, z+ portals, neighbour 1, z- portal
    pk[1, :4] = (3, 2, 4, 5)
    pk[1, 6:10] = (0, 0x8001, 0x8002, 0xFFFF)      # neighbour 0, z+ portal, x+ portal, wall
    bmin, bmax = np.array([0, 0, 0], np.float32), np.array([2, 1, 1], np.float32)
    mine = scenes.pack_tile(verts, pk, bmin=tuple(bmin), bmax=tuple(bmax))
    buf = np.zeros(len(mine) + 1024, np.uint8)
    size = reflib.L.bpo_ref_create_tile(verts.reshape(-1), 6, pk.reshape(-1), np.ones(2, np.uint16), np.zeros(2, np.uint8),
                                        2, 6, 0.88, 0.18, 0.2, bmin, bmax, 0.05, 0.05, buf, len(buf))
    assert size == len(mine) and bytes(buf[:size]) == mine


def test_generator_can_tile_a_scene():
    one = scenes.gen_scene(scenes.BOX_ROOM, 5, 5, size_x=10.0, size_z=10.0, num_boxes=4, box_min=0.5, box_max=2.0)
    four = scenes.gen_scene(scenes.BOX_ROOM, 5, 5, size_x=10.0, size_z=10.0, num_boxes=4, box_min=0.5, box_max=2.0,
                            tiles_x=2, tiles_z=2)
    assert struct.unpack_from("<i", one, 8)[0] == 1 and struct.unpack_from("<i", four, 8)[0] == 4
    # same floor: the polygon counts of the four tiles add up to the single tile's
    off, total = 40, 0
    for _ in range(4):
        ref, size = struct.unpack_from("<Ii", four, off)
        total += struct.unpack_from("<i", four, off + 8 + 24)[0]
        off += 8 + size
    assert off == len(four) and total == struct.unpack_from("<i", one, 48 + 24)[0]


def test_oracle_rejects_multi_tile_meshes(oracle):
    # the reference's PathFinder is undefined on them (refs built with salt and tile swapped,
    # PathFinder.cpp:67, 318), so neither the oracle nor the engine accepts them
    four = scenes.gen_scene(scenes.BOX_ROOM, 5, 5, size_x=10.0, size_z=10.0, num_boxes=4, box_min=0.5, box_max=2.0,
                            tiles_x=2, tiles_z=2)
    with pytest.raises(RuntimeError, match="multi-tile"):
        bpo.Nav(oracle, four)


def test_packed_tile_matches_fixture_bytes():
    # pins the packer (tile layout, BV tree, MSET header) where the reference builder is absent:
    # the fixture's navmesh bytes were loaded and queried by the compiled reference
    for name, fn in meshes.ALL.items():
        want = np.load(os.path.join(ROOT, "tests", "golden", f"mesh_{name}.npz"))["blob"].tobytes()
        assert fn() == want, name


def test_dataset_reader_round_trip(tmp_path):
    from bps_nav_amd.bps_sim import load_dataset
    blob = meshes.two_rooms()
    (tmp_path / "assets" / "scn").mkdir(parents=True)
    (tmp_path / "assets" / "scn" / "a.navmesh").write_bytes(blob)
    eps = [{"scene_id": "scn/a.glb", "start_position": [1, 0, 1], "start_rotation": [0, 0.6, 0, 0.8],
            "goals": [{"position": [7, 0, 3]}]},
           {"scene_id": "scn/a.glb", "start_position": [2, 0, 3], "start_rotation": [0, 0, 0, 1],
            "goals": [{"position": [6, 0, 1]}]}]
    (tmp_path / "content").mkdir()
    with gzip.open(tmp_path / "content" / "a.json.gz", "wt") as f:
        json.dump({"episodes": eps}, f)
    sc = load_dataset(str(tmp_path / "content"), str(tmp_path / "assets"))
    assert len(sc) == 1 and sc[0][0] == blob
    assert np.allclose(sc[0][1], [[1, 0, 1, 0, 0.6, 0, 0.8, 7, 0, 3], [2, 0, 3, 0, 0, 0, 1, 6, 0, 1]])


def test_oracle_rejects_malformed_navmeshes(oracle):
    blob = bytearray(meshes.l_shape())
    with pytest.raises(RuntimeError, match="magic"):
        bpo.Nav(oracle, bytes(b"XXXX" + blob[4:]))
    with pytest.raises(RuntimeError, match="truncated"):
        bpo.Nav(oracle, bytes(blob[:200]))
    bad = bytearray(blob)
    struct.pack_into("<H", bad, 48 + 100 + 12 * struct.unpack_from("<i", blob, 48 + 28)[0] + 4, 999)  # vertex index
    with pytest.raises(RuntimeError, match="vertex index"):
        bpo.Nav(oracle, bytes(bad))


def test_oracle_matches_compiled_reference_on_fresh_inputs(oracle, reflib):
    """Beyond the committed vectors: fresh random scenes and queries, oracle vs reference, bit
    for bit (development container only)."""
    if reflib is None:
        pytest.skip("compiled reference not available outside the development container")
    rng = np.random.default_rng(123)
    for config, idx in ((1, 7), (2, 9), (3, 1), (4, 2)):
        blob = scenes.config_scene(config, idx)
        no, nr = bpo.Nav(oracle, blob), bpo.Nav(reflib, blob)
        pts = scenes.sample_points(blob, idx, 1500) + rng.normal(0, 0.3, (1500, 3)).astype(np.float32)
        xo, ro = no.snap(pts)
        xr, rr = nr.snap(pts)
        assert np.array_equal(ro, rr) and np.array_equal(common.bits(xo), common.bits(xr))
        ok = rr != 0
        end = xr[ok] + rng.normal(0, 0.25, (ok.sum(), 3)).astype(np.float32)
        so, sro = no.try_step(xr[ok], rr[ok], end)
        sr, srr = nr.try_step(xr[ok], rr[ok], end)
        assert np.array_equal(sro, srr) and np.array_equal(common.bits(so), common.bits(sr))
        m = ok.sum() // 2
        go = no.geodesic(xr[ok][:m], rr[ok][:m], xr[ok][m:2 * m], rr[ok][m:2 * m])
        gr = nr.geodesic(xr[ok][:m], rr[ok][:m], xr[ok][m:2 * m], rr[ok][m:2 * m])
        assert np.array_equal(common.bits(go), common.bits(gr))
