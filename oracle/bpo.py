"""TEST INFRASTRUCTURE: ctypes wrapper over the bpo_* C surface exported by both
oracle/liboracle.so (independent CPU restatement, kind "port") and
oracle/_ref/libbpsref.so (compiled reference PathFinder + Detour, kind "reference").

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may import this.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(_HERE, "liboracle.so")
REF_SO = os.path.join(_HERE, "_ref", "libbpsref.so")

_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_u32p = np.ctypeslib.ndpointer(np.uint32, flags="C_CONTIGUOUS")
_u8p = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")
_i64p = np.ctypeslib.ndpointer(np.int64, flags="C_CONTIGUOUS")


def build_oracle():
    subprocess.check_call(["make", "-C", _HERE, "liboracle.so"], stdout=subprocess.DEVNULL)


def build_ref():
    subprocess.check_call(["make", "-C", _HERE, "ref"], stdout=subprocess.DEVNULL)


class Lib:
    def __init__(self, path):
        self.path = path
        L = self.L = C.CDLL(path)
        L.bpo_last_error.restype = C.c_char_p
        L.bpo_kind.restype = C.c_char_p
        L.bpo_nav_load.restype = C.c_void_p
        L.bpo_nav_load.argtypes = [C.c_char_p, C.c_size_t]
        L.bpo_nav_snap.argtypes = [C.c_void_p, _f32p, C.c_uint32, _f32p, _u32p]
        L.bpo_nav_try_step.argtypes = [C.c_void_p, _f32p, _u32p, _f32p, C.c_uint32, _f32p, _u32p]
        L.bpo_nav_geodesic.argtypes = [C.c_void_p, _f32p, _u32p, _f32p, _u32p, C.c_uint32, _f32p]
        L.bpo_nav_sample.argtypes = [C.c_void_p, _f32p, C.c_uint32, _f32p]
        L.bpo_nav_free.argtypes = [C.c_void_p]
        L.bpo_sim_create.restype = C.c_void_p
        L.bpo_sim_create.argtypes = [C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint64, C.c_uint32, C.c_int]
        L.bpo_sim_add_scene.argtypes = [C.c_void_p, C.c_char_p, C.c_size_t, _f32p, C.c_uint32]
        L.bpo_sim_finalize.argtypes = [C.c_void_p]
        L.bpo_sim_set_task.argtypes = [C.c_void_p, C.c_uint32]
        L.bpo_sim_swap_scene.argtypes = [C.c_void_p, C.c_uint32, C.c_char_p, C.c_size_t, _f32p, C.c_uint32]
        L.bpo_sim_swap_remaining.argtypes = [C.c_void_p, C.c_uint32]
        L.bpo_sim_swap_remaining.restype = C.c_uint32
        L.bpo_sim_envs_per_group.argtypes = [C.c_void_p]
        L.bpo_sim_envs_per_group.restype = C.c_uint32
        L.bpo_sim_reset.argtypes = [C.c_void_p, C.c_uint32]
        L.bpo_sim_step.argtypes = [C.c_void_p, C.c_uint32, _i64p]
        L.bpo_sim_bad_action.argtypes = [C.c_void_p]
        L.bpo_sim_get_outputs.argtypes = [C.c_void_p, C.c_uint32, _f32p, _u8p, _f32p, _f32p]
        L.bpo_sim_get_state.argtypes = [C.c_void_p, C.c_uint32, _f32p, _f32p, _f32p, _u32p, _u32p, _u32p, _u32p, _u32p]
        L.bpo_sim_destroy.argtypes = [C.c_void_p]
        L.bpo_random_point_in_convex_poly.argtypes = [_f32p, C.c_int, C.c_float, C.c_float, _f32p]
        self.kind = L.bpo_kind().decode()
        if self.kind == "port":
            L.bpo_sim_counters.argtypes = [C.c_void_p, np.ctypeslib.ndpointer(np.uint64, flags="C_CONTIGUOUS")]
            L.bpo_nav_poly_count.argtypes = [C.c_void_p]
            L.bpo_nav_poly_info.argtypes = [C.c_void_p, _u32p, np.ctypeslib.ndpointer(np.uint16), np.ctypeslib.ndpointer(np.int32)]
            L.bpo_nav_last_corridor.argtypes = [C.c_void_p, _u32p, C.c_int]
            L.bpo_nav_pass_check.argtypes = [C.c_void_p, C.c_int, np.ctypeslib.ndpointer(np.uint64, flags="C_CONTIGUOUS")]
        else:
            L.bpo_nav_find_random_points.argtypes = [C.c_void_p, C.c_uint64, C.c_uint32, _f32p, _u32p]
            L.bpo_ref_create_tile.argtypes = [
                np.ctypeslib.ndpointer(np.uint16), C.c_int, np.ctypeslib.ndpointer(np.uint16),
                np.ctypeslib.ndpointer(np.uint16), _u8p, C.c_int, C.c_int, C.c_float, C.c_float, C.c_float,
                _f32p, _f32p, C.c_float, C.c_float, _u8p, C.c_int]

    def error(self):
        return self.L.bpo_last_error().decode()

    def random_point_in_convex_poly(self, pts, s, t):
        pts = np.ascontiguousarray(pts, np.float32)
        out = np.zeros(3, np.float32)
        self.L.bpo_random_point_in_convex_poly(pts.reshape(-1), len(pts), s, t, out)
        return out


COUNTER_NAMES = ["move_calls", "move_polys", "move_verts", "height_tris", "path_calls", "astar_pops",
                 "astar_links", "corridor_polys", "snap_calls", "snap_bv_nodes", "snap_cands",
                 "snap_cand_verts", "snap_cand_tris"]


class Nav:
    """One navmesh + one query context (PathFinder-level calls)."""

    def __init__(self, lib, navmesh_bytes):
        self.lib = lib
        self.h = lib.L.bpo_nav_load(navmesh_bytes, len(navmesh_bytes))
        if not self.h:
            raise RuntimeError("nav load failed: " + lib.error())

    def close(self):
        if self.h:
            self.lib.L.bpo_nav_free(self.h)
            self.h = None

    def __del__(self):
        self.close()

    def snap(self, pts):
        pts = np.ascontiguousarray(pts, np.float32).reshape(-1, 3)
        n = len(pts)
        xyz = np.zeros((n, 3), np.float32)
        ref = np.zeros(n, np.uint32)
        self.lib.L.bpo_nav_snap(self.h, pts, n, xyz, ref)
        return xyz, ref

    def try_step(self, sxyz, sref, exyz):
        sxyz = np.ascontiguousarray(sxyz, np.float32).reshape(-1, 3)
        exyz = np.ascontiguousarray(exyz, np.float32).reshape(-1, 3)
        sref = np.ascontiguousarray(sref, np.uint32)
        n = len(sxyz)
        xyz = np.zeros((n, 3), np.float32)
        ref = np.zeros(n, np.uint32)
        self.lib.L.bpo_nav_try_step(self.h, sxyz, sref, exyz, n, xyz, ref)
        return xyz, ref

    def geodesic(self, sxyz, sref, exyz, eref):
        sxyz = np.ascontiguousarray(sxyz, np.float32).reshape(-1, 3)
        exyz = np.ascontiguousarray(exyz, np.float32).reshape(-1, 3)
        sref = np.ascontiguousarray(sref, np.uint32)
        eref = np.ascontiguousarray(eref, np.uint32)
        n = len(sxyz)
        out = np.zeros(n, np.float32)
        self.lib.L.bpo_nav_geodesic(self.h, sxyz, sref, exyz, eref, n, out)
        return out

    def sample(self, u):
        u = np.ascontiguousarray(u, np.float32).reshape(-1, 3)
        out = np.zeros((len(u), 3), np.float32)
        self.lib.L.bpo_nav_sample(self.h, u, len(u), out)
        return out

    def poly_info(self):
        n = self.lib.L.bpo_nav_poly_count(self.h)
        refs = np.zeros(n, np.uint32)
        flags = np.zeros(n, np.uint16)
        isl = np.zeros(n, np.int32)
        self.lib.L.bpo_nav_poly_info(self.h, refs, flags, isl)
        return refs, flags, isl

    def pass_check(self, rows):
        """Switches the check of the GPU kernel's multi-node pass rules (orc::Query::PassCheck) to
        `rows` nodes per pass (0: off) and returns the counts gathered since the last call."""
        out = np.zeros(6, np.uint64)
        self.lib.L.bpo_nav_pass_check(self.h, int(rows), out)
        return dict(zip(("passes", "nodes", "wrong_node", "wrong_update", "pairs", "ties"), (int(v) for v in out)))

    def last_corridor(self):
        buf = np.zeros(256, np.uint32)
        n = self.lib.L.bpo_nav_last_corridor(self.h, buf, 256)
        return buf[:n].copy()


class Sim:
    """CPU simulator with the reference's worker-thread dispatch."""

    def __init__(self, lib, scenes, num_envs, double_buffered=False, reset_mode=0, seed=0, max_steps=0, threads=1,
                 task=0):
        """task: 0 PointNav, 1 Flee, 2 Exploration (infos column 0 holds the single info value of 1 and 2)."""
        self.lib = lib
        self.h = lib.L.bpo_sim_create(num_envs, len(scenes), int(double_buffered), reset_mode, seed, max_steps, threads)
        lib.L.bpo_sim_set_task(self.h, task)
        for blob, eps in scenes:
            eps = np.ascontiguousarray(eps, np.float32).reshape(-1, 10)
            if lib.L.bpo_sim_add_scene(self.h, blob, len(blob), eps, len(eps)) != 0:
                raise RuntimeError("add_scene failed: " + lib.error())
        if lib.L.bpo_sim_finalize(self.h) != 0:
            raise RuntimeError("finalize failed: " + lib.error())
        self.n = lib.L.bpo_sim_envs_per_group(self.h)

    def close(self):
        if self.h:
            self.lib.L.bpo_sim_destroy(self.h)
            self.h = None

    def __del__(self):
        self.close()

    def swap_scene(self, slot, blob, eps):
        eps = np.ascontiguousarray(eps, np.float32).reshape(-1, 10)
        if self.lib.L.bpo_sim_swap_scene(self.h, slot, blob, len(blob), eps, len(eps)) != 0:
            raise RuntimeError("swap_scene failed: " + self.lib.error())

    def swap_remaining(self, slot):
        return int(self.lib.L.bpo_sim_swap_remaining(self.h, slot))

    def reset(self, group=0):
        self.lib.L.bpo_sim_reset(self.h, group)

    def step(self, actions, group=0):
        actions = np.ascontiguousarray(actions, np.int64)
        assert len(actions) == self.n
        self.lib.L.bpo_sim_step(self.h, group, actions)

    def outputs(self, group=0):
        n = self.n
        r = np.zeros(n, np.float32)
        m = np.zeros(n, np.uint8)
        i = np.zeros((n, 3), np.float32)
        p = np.zeros((n, 2), np.float32)
        self.lib.L.bpo_sim_get_outputs(self.h, group, r, m, i, p)
        return dict(rewards=r, masks=m, infos=i, polars=p)

    def state(self, group=0):
        n = self.n
        pos = np.zeros((n, 3), np.float32)
        rot = np.zeros((n, 4), np.float32)
        goal = np.zeros((n, 3), np.float32)
        arrs = [np.zeros(n, np.uint32) for _ in range(5)]
        self.lib.L.bpo_sim_get_state(self.h, group, pos, rot, goal, *arrs)
        return dict(position=pos, rotation=rot, goal=goal, poly_ref=arrs[0], goal_ref=arrs[1], step=arrs[2],
                    episode=arrs[3], num_resets=arrs[4])

    def counters(self):
        out = np.zeros(13, np.uint64)
        self.lib.L.bpo_sim_counters(self.h, out)
        return dict(zip(COUNTER_NAMES, (int(v) for v in out)))

    def bad_action(self):
        return bool(self.lib.L.bpo_sim_bad_action(self.h))


def load_oracle():
    if not os.path.exists(ORACLE_SO):
        build_oracle()
    return Lib(ORACLE_SO)


def load_ref():
    """Returns the compiled-reference library, or None where it has not been built."""
    if not os.path.exists(REF_SO):
        return None
    return Lib(REF_SO)
