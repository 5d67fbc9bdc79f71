"""ctypes binding of libbpsx.so (declarations in include/bpsx.h).

The library is built in-tree by __graft_entry__.build(); importing this module never
compiles anything and fails loudly if the library is missing.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("BPSX_LIBRARY") or os.path.join(_HERE, "libbpsx.so")


class Config(C.Structure):
    _fields_ = [("num_environments", C.c_uint32), ("num_active_scenes", C.c_uint32),
                ("double_buffered", C.c_uint32), ("reset_mode", C.c_uint32), ("seed", C.c_uint64),
                ("gpu_id", C.c_int32), ("max_steps", C.c_uint32), ("task", C.c_uint32), ("scene_reserve", C.c_float),
                ("rotate_scenes", C.c_uint32), ("rotation_interval_ms", C.c_uint32)]


class Outputs(C.Structure):
    _fields_ = [("rewards", C.c_void_p), ("masks", C.c_void_p), ("infos", C.c_void_p),
                ("polars", C.c_void_p), ("n", C.c_uint32), ("info_width", C.c_uint32)]


class State(C.Structure):
    _fields_ = [("position", C.c_void_p), ("rotation", C.c_void_p), ("goal", C.c_void_p),
                ("poly_ref", C.c_void_p), ("goal_ref", C.c_void_p), ("step", C.c_void_p),
                ("episode", C.c_void_p), ("num_resets", C.c_void_p), ("n", C.c_uint32)]


class TileDesc(C.Structure):
    _fields_ = [("verts", C.c_void_p), ("vert_count", C.c_uint32), ("polys", C.c_void_p),
                ("poly_flags", C.c_void_p), ("poly_areas", C.c_void_p), ("poly_count", C.c_uint32),
                ("nvp", C.c_uint32), ("walkable_height", C.c_float), ("walkable_radius", C.c_float),
                ("walkable_climb", C.c_float), ("bmin", C.c_float * 3), ("bmax", C.c_float * 3),
                ("cs", C.c_float), ("ch", C.c_float), ("tile_x", C.c_int32), ("tile_y", C.c_int32),
                ("tile_layer", C.c_int32), ("build_bv_tree", C.c_uint32)]


class SceneParams(C.Structure):
    _fields_ = [("kind", C.c_uint32), ("seed", C.c_uint64), ("cell", C.c_uint32),
                ("size_x", C.c_float), ("size_z", C.c_float), ("num_boxes", C.c_uint32),
                ("box_min", C.c_float), ("box_max", C.c_float), ("rooms_min", C.c_uint32),
                ("rooms_max", C.c_uint32), ("room_min", C.c_float), ("room_max", C.c_float),
                ("door_width", C.c_float), ("clutter_frac", C.c_float), ("maze_w", C.c_uint32),
                ("maze_h", C.c_uint32), ("corridor_min", C.c_float), ("corridor_max", C.c_float),
                ("wall", C.c_float), ("braid", C.c_float), ("tri_frac", C.c_float),
                ("hex_frac", C.c_float), ("origin", C.c_float * 3), ("tiles_x", C.c_uint32),
                ("tiles_z", C.c_uint32)]


_lib = None


def lib():
    """Returns the loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'`")
        L = C.CDLL(LIB_PATH)
        L.bpsx_last_error.restype = C.c_char_p
        L.bpsx_free.argtypes = [C.c_void_p]
        L.bpsx_gen_scene.argtypes = [C.POINTER(SceneParams), C.POINTER(C.c_void_p), C.POINTER(C.c_size_t)]
        L.bpsx_sample_points.argtypes = [C.c_char_p, C.c_size_t, C.c_uint64, C.c_uint32, C.c_void_p]
        L.bpsx_pack_tile.argtypes = [C.POINTER(TileDesc), C.POINTER(C.c_void_p), C.POINTER(C.c_size_t)]
        L.bpsx_pack_mset.argtypes = [C.POINTER(C.c_void_p), C.POINTER(C.c_size_t), C.c_uint32,
                                     C.POINTER(C.c_float), C.c_float, C.c_float, C.c_uint32, C.c_uint32,
                                     C.POINTER(C.c_void_p), C.POINTER(C.c_size_t)]
        if hasattr(L, "bpsx_create"):
            L.bpsx_create.argtypes = [C.POINTER(Config), C.POINTER(C.c_void_p)]
            L.bpsx_add_scene.argtypes = [C.c_void_p, C.c_char_p, C.c_size_t, C.c_void_p, C.c_uint32]
            L.bpsx_finalize.argtypes = [C.c_void_p]
            L.bpsx_swap_scene.argtypes = [C.c_void_p, C.c_uint32, C.c_char_p, C.c_size_t, C.c_void_p, C.c_uint32]
            L.bpsx_swap_status.argtypes = [C.c_void_p, C.c_uint32, C.POINTER(C.c_uint32), C.POINTER(C.c_uint64)]
            L.bpsx_active_scenes.argtypes = [C.c_void_p, C.c_void_p]
            L.bpsx_rotation_log.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32, C.POINTER(C.c_uint32)]
            L.bpsx_swap_stats.argtypes = [C.c_void_p, C.POINTER(C.c_double)]
            L.bpsx_destroy.argtypes = [C.c_void_p]
            L.bpsx_destroy.restype = None
            L.bpsx_num_groups.argtypes = [C.c_void_p, C.POINTER(C.c_uint32)]
            L.bpsx_reset.argtypes = [C.c_void_p, C.c_uint32, C.c_void_p]
            L.bpsx_step_start.argtypes = [C.c_void_p, C.c_uint32, C.c_void_p, C.c_int, C.c_void_p]
            L.bpsx_step_end.argtypes = [C.c_void_p, C.c_uint32]
            L.bpsx_set_stream_ordered.argtypes = [C.c_void_p, C.c_int]
            L.bpsx_synchronize.argtypes = [C.c_void_p]
            L.bpsx_get_outputs.argtypes = [C.c_void_p, C.c_uint32, C.POINTER(Outputs)]
            L.bpsx_get_state.argtypes = [C.c_void_p, C.c_uint32, C.POINTER(State)]
            L.bpsx_check_errors.argtypes = [C.c_void_p]
            L.bpsx_get_counters.argtypes = [C.c_void_p, C.c_void_p]
            L.bpsx_set_profiling.argtypes = [C.c_void_p, C.c_int]
            L.bpsx_get_kernel_times.argtypes = [C.c_void_p, C.POINTER(C.c_double), C.POINTER(C.c_uint64)]
            L.bpsx_kernel_name.argtypes = [C.c_uint32]
            L.bpsx_kernel_name.restype = C.c_char_p
            L.bpsx_snap_points.argtypes = [C.c_void_p, C.c_uint32, C.c_void_p, C.c_uint32, C.c_void_p, C.c_void_p]
            L.bpsx_try_steps.argtypes = [C.c_void_p, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p,
                                         C.c_uint32, C.c_void_p, C.c_void_p]
            L.bpsx_geodesic.argtypes = [C.c_void_p, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p,
                                        C.c_void_p, C.c_uint32, C.c_void_p]
            L.bpsx_geodesic_static.argtypes = [C.c_void_p, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p,
                                               C.c_void_p, C.c_uint32, C.c_void_p, C.c_void_p]
            L.bpsx_random_points.argtypes = [C.c_void_p, C.c_uint32, C.c_void_p, C.c_uint32, C.c_void_p, C.c_void_p]
        _lib = L
    return _lib


def check(rc):
    if rc != 0:
        raise RuntimeError(f"bpsx error {rc}: {lib().bpsx_last_error().decode()}")
