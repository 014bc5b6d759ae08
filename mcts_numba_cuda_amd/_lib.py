"""ctypes binding of libmctsnc_hip.so (C ABI: include/mctsnc_hip.h).  No fallback: without the library every
search call raises."""
import ctypes
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libmctsnc_hip.so")
MAX_ACTIONS = 512

GAME_C4, GAME_GOMOKU = 0, 1


class Config(ctypes.Structure):
    _fields_ = [("game", ctypes.c_int32), ("board_m", ctypes.c_int32), ("board_n", ctypes.c_int32),
                ("extra_info_memory", ctypes.c_int32), ("max_actions", ctypes.c_int32), ("n_trees", ctypes.c_int32),
                ("n_playouts", ctypes.c_int32), ("variant", ctypes.c_int32), ("ucb_c", ctypes.c_float),
                ("seed", ctypes.c_uint64), ("max_tree_size", ctypes.c_int64), ("device", ctypes.c_int32)]


class Result(ctypes.Structure):
    _fields_ = [("steps", ctypes.c_int64), ("best_action", ctypes.c_int32), ("best_win_flag", ctypes.c_int32),
                ("best_n", ctypes.c_int64), ("best_n_wins", ctypes.c_int64), ("n_root_entries", ctypes.c_int32),
                ("root_actions_expanded", ctypes.c_int16 * (MAX_ACTIONS + 2)),
                ("root_ns", ctypes.c_int64 * MAX_ACTIONS), ("actions_ns", ctypes.c_int64 * MAX_ACTIONS),
                ("actions_ns_wins", ctypes.c_int64 * MAX_ACTIONS), ("actions_win_flags", ctypes.c_uint8 * MAX_ACTIONS),
                ("time_total", ctypes.c_double), ("time_loop", ctypes.c_double), ("time_reduce", ctypes.c_double),
                ("time_device_loop", ctypes.c_double), ("depth_sum", ctypes.c_int64), ("size_sum", ctypes.c_int64),
                ("max_depth", ctypes.c_int32), ("max_size", ctypes.c_int32), ("playout_plies", ctypes.c_uint64),
                ("u1_events", ctypes.c_uint64), ("stat_levels", ctypes.c_uint64), ("stat_children", ctypes.c_uint64),
                ("stat_expanded", ctypes.c_uint64), ("stat_played", ctypes.c_uint64), ("time_select", ctypes.c_double),
                ("time_expand", ctypes.c_double), ("time_playout", ctypes.c_double), ("time_backup", ctypes.c_double),
                ("time_exchange", ctypes.c_double)]


ARRAYS = {  # name -> (id, dtype, trailing shape builder)
    "trees": (0, np.int32), "depths": (1, np.int16), "turns": (2, np.int8), "leaves": (3, np.uint8),
    "terminals": (4, np.uint8), "outcomes": (5, np.int8), "ns": (6, np.int32), "ns_wins": (7, np.int32),
    "boards": (8, np.int8), "extra_infos": (9, np.int8), "selected_path": (10, np.int32),
    "actions_expanded": (11, np.int16), "playout_outcomes": (12, np.int32),
    "playout_outcomes_children": (13, np.int32), "node_selected": (14, np.int32),
    "rng_playout": (15, np.uint64), "rng_expand": (16, np.uint64),
}

# mctsnc_set_option(): names of the MCTSNC_OPT_* constants of include/mctsnc_hip.h
OPTIONS = {"agent_fences": 0, "solo_trees": 1, "solo_threads": 2, "team_pool": 3, "team_pool_threads": 4, "prep_levels": 5,
           "plain_launch": 6, "probe_steps": 7, "spin_limit": 8}

_lib = None


class EngineError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"libmctsnc_hip error {code}: {message}")
        self.code = code


def lib():
    """Loads the shared library; raises if it has not been built (run mcts_numba_cuda_amd/build.py)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m mcts_numba_cuda_amd.build` "
                               "(there is no CPU fallback for the search engine)")
        L = ctypes.CDLL(LIB_PATH)
        vp = ctypes.c_void_p
        L.mctsnc_create.restype = ctypes.c_int
        L.mctsnc_create.argtypes = [ctypes.POINTER(Config), ctypes.POINTER(vp)]
        L.mctsnc_init_device.restype = ctypes.c_int
        L.mctsnc_init_device.argtypes = [vp]
        L.mctsnc_run.restype = ctypes.c_int
        L.mctsnc_run.argtypes = [vp, vp, vp, ctypes.c_int32, ctypes.c_int32, ctypes.c_double, ctypes.c_double, ctypes.c_double,
                                 ctypes.POINTER(Result)]
        L.mctsnc_run_batch.restype = ctypes.c_int
        L.mctsnc_run_batch.argtypes = [ctypes.POINTER(vp), ctypes.c_int32, vp, vp, ctypes.c_int32, vp, ctypes.c_double,
                                       ctypes.c_double, ctypes.c_double, ctypes.POINTER(Result)]
        L.mctsnc_run_batch_noalloc.restype = ctypes.c_int
        L.mctsnc_run_batch_noalloc.argtypes = L.mctsnc_run_batch.argtypes
        L.mctsnc_read_size.restype = ctypes.c_int64
        L.mctsnc_read_size.argtypes = [vp, ctypes.c_int32, ctypes.c_int32]
        L.mctsnc_read.restype = ctypes.c_int
        L.mctsnc_read.argtypes = [vp, ctypes.c_int32, ctypes.c_int32, vp, ctypes.c_size_t]
        L.mctsnc_reseed.restype = ctypes.c_int
        L.mctsnc_reseed.argtypes = [vp]
        L.mctsnc_set_option.restype = ctypes.c_int
        L.mctsnc_set_option.argtypes = [vp, ctypes.c_int32, ctypes.c_int32]
        L.mctsnc_set_stage_timing.restype = ctypes.c_int
        L.mctsnc_set_stage_timing.argtypes = [vp, ctypes.c_int32]
        L.mctsnc_destroy.restype = None
        L.mctsnc_destroy.argtypes = [vp]
        L.mctsnc_last_error.restype = ctypes.c_char_p
        L.mctsnc_last_error.argtypes = []
        _lib = L
    return _lib


def check(rc):
    if rc != 0:
        raise EngineError(rc, lib().mctsnc_last_error().decode())
