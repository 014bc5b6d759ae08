"""ctypes front end of the CPU oracle (``mctsnc_oracle.c``).

TEST INFRASTRUCTURE: only tests, the smoke check and the CPU-baseline leg of the
benchmark import this module; the product package never does.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmctsnc_oracle.so")

GAMES = {"c4": 0, "gomoku": 1}
VARIANTS = ["ocp_thrifty", "ocp_prodigal", "acp_thrifty", "acp_prodigal"]
MAX_TREE_DEPTH = 2048


def build(force=False):
    """Compiles the oracle with gcc through its Makefile."""
    if force:
        for path in (_LIB_PATH, os.path.join(_HERE, "libpuct_oracle.so")):
            if os.path.exists(path):
                os.remove(path)
    subprocess.check_call(["make", "-s", "-C", _HERE])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i32, i64, u64, dbl = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_uint64, ctypes.c_double
        L.mo_create.restype = vp
        L.mo_create.argtypes = [i32] * 8 + [dbl, u64, i64]
        L.mo_destroy.argtypes = [vp]
        L.mo_set_threads.argtypes = [vp, i32]
        L.mo_run.restype = i32
        L.mo_run.argtypes = [vp, vp, vp, i32, i32, i64]
        L.mo_tree_size.restype = i32
        L.mo_tree_size.argtypes = [vp, i32]
        L.mo_tree_selected.restype = i32
        L.mo_tree_selected.argtypes = [vp, i32]
        L.mo_tree_array.restype = vp
        L.mo_tree_array.argtypes = [vp, i32, i32]
        L.mo_result_array.restype = vp
        L.mo_result_array.argtypes = [vp, i32]
        L.mo_rng_states.restype = vp
        L.mo_rng_states.argtypes = [vp, i32]
        for name, rt in [("mo_best_action", i32), ("mo_best_win_flag", i32), ("mo_best_n", i64),
                         ("mo_best_n_wins", i64), ("mo_u1_events", u64), ("mo_plies", u64)]:
            getattr(L, name).restype = rt
            getattr(L, name).argtypes = [vp]
        L.mo_ucb.restype = ctypes.c_float
        L.mo_ucb.argtypes = [i32, i32, i32, ctypes.c_float]
        L.mo_argmax_tournament_f32.restype = i32
        L.mo_argmax_tournament_f32.argtypes = [vp, i32, i32]
        L.mo_argmax_tournament_lex.restype = i32
        L.mo_argmax_tournament_lex.argtypes = [vp, vp, vp, i32, i32]
        L.mo_game_outcome.restype = i32
        L.mo_game_outcome.argtypes = [i32, i32, i32, vp, vp, i32, i32]
        L.mo_rng_init.argtypes = [vp, i64, u64]
        L.mo_rng_next.restype = u64
        L.mo_rng_next.argtypes = [vp]
        L.mo_rng_uniform.restype = ctypes.c_float
        L.mo_rng_uniform.argtypes = [vp]
        L.mo_rng_jump.argtypes = [vp]
        _lib = L
    return _lib


def _as_array(ptr, shape, dtype):
    n = int(np.prod(shape))
    if n == 0:
        return np.zeros(shape, dtype=dtype)
    buf = (ctypes.c_char * (n * np.dtype(dtype).itemsize)).from_address(ptr)
    return np.frombuffer(buf, dtype=dtype).reshape(shape).copy()


def max_tree_size(board_shape, extra_info_memory, max_actions, n_trees, variant, device_memory_gib):
    """The reference's node-pool sizing (src/mctsnc.py:350-358)."""
    E = max(extra_info_memory, 1)
    per_state_additional = 2 + 1 + 2 * 1 + 1 + 2 * 4
    per_tree_additional = 4 + 4 + 2 * (max_actions + 2) + 4 * 2 + 4 * (MAX_TREE_DEPTH + 2)
    if "acp" in variant:
        per_tree_additional += 4 * max_actions * 2
    per_state = int(np.prod(board_shape)) + E + 4 * (1 + max_actions) + per_state_additional
    s = (int(device_memory_gib * 1024**3) - n_trees * per_tree_additional) // (per_state * n_trees)
    return min(s, 2**24)


class Oracle:
    """One oracle engine: same life cycle as the reference's MCTSNC instance (RNG streams persist across runs)."""

    def __init__(self, game, board_shape, extra_info_memory, max_actions, n_trees, n_playouts, variant,
                 ucb_c=2.0, seed=0, device_memory=2.0, max_tree_size_override=None, threads=1):
        self.L = lib()
        self.game = game
        self.m, self.n = board_shape
        self.E = max(extra_info_memory, 1)
        self.A = max_actions
        self.T, self.P = n_trees, n_playouts
        self.variant = variant
        self.S = max_tree_size_override if max_tree_size_override is not None else \
            max_tree_size(board_shape, extra_info_memory, max_actions, n_trees, variant, device_memory)
        self.h = self.L.mo_create(GAMES[game], self.m, self.n, self.E, self.A, self.T, self.P,
                                  VARIANTS.index(variant), float(ucb_c), int(seed), int(self.S))
        self.L.mo_set_threads(self.h, threads)

    def __del__(self):
        if getattr(self, "h", None):
            self.L.mo_destroy(self.h)
            self.h = None

    def run(self, root_board, root_extra_info, root_turn, steps):
        b = np.ascontiguousarray(root_board, dtype=np.int8)
        if root_extra_info is None:
            ep, el = None, 0
        else:
            e = np.ascontiguousarray(root_extra_info, dtype=np.int8)
            ep, el = e.ctypes.data, e.size
        return self.L.mo_run(self.h, b.ctypes.data, ep, el, int(root_turn), int(steps))

    # ---- results -------------------------------------------------------------------------------
    @property
    def best(self):
        L, h = self.L, self.h
        return dict(action=L.mo_best_action(h), win_flag=bool(L.mo_best_win_flag(h)), n=L.mo_best_n(h),
                    n_wins=L.mo_best_n_wins(h))

    def result(self, name):
        which, shape, dt = {"root_actions_expanded": (0, (self.A + 2,), np.int16),
                            "root_ns": (1, (self.A,), np.int64),
                            "actions_ns": (2, (self.A,), np.int64),
                            "actions_ns_wins": (3, (self.A,), np.int64),
                            "actions_win_flags": (4, (self.A,), np.uint8)}[name]
        return _as_array(self.L.mo_result_array(self.h, which), shape, dt)

    def tree_size(self, ti):
        return self.L.mo_tree_size(self.h, ti)

    def tree_selected(self, ti):
        return self.L.mo_tree_selected(self.h, ti)

    def tree(self, ti, name):
        sz = self.tree_size(ti)
        which, shape, dt = {"trees": (0, (sz, 1 + self.A), np.int32),
                            "depths": (1, (sz,), np.int16),
                            "turns": (2, (sz,), np.int8),
                            "leaves": (3, (sz,), np.uint8),
                            "terminals": (4, (sz,), np.uint8),
                            "outcomes": (5, (sz,), np.int8),
                            "ns": (6, (sz,), np.int32),
                            "ns_wins": (7, (sz,), np.int32),
                            "boards": (8, (sz, self.m, self.n), np.int8),
                            "extras": (9, (sz, self.E), np.int8),
                            "path": (10, (MAX_TREE_DEPTH + 2,), np.int32),
                            "actions_expanded": (11, (self.A + 2,), np.int16),
                            "playout_outcomes": (12, (2,), np.int32),
                            "playout_outcomes_children": (13, (self.A, 2), np.int32)}[name]
        return _as_array(self.L.mo_tree_array(self.h, ti, which), shape, dt)

    def rng_states(self, which="playout"):
        if which == "playout":
            n = self.T * self.P if self.variant.startswith("ocp") else self.T * self.A * self.P
            return _as_array(self.L.mo_rng_states(self.h, 0), (n, 2), np.uint64)
        raise ValueError(which)

    @property
    def u1_events(self):
        return self.L.mo_u1_events(self.h)

    @property
    def plies(self):
        return self.L.mo_plies(self.h)

    def tree_stats(self):
        """mean_depth / max_depth / mean_size / max_size as in _make_performance_info (src/mctsnc.py:472-492)."""
        total_depth, max_depth, sizes = 0, -1, []
        for ti in range(self.T):
            d = self.tree(ti, "depths")
            total_depth += int(d.astype(np.int64).sum())
            max_depth = max(max_depth, int(d.max()))
            sizes.append(self.tree_size(ti))
        total = int(np.sum(sizes))
        return dict(mean_depth=total_depth / total, max_depth=max_depth, mean_size=total / self.T,
                    max_size=int(np.max(sizes)))
