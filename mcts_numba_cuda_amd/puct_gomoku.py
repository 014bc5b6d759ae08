"""Host side of the Gomoku PUCT search loop with virtual loss: a ctypes binding of the puct_gomoku_* entry points of
libpuct_hip.so (C ABI: include/puct_gomoku.h).  No CPU fallback: without the library or a GPU every call raises."""
import atexit
import ctypes
import sys
import weakref

import numpy as np

from . import puct

ARRAYS = {  # name -> (id, dtype, shape builder)
    "edge_child": (0, np.int32, "TNE"), "edge_prior": (1, np.float32, "TNE"), "edge_w": (2, np.float32, "TNE"),
    "edge_n": (3, np.int32, "TNE"), "edge_inflight": (4, np.int32, "TNE"), "edge_action": (5, np.uint8, "TNE"),
    "node_expanded": (6, np.int32, "TN"), "node_expand_inflight": (7, np.int32, "TN"), "node_count": (8, np.int32, "T"),
    "node_board": (9, np.uint32, "TNB"), "node_turn": (10, np.int8, "TN"), "node_value": (11, np.float32, "TN"),
    "out_selected": (12, np.int32, "TW"), "out_path": (13, np.int32, "TWD"), "out_len": (14, np.int32, "TW"),
    "path_values": (15, np.float32, "TWD"), "node_legal": (16, np.int32, "TN"),
}
EDGES = 256


class Config(ctypes.Structure):
    _fields_ = [("board_m", ctypes.c_int32), ("board_n", ctypes.c_int32), ("trees", ctypes.c_int32),
                ("traversals", ctypes.c_int32), ("max_nodes", ctypes.c_int32), ("path_depth", ctypes.c_int32),
                ("cpuct", ctypes.c_float), ("c_pw", ctypes.c_float), ("alpha_pw", ctypes.c_float),
                ("dirichlet_alpha", ctypes.c_float), ("seed", ctypes.c_uint64),
                ("device", ctypes.c_int32), ("evaluators", ctypes.c_int32), ("agent_fences", ctypes.c_int32)]


class Result(ctypes.Structure):
    _fields_ = [("steps", ctypes.c_int64), ("best_action", ctypes.c_int32), ("best_n", ctypes.c_int64),
                ("root_n", ctypes.c_int64 * 256), ("root_w", ctypes.c_double * 256), ("selections", ctypes.c_int64 * 5),
                ("expansions_committed", ctypes.c_int64), ("nodes_total", ctypes.c_int64),
                ("max_nodes_in_tree", ctypes.c_int32), ("time_total", ctypes.c_double), ("time_device", ctypes.c_double),
                ("nodes_read", ctypes.c_int64), ("edges_scored", ctypes.c_int64), ("time_select", ctypes.c_double),
                ("time_expand", ctypes.c_double), ("time_backup", ctypes.c_double)]


class EngineError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"libpuct_hip error {code}: {message}")
        self.code = code


_bound = False


def _lib():
    global _bound
    L = puct._lib()
    if not _bound:
        vp = ctypes.c_void_p
        L.puct_gomoku_create.restype = ctypes.c_int
        L.puct_gomoku_create.argtypes = [ctypes.POINTER(Config), ctypes.POINTER(vp)]
        L.puct_gomoku_destroy.restype = None
        L.puct_gomoku_destroy.argtypes = [vp]
        L.puct_gomoku_run.restype = ctypes.c_int
        L.puct_gomoku_run.argtypes = [vp, vp, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.POINTER(Result)]
        L.puct_gomoku_array_bytes.restype = ctypes.c_int64
        L.puct_gomoku_array_bytes.argtypes = [vp, ctypes.c_int32]
        L.puct_gomoku_read.restype = ctypes.c_int
        L.puct_gomoku_read.argtypes = [vp, ctypes.c_int32, vp, ctypes.c_size_t]
        L.puct_gomoku_last_error.restype = ctypes.c_char_p
        _bound = True
    return L


def _check(rc):
    if rc != 0:
        raise EngineError(rc, _lib().puct_gomoku_last_error().decode("utf-8", "replace"))


class PUCTGomoku:
    """PUCT search on Gomoku with virtual loss: `trees` independent trees on one root, `traversals` selections per
    tree and step (claims taken in a fixed order, so a search is reproducible), a synthetic evaluator (Dirichlet(dirichlet_alpha) priors over the legal cells and a
    value in [-1, 1), both pure functions of the position and the seed); `evaluators` workgroups per tree work out the
    priors of new nodes beside the tree's own workgroup (0: it does that itself; same trees either way; `agent_fences` makes them hand over with full
    device-scope releases even where they share an L2, which is slower and changes nothing else).  `run` returns the cell with the most root
    visits; `root_n`, `root_q`, `selections`, `performance_info` describe the last search."""

    def __init__(self, board_shape=(15, 15), trees=16, traversals=16, max_nodes=16384, path_depth=64, cpuct=1.5,
                 c_pw=1.0, alpha_pw=0.5, dirichlet_alpha=0.3, seed=0, device=0, evaluators=4, agent_fences=False):
        self.cfg = Config(int(board_shape[0]), int(board_shape[1]), int(trees), int(traversals), int(max_nodes),
                          int(path_depth), float(cpuct), float(c_pw), float(alpha_pw), float(dirichlet_alpha), int(seed),
                          int(device), int(evaluators), int(bool(agent_fences)))
        self._engine = ctypes.c_void_p()
        _check(_lib().puct_gomoku_create(ctypes.byref(self.cfg), ctypes.byref(self._engine)))
        self.result = None
        _LIVE.add(self)

    def __del__(self):
        if not sys.is_finalizing():   # engines alive at interpreter exit were closed by the exit hook below
            self.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
        return False

    def close(self):
        eng, self._engine = getattr(self, "_engine", None), None
        if eng:
            _lib().puct_gomoku_destroy(eng)

    def run(self, board, turn, steps, fused=True):
        board = np.ascontiguousarray(board, dtype=np.int8)
        if board.shape != (self.cfg.board_m, self.cfg.board_n):
            raise ValueError(f"board must have shape {(self.cfg.board_m, self.cfg.board_n)}")
        res = Result()
        _check(_lib().puct_gomoku_run(self._engine, board.ctypes.data, int(turn), int(steps), int(bool(fused)),
                                      ctypes.byref(res)))
        self.result = res
        cells = self.cfg.board_m * self.cfg.board_n
        self.root_n = np.array(res.root_n[:cells], dtype=np.int64)
        root_w = np.array(res.root_w[:cells], dtype=np.float64)
        with np.errstate(divide="ignore", invalid="ignore"):
            self.root_q = np.where(self.root_n > 0, root_w / self.root_n, np.nan)
        self.selections = dict(zip(("invalid", "expand", "terminal", "depth_limit", "busy"), res.selections))
        total = sum(res.selections)
        leaves = total - res.selections[0] - res.selections[4]    # selections that reached a node to evaluate
        self.performance_info = {
            "steps": int(res.steps), "selections": int(total), "selections_per_second": total / max(res.time_device, 1e-12),
            "leaves": int(leaves), "leaves_per_second": leaves / max(res.time_device, 1e-12),
            "leaves_per_step": leaves / max(res.steps, 1), "busy_share": res.selections[4] / max(total, 1),
            "steps_per_second": res.steps / max(res.time_device, 1e-12), "expansions": int(res.expansions_committed),
            "nodes_total": int(res.nodes_total), "max_nodes_in_tree": int(res.max_nodes_in_tree),
            "nodes_read": int(res.nodes_read), "edges_scored": int(res.edges_scored),
            "times_[ms]": {"total": 1e3 * res.time_total, "device": 1e3 * res.time_device, "select": 1e3 * res.time_select,
                           "expand": 1e3 * res.time_expand, "backup": 1e3 * res.time_backup}}
        self.best_action = int(res.best_action)
        return self.best_action

    def read_array(self, name):
        aid, dtype, shape = ARRAYS[name]
        dims = {"T": self.cfg.trees, "N": self.cfg.max_nodes, "E": EDGES, "W": self.cfg.traversals,
                "D": self.cfg.path_depth, "B": 16}
        out = np.empty(tuple(dims[c] for c in shape), dtype=dtype)
        nbytes = _lib().puct_gomoku_array_bytes(self._engine, aid)
        if nbytes != out.nbytes:
            raise EngineError(-1, f"array {name}: library reports {nbytes} bytes, expected {out.nbytes}")
        _check(_lib().puct_gomoku_read(self._engine, aid, out.ctypes.data, out.nbytes))
        return out


_LIVE = weakref.WeakSet()


@atexit.register
def _close_all_engines():
    """Interpreter exit: engines still alive are released while the HIP runtime is fully up."""
    for e in list(_LIVE):
        try:
            e.close()
        except Exception:
            pass
