"""ctypes binding of the sequential CPU oracle of PUCT select / backup (oracle/puct_oracle.c).  Test infrastructure
only: product code never imports this module."""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libpuct_oracle.so")
_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            from . import oracle
            oracle.build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, ci, cf = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
        L.po_select.restype = None
        L.po_select.argtypes = [cf, cf, cf, ci] + [vp] * 11 + [ci] * 5
        L.po_node_select.restype = None
        L.po_node_select.argtypes = [ci, cf, cf, cf] + [vp] * 11 + [ci] * 5
        L.po_backup.restype = None
        L.po_backup.argtypes = [ci, ci] + [vp] * 11 + [ci] * 5
        _lib = L
    return _lib


def _ptr(a):
    return None if a is None else a.ctypes.data


def select(h, cpuct=1.0, c_pw=1.0, alpha_pw=0.5, soft_winner=0):
    """Runs the traversals of one launch one after another (tree-major, wid ascending) on the host arrays of `h`
    (the dictionary layout of src/puct/test_puct_gpu_v3.py:85-111), in place."""
    trees, nodes, edges = h["edge_child"].shape
    warps, depth = h["out_path"].shape[1:]
    for k in ("edge_child", "edge_n", "edge_inflight", "node_expand_inflight", "node_expanded", "node_count",
              "out_selected", "out_path", "out_len"):
        assert h[k].dtype == np.int32 and h[k].flags.c_contiguous, k
    for k in ("edge_prior", "edge_w"):
        assert h[k].dtype == np.float32 and h[k].flags.c_contiguous, k
    lib().po_select(cpuct, c_pw, alpha_pw, int(soft_winner), _ptr(h["edge_child"]), _ptr(h["edge_prior"]),
                    _ptr(h["edge_w"]), _ptr(h["edge_n"]), _ptr(h["edge_inflight"]), _ptr(h["node_expand_inflight"]),
                    _ptr(h["node_expanded"]), _ptr(h["node_count"]), _ptr(h["out_selected"]), _ptr(h["out_path"]),
                    _ptr(h["out_len"]), trees, nodes, edges, warps, depth)
    return h


def node_select(h, cpuct=1.0, c_pw=1.0, alpha_pw=0.5, variant="preclaim"):
    """Selection with node-level virtual loss (h["node_inflight"]), src/puct/puct_gpu_v2.py:573-840, the traversals one
    after another (tree-major, wid ascending), in place; variant "preclaim" or "winner_recalc"."""
    trees, nodes, edges = h["edge_child"].shape
    warps, depth = h["out_path"].shape[1:]
    for k in ("edge_child", "edge_n", "node_inflight", "node_expand_inflight", "node_expanded", "node_count",
              "out_selected", "out_path", "out_len"):
        assert h[k].dtype == np.int32 and h[k].flags.c_contiguous, k
    for k in ("edge_prior", "edge_w"):
        assert h[k].dtype == np.float32 and h[k].flags.c_contiguous, k
    assert variant in ("preclaim", "winner_recalc")
    lib().po_node_select(int(variant == "preclaim"), cpuct, c_pw, alpha_pw, _ptr(h["edge_child"]), _ptr(h["edge_prior"]),
                         _ptr(h["edge_w"]), _ptr(h["edge_n"]), _ptr(h["node_inflight"]), _ptr(h["node_expand_inflight"]),
                         _ptr(h["node_expanded"]), _ptr(h["node_count"]), _ptr(h["out_selected"]), _ptr(h["out_path"]),
                         _ptr(h["out_len"]), trees, nodes, edges, warps, depth)
    return h


def backup(h, values=None, virtual_loss=1, node_level=False):
    """Edge-level (default) or node-level backup on host arrays, in place; values=None only releases the claims."""
    trees, nodes, edges = h["edge_child"].shape
    warps, depth = h["out_path"].shape[1:]
    if values is not None:
        assert values.dtype == np.float32 and values.shape == h["out_path"].shape and values.flags.c_contiguous
    lib().po_backup(int(node_level), int(virtual_loss), _ptr(h["edge_child"]), _ptr(h["edge_w"]), _ptr(h["edge_n"]),
                    _ptr(h.get("edge_inflight")), _ptr(h.get("node_inflight")), _ptr(h["node_expand_inflight"]),
                    _ptr(h["node_count"]), _ptr(h["out_selected"]), _ptr(h["out_path"]), _ptr(h["out_len"]),
                    _ptr(values), trees, nodes, edges, warps, depth)
    return h


class _GomokuArrays(ctypes.Structure):
    _fields_ = [(n, ctypes.c_void_p) for n in
                ("edge_child", "edge_prior", "edge_w", "edge_n", "edge_inflight", "edge_action", "node_expanded",
                 "node_expand_inflight", "node_count", "node_board", "node_turn", "node_value", "out_selected",
                 "out_path", "out_len", "path_values", "node_legal")]


def gomoku_search(board, turn, steps, trees=16, traversals=16, max_nodes=16384, path_depth=64, cpuct=1.5, c_pw=1.0,
                  alpha_pw=0.5, dirichlet_alpha=0.3, seed=0, threads=8):
    """Gomoku PUCT search on the host (oracle/puct_oracle.c: po_gomoku_search), `threads` trees at a time; returns
    every array plus the tallies."""
    board = np.ascontiguousarray(board, dtype=np.int8)
    m, n = board.shape
    T, N, E, W, D = trees, max_nodes, 256, traversals, path_depth
    h = {
        "edge_child": np.zeros((T, N, E), np.int32), "edge_prior": np.zeros((T, N, E), np.float32),
        "edge_w": np.zeros((T, N, E), np.float32), "edge_n": np.zeros((T, N, E), np.int32),
        "edge_inflight": np.zeros((T, N, E), np.int32), "edge_action": np.zeros((T, N, E), np.uint8),
        "node_expanded": np.zeros((T, N), np.int32), "node_expand_inflight": np.zeros((T, N), np.int32),
        "node_count": np.zeros((T,), np.int32), "node_board": np.zeros((T, N, 16), np.uint32),
        "node_turn": np.zeros((T, N), np.int8), "node_value": np.zeros((T, N), np.float32),
        "out_selected": np.zeros((T, W), np.int32), "out_path": np.full((T, W, D), -1, np.int32),
        "out_len": np.zeros((T, W), np.int32), "path_values": np.zeros((T, W, D), np.float32),
        "node_legal": np.zeros((T, N), np.int32),
    }
    arrays = _GomokuArrays(*[h[name].ctypes.data for name, _ in _GomokuArrays._fields_])
    tally = np.zeros((T, 8), np.int64)
    L = lib()
    L.po_gomoku_search.restype = None
    L.po_gomoku_search.argtypes = [ctypes.POINTER(_GomokuArrays), ctypes.c_void_p] + [ctypes.c_int] * 8 + \
        [ctypes.c_float] * 4 + [ctypes.c_uint64, ctypes.c_int, ctypes.c_void_p]
    L.po_gomoku_search(ctypes.byref(arrays), board.ctypes.data, int(turn), m, n, T, N, W, D, int(steps), cpuct, c_pw,
                       alpha_pw, dirichlet_alpha, int(seed), int(threads), tally.ctypes.data)
    h["tally"] = tally
    return h


def evaluator():
    """The synthetic evaluator's primitives, for the tests that pin them."""
    L = lib()
    for name in ("po_det_expf", "po_det_logf"):
        getattr(L, name).restype = ctypes.c_float
        getattr(L, name).argtypes = [ctypes.c_float]
    L.po_gamma.restype = ctypes.c_float
    L.po_gamma.argtypes = [ctypes.c_float, ctypes.c_uint64]
    L.po_cell_key.restype = ctypes.c_uint32
    L.po_cell_key.argtypes = [ctypes.c_float, ctypes.c_uint64, ctypes.c_int]
    L.po_value.restype = ctypes.c_float
    L.po_value.argtypes = [ctypes.c_uint64]
    L.po_board_hash.restype = ctypes.c_uint64
    L.po_board_hash.argtypes = [ctypes.c_uint64, ctypes.c_int, ctypes.c_void_p]
    L.po_makes_five.restype = ctypes.c_int
    L.po_makes_five.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int]
    return L
