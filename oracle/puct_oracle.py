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
