"""Host side of the PUCT select / backup path: a ctypes binding of libpuct_hip.so (C ABI: include/puct_select.h) with
the calling convention of the reference's binding, src/puct/puct_gpu_v3_cpp.py:118-156 — `launch_select(d, ...)` takes
a dictionary of device arrays — here hipmem.DeviceArray objects or torch tensors on the GPU instead of numba device
arrays.  There is no CPU fallback: without the library, or with arrays that are not on the GPU, every call raises.

When torch is used in the same process, import torch before this package: torch ships its own copy of the HIP
runtime, and the copy that is loaded first serves both."""
import ctypes
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libpuct_hip.so")

# packing of the selection word, src/puct/puct_gpu_v3.py:14-48
NODE_EXPANDED_TERMINAL = -1
PACKED_NODE_LIMIT = 16384
PACKED_NODE_MASK = 0x3FFF
PACKED_EDGE_MASK = 0xFF
PACKED_SLOT_SHIFT = 14
PACKED_KIND_SHIFT = 22
PACKED_KIND_MASK = 0x7
PACKED_REASON_SHIFT = 25
SELECT_INVALID, SELECT_EXPAND, SELECT_TERMINAL, SELECT_DEPTH_LIMIT, SELECT_BUSY = range(5)
PACKED_INVALID = (SELECT_INVALID << PACKED_KIND_SHIFT) | PACKED_NODE_MASK
REASON_UNSET, REASON_OK_EXPAND, REASON_OK_TERMINAL, REASON_OK_DEPTH_LIMIT = 0, 1, 2, 3
REASON_BUSY_EXPAND_INFLIGHT, REASON_BUSY_WINNER_RECALC = 4, 5
REASON_INVALID_SHAPE, REASON_INVALID_NODE_INFO, REASON_INVALID_NO_VALID_EDGE = 10, 11, 14
REASON_INVALID_CHILD_OOB, REASON_INVALID_UNKNOWN = 15, 16

_LIB = None


def _lib():
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m mcts_numba_cuda_amd.build` "
                               "(there is no CPU fallback for PUCT select/backup)")
        lib = ctypes.CDLL(LIB_PATH)
        c_void, c_int, c_float = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
        lib.puct_select_winner_recalc_launch.argtypes = [c_float] * 3 + [c_int] + [c_void] * 11 + [c_int] * 5 + [c_void]
        lib.puct_select_winner_recalc_launch.restype = c_int
        lib.puct_cpp_cuda_error_string.argtypes = [c_int]
        lib.puct_cpp_cuda_error_string.restype = ctypes.c_char_p
        lib.puct_edge_backup_launch.argtypes = [c_int] + [c_void] * 9 + [c_int] * 5 + [c_void]
        lib.puct_edge_backup_launch.restype = c_int
        for fn in (lib.puct_node_select_preclaim_launch, lib.puct_node_select_winner_recalc_launch):
            fn.argtypes = [c_float] * 3 + [c_void] * 11 + [c_int] * 5 + [c_void]
            fn.restype = c_int
        lib.puct_node_backup_launch.argtypes = [c_int] + [c_void] * 10 + [c_int] * 5 + [c_void]
        lib.puct_node_backup_launch.restype = c_int
        _LIB = lib
    return _LIB


def is_available():
    try:
        _lib()
        return True
    except (OSError, RuntimeError):
        return False


def decode(raw):
    """(kind, slot, node) of a packed selection word (src/puct/test_puct_gpu_v3.py:78-82)."""
    raw = int(raw)
    return ((raw >> PACKED_KIND_SHIFT) & PACKED_KIND_MASK, (raw >> PACKED_SLOT_SHIFT) & PACKED_EDGE_MASK,
            raw & PACKED_NODE_MASK)


def reason(raw):
    return (int(raw) >> PACKED_REASON_SHIFT) & 0x3F


def _device_ptr(t, dtype, name):
    """Device address of a contiguous array of `dtype`: a hipmem.DeviceArray or a torch tensor on the GPU."""
    from .hipmem import DeviceArray
    if isinstance(t, DeviceArray):
        if t.dtype != np.dtype(dtype):
            raise ValueError(f"{name}: expected {np.dtype(dtype)}, got {t.dtype}")
        return ctypes.c_void_p(t.data_ptr())
    import torch
    want = {np.int32: torch.int32, np.float32: torch.float32}[dtype]
    if not isinstance(t, torch.Tensor) or not t.is_cuda or t.dtype != want or not t.is_contiguous():
        raise ValueError(f"{name}: expected a contiguous {want} tensor on the GPU")
    return ctypes.c_void_p(t.data_ptr())


def _stream_handle(d):
    """torch's current stream when the arrays are torch tensors, the default stream otherwise."""
    import sys
    torch = sys.modules.get("torch")
    if torch is not None and isinstance(d["edge_child"], torch.Tensor):
        return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    return ctypes.c_void_p(0)


def _check(code, what):
    if code != 0:
        msg = _lib().puct_cpp_cuda_error_string(code).decode("utf-8", "replace")
        raise RuntimeError(f"PUCT {what} launch failed: {msg} ({code})")


def _shape(d):
    trees, nodes, edges = d["edge_child"].shape
    warps, path_depth = d["out_path"].shape[1], d["out_path"].shape[2]
    if tuple(d["out_selected"].shape) != (trees, warps) or tuple(d["out_len"].shape) != (trees, warps):
        raise ValueError("out_selected / out_len must have shape [trees, warps]")
    for k in ("edge_prior", "edge_w", "edge_n", "edge_inflight"):
        if k in d and tuple(d[k].shape) != (trees, nodes, edges):
            raise ValueError(f"{k} must have shape [trees, nodes, edges]")
    for k in ("node_expand_inflight", "node_expanded", "node_inflight"):
        if k in d and tuple(d[k].shape) != (trees, nodes):
            raise ValueError(f"{k} must have shape [trees, nodes]")
    if tuple(d["node_count"].shape) != (trees,):
        raise ValueError("node_count must have shape [trees]")
    return trees, nodes, edges, warps, path_depth


def launch_select(d, cpuct=1.0, c_pw=1.0, alpha_pw=0.5, soft_winner=0):
    """Asynchronous PUCT selection on torch's current stream (src/puct/puct_gpu_v3_cpp.py:118-156)."""
    trees, nodes, edges, warps, path_depth = _shape(d)
    i32, f32 = np.int32, np.float32
    code = _lib().puct_select_winner_recalc_launch(
        cpuct, c_pw, alpha_pw, int(soft_winner),
        _device_ptr(d["edge_child"], i32, "edge_child"), _device_ptr(d["edge_prior"], f32, "edge_prior"),
        _device_ptr(d["edge_w"], f32, "edge_w"), _device_ptr(d["edge_n"], i32, "edge_n"),
        _device_ptr(d["edge_inflight"], i32, "edge_inflight"),
        _device_ptr(d["node_expand_inflight"], i32, "node_expand_inflight"),
        _device_ptr(d["node_expanded"], i32, "node_expanded"), _device_ptr(d["node_count"], i32, "node_count"),
        _device_ptr(d["out_selected"], i32, "out_selected"), _device_ptr(d["out_path"], i32, "out_path"),
        _device_ptr(d["out_len"], i32, "out_len"), trees, nodes, edges, warps, path_depth, _stream_handle(d))
    _check(code, "select")


VARIANT_PRECLAIM, VARIANT_WINNER_RECALC = "preclaim", "winner_recalc"   # src/puct/test_puct_gpu_v2.py:317-352


def launch_node_select(d, cpuct=1.0, c_pw=1.0, alpha_pw=0.5, variant=VARIANT_PRECLAIM):
    """Asynchronous PUCT selection with node-level virtual loss (d["node_inflight"], int32 [trees, nodes]): the two
    kernels of src/puct/puct_gpu_v2.py:573-840, chosen by `variant` as in the reference's launch helper
    (src/puct/test_puct_gpu_v2.py:317-352).  Selection words have the v2 layout (no reason field, no BUSY kind)."""
    trees, nodes, edges, warps, path_depth = _shape(d)
    i32, f32 = np.int32, np.float32
    if variant == VARIANT_PRECLAIM:
        fn = _lib().puct_node_select_preclaim_launch
    elif variant == VARIANT_WINNER_RECALC:
        fn = _lib().puct_node_select_winner_recalc_launch
    else:
        raise ValueError(f"unknown select variant: {variant}")
    code = fn(cpuct, c_pw, alpha_pw,
              _device_ptr(d["edge_child"], i32, "edge_child"), _device_ptr(d["edge_prior"], f32, "edge_prior"),
              _device_ptr(d["edge_w"], f32, "edge_w"), _device_ptr(d["edge_n"], i32, "edge_n"),
              _device_ptr(d["node_inflight"], i32, "node_inflight"),
              _device_ptr(d["node_expand_inflight"], i32, "node_expand_inflight"),
              _device_ptr(d["node_expanded"], i32, "node_expanded"), _device_ptr(d["node_count"], i32, "node_count"),
              _device_ptr(d["out_selected"], i32, "out_selected"), _device_ptr(d["out_path"], i32, "out_path"),
              _device_ptr(d["out_len"], i32, "out_len"), trees, nodes, edges, warps, path_depth, _stream_handle(d))
    _check(code, "node select")


def launch_edge_backup(d, path_edge_values=None, virtual_loss=1):
    """Releases the edge-level claims of launch_select; with `path_edge_values` (float32 [trees, warps, path_depth],
    already in the perspective of each edge's owner) it also adds one visit and the value to every path edge."""
    trees, nodes, edges, warps, path_depth = _shape(d)
    i32, f32 = np.int32, np.float32
    values = ctypes.c_void_p(0)
    if path_edge_values is not None:
        if tuple(path_edge_values.shape) != (trees, warps, path_depth):
            raise ValueError("path_edge_values must have shape [trees, warps, path_depth]")
        values = _device_ptr(path_edge_values, f32, "path_edge_values")
    code = _lib().puct_edge_backup_launch(
        int(virtual_loss), _device_ptr(d["edge_w"], f32, "edge_w"), _device_ptr(d["edge_n"], i32, "edge_n"),
        _device_ptr(d["edge_inflight"], i32, "edge_inflight"),
        _device_ptr(d["node_expand_inflight"], i32, "node_expand_inflight"),
        _device_ptr(d["node_count"], i32, "node_count"), _device_ptr(d["out_selected"], i32, "out_selected"),
        _device_ptr(d["out_path"], i32, "out_path"), _device_ptr(d["out_len"], i32, "out_len"), values,
        trees, nodes, edges, warps, path_depth, _stream_handle(d))
    _check(code, "edge backup")


def launch_node_backup(d, path_edge_values, virtual_loss=1):
    """Backup with node-level virtual loss (d["node_inflight"]), src/puct/puct_gpu_v2.py:847-927."""
    trees, nodes, edges, warps, path_depth = _shape(d)
    i32, f32 = np.int32, np.float32
    if tuple(path_edge_values.shape) != (trees, warps, path_depth):
        raise ValueError("path_edge_values must have shape [trees, warps, path_depth]")
    code = _lib().puct_node_backup_launch(
        int(virtual_loss), _device_ptr(d["edge_child"], i32, "edge_child"), _device_ptr(d["edge_w"], f32, "edge_w"),
        _device_ptr(d["edge_n"], i32, "edge_n"), _device_ptr(d["node_inflight"], i32, "node_inflight"),
        _device_ptr(d["node_expand_inflight"], i32, "node_expand_inflight"),
        _device_ptr(d["node_count"], i32, "node_count"), _device_ptr(d["out_selected"], i32, "out_selected"),
        _device_ptr(d["out_path"], i32, "out_path"), _device_ptr(d["out_len"], i32, "out_len"),
        _device_ptr(path_edge_values, f32, "path_edge_values"), trees, nodes, edges, warps, path_depth,
        _stream_handle(d))
    _check(code, "node backup")
