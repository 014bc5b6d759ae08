"""mctsnc_run_batch_noalloc -- the batched search for callers that must not allocate device memory -- against
mctsnc_run_batch, through the C ABI: identical results (every integer of the result structs, the trees' visit
counters, the carried random streams) on two calls in a row, the second with a smaller batch, which finds the
library's static scratch still holding the first call's buffers.  Collected last on purpose."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

INT_FIELDS = ["steps", "best_action", "best_win_flag", "best_n", "best_n_wins", "n_root_entries", "depth_sum", "size_sum", "max_depth",
              "max_size", "playout_plies", "u1_events", "stat_levels", "stat_children", "stat_expanded", "stat_played"]
ARRAY_FIELDS = ["root_actions_expanded", "root_ns", "actions_ns", "actions_ns_wins", "actions_win_flags"]


def engines_for(game, n, variant, n_trees, n_playouts):
    from mcts_numba_cuda_amd import MCTSNC
    out = []
    for _ in range(n):
        if game == "c4":
            e = MCTSNC((6, 7), 7, 7, search_time_limit=np.inf, search_steps_limit=np.inf, n_trees=n_trees, n_playouts=n_playouts, variant=variant,
                       device_memory=0.05, seed=3, verbose_info=False)
        else:
            e = MCTSNC((9, 9), 0, 81, search_time_limit=np.inf, search_steps_limit=np.inf, n_trees=n_trees, n_playouts=n_playouts, variant=variant,
                       device_memory=0.05, seed=3, verbose_info=False, game="gomoku")
        e.init_device_side_arrays()
        out.append(e)
    return out


def roots_for(game, n, seed):
    from helpers import random_c4_root, random_gomoku_root
    rng = np.random.default_rng(seed)
    boards, extras, turns = [], [], []
    for i in range(n):
        if game == "c4":
            b, f, t = random_c4_root(rng, 4 + i % 9)
        else:
            b, t = random_gomoku_root(rng, 9, 9, i % 7)
            f = np.zeros(1, np.int8)
        boards.append(b); extras.append(f); turns.append(t)
    return np.ascontiguousarray(np.stack(boards)), np.ascontiguousarray(np.stack(extras)), np.asarray(turns, np.int32)


def call(entry_name, engines, boards, extras, turns, steps):
    """One call of a batch entry point through the C ABI; returns the result structs."""
    from mcts_numba_cuda_amd import _lib
    L = _lib.lib()
    n = len(engines)
    handles = (ctypes.c_void_p * n)(*[e._engine for e in engines])
    results = (_lib.Result * n)()
    rc = getattr(L, entry_name)(handles, n, boards.ctypes.data, extras.ctypes.data, extras.shape[1], turns.ctypes.data,
                                float("inf"), float("inf"), float(steps), results)
    return rc, results


def assert_same(res_a, res_b, engines_a, engines_b, label):
    for i, (a, b) in enumerate(zip(res_a, res_b)):
        for f in INT_FIELDS:
            assert getattr(a, f) == getattr(b, f), f"{label}: search {i}, {f}: {getattr(a, f)} != {getattr(b, f)}"
        for f in ARRAY_FIELDS:
            np.testing.assert_array_equal(np.ctypeslib.as_array(getattr(a, f)), np.ctypeslib.as_array(getattr(b, f)), err_msg=f"{label}: search {i}, {f}")
    for i, (ea, eb) in enumerate(zip(engines_a, engines_b)):
        for t in range(ea.n_trees):
            for arr in ("ns", "ns_wins", "trees"):
                np.testing.assert_array_equal(ea.read_array(arr, t), eb.read_array(arr, t), err_msg=f"{label}: search {i}, tree {t}, {arr}")
        np.testing.assert_array_equal(ea.read_array("rng_playout"), eb.read_array("rng_playout"), err_msg=f"{label}: search {i}, random streams")


@pytest.mark.parametrize("game,variant,n_trees,n_playouts,steps", [
    ("c4", "acp_prodigal", 4, 64, 400),
    ("c4", "ocp_thrifty", 3, 32, 300),
    ("gomoku", "acp_thrifty", 2, 64, 12),
    ("gomoku", "ocp_prodigal", 2, 32, 60),
])
def test_two_calls_in_a_row_equal_the_allocating_entry_point(game, variant, n_trees, n_playouts, steps):
    n_first, n_second = 6, 2
    mine = engines_for(game, n_first, variant, n_trees, n_playouts)
    theirs = engines_for(game, n_first, variant, n_trees, n_playouts)
    boards, extras, turns = roots_for(game, n_first, seed=11)
    rc_a, res_a = call("mctsnc_run_batch_noalloc", mine, boards, extras, turns, steps)
    rc_b, res_b = call("mctsnc_run_batch", theirs, boards, extras, turns, steps)
    assert rc_a == 0 and rc_b == 0
    assert_same(res_a, res_b, mine, theirs, "first call")
    # second call: a smaller batch on engines that carry their random streams on, other roots
    boards2, extras2, turns2 = roots_for(game, n_second, seed=12)
    rc_a, res_a = call("mctsnc_run_batch_noalloc", mine[:n_second], boards2, extras2, turns2, steps // 2)
    rc_b, res_b = call("mctsnc_run_batch", theirs[:n_second], boards2, extras2, turns2, steps // 2)
    assert rc_a == 0 and rc_b == 0
    assert_same(res_a, res_b, mine[:n_second], theirs[:n_second], "second call")
    # and a single search (n = 1), which mctsnc_run serves from the engine's own buffers
    rc_a, res_a = call("mctsnc_run_batch_noalloc", mine[:1], boards[:1], extras[:1], turns[:1], steps)
    rc_b, res_b = call("mctsnc_run_batch", theirs[:1], boards[:1], extras[:1], turns[:1], steps)
    assert rc_a == 0 and rc_b == 0
    assert_same(res_a, res_b, mine[:1], theirs[:1], "single search")


def test_a_batch_beyond_the_scratch_is_rejected_with_both_sizes():
    from mcts_numba_cuda_amd import MCTSNC, _lib
    n = 60   # 60 x 512 trees of a 9x9 board need 148 bytes per tree + 2560 per search = 4.7 MB, more than the 4 MiB of the static array
    engines = []
    for _ in range(n):
        e = MCTSNC((9, 9), 0, 81, search_time_limit=np.inf, search_steps_limit=np.inf, n_trees=512, n_playouts=1, variant="ocp_prodigal",
                   device_memory=0.05, verbose_info=False, game="gomoku")
        e.init_device_side_arrays()
        engines.append(e)
    boards = np.zeros((n, 9, 9), np.int8)
    extras = np.zeros((n, 1), np.int8)
    turns = np.ones(n, np.int32)
    rc, _ = call("mctsnc_run_batch_noalloc", engines, boards, extras, turns, 2)
    assert rc == -1
    msg = _lib.lib().mctsnc_last_error().decode()
    assert "bytes of device scratch" in msg and str(4 << 20) in msg
    # the same batch passes through the allocating entry point, and a batch that fits still passes afterwards
    rc, res_b = call("mctsnc_run_batch", engines, boards, extras, turns, 2)
    assert rc == 0
    for e in engines:
        e.reseed()
    rc, res_a = call("mctsnc_run_batch_noalloc", engines[:50], boards[:50], extras[:50], turns[:50], 2)
    assert rc == 0
    for a, b in zip(res_a, res_b):   # every engine has the same seed and root: one result, whichever entry point
        for f in INT_FIELDS:
            assert getattr(a, f) == getattr(b, f), f
