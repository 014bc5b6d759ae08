"""The two complete MCTSNC runs the reference prints in its README.md (Connect 4: 8 trees x 128 playouts, all-children
playouts, 6373 steps from a mid-game position with two full columns; Gomoku 15x15: same engine settings, 442 steps
from a position with 15 stones), kept as data in tests/golden/readme_examples.json.

They are the reference's only recorded Gomoku search and its only recorded search with these settings, so they pin
what the Connect 4 archives leave open: the Gomoku playout mechanics (row-major legal list, swap-remove order,
exactly-five rule), the random stream layout with 225 actions, and the final reduction over 225 actions.  The CPU
tests run the oracle on them; the GPU tests run the engine on them directly, without the oracle in between."""
import json
import math
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
THREADS = min(8, os.cpu_count() or 1)
SHAPES = {"c4": ((6, 7), 7, 7), "gomoku": ((15, 15), 1, 225)}


def load(name):
    with open(os.path.join(GOLDEN, "readme_examples.json")) as f:
        ex = json.load(f)[name]
    board = np.array([[{"X": 1, "O": -1, ".": 0}[ch] for ch in row] for row in ex["board_rows"]], dtype=np.int8)
    assert board.shape == SHAPES[name][0]
    if name == "c4":
        extra = (board != 0).sum(axis=0).astype(np.int8)   # column fills (src/c4.py:24-47)
    else:
        extra = None
    return ex, board, extra


def check_against_printout(ex, steps, best, n_root, actions, trees):
    """actions: {action: (n, n_wins, win_flag)} for every root action the engine reports."""
    assert steps == ex["steps"]
    assert n_root == ex["playouts"] == ex["best"]["n_root"]
    shown = {int(a): row for a, row in ex["actions"].items()}
    if not ex["rows_elided"]:
        assert sorted(actions) == sorted(shown)
    for a, row in shown.items():
        assert a in actions, f"root action {a} missing"
        n, n_wins, win_flag = actions[a]
        assert (n, n_wins, bool(win_flag)) == (row["n"], row["n_wins"], row["win_flag"]), f"action {a}: {(n, n_wins, win_flag)} vs {row}"
        assert row["n_root"] == n_root
        q = n_wins / n
        assert q == row["q"]                                   # plain double division on both sides (src/mctsnc.py:522)
        ucb = q + ex["params"]["ucb_c"] * math.sqrt(math.log(n_root) / n)
        assert abs(ucb - row["ucb"]) <= 4e-16 * max(1.0, abs(ucb))   # libm log/sqrt of the printing machine: last bit at most
    assert best == ex["best"]["index"]
    assert actions[best][:2] == (ex["best"]["n"], ex["best"]["n_wins"])
    assert trees["max_depth"] == ex["trees"]["max_depth"] and trees["max_size"] == ex["trees"]["max_size"]
    assert trees["mean_size"] == ex["trees"]["mean_size"]
    assert abs(trees["mean_depth"] - ex["trees"]["mean_depth"]) <= 1e-15 * ex["trees"]["mean_depth"]


# ---- CPU: the oracle reproduces the printouts ------------------------------------------------------------------------

def run_oracle(name):
    import replay
    from oracle.oracle import Oracle
    ex, board, extra = load(name)
    p = ex["params"]
    shape, E, A = SHAPES[name]
    o = Oracle(name, shape, E, A, p["n_trees"], p["n_playouts"], p["variant"], ucb_c=p["ucb_c"], seed=p["seed"],
               device_memory=p["device_memory"], threads=THREADS)
    assert o.S == ex["max_tree_size"]   # "calculated max_tree_size" of the printout
    res = replay.oracle_run_search(o, board, extra, ex["turn"], ex["steps"])
    check_against_printout(ex, ex["steps"], res["best"], res["n_root"], res["actions"], res["trees"])
    return o


def test_oracle_reproduces_readme_c4_run():
    run_oracle("c4")


@pytest.mark.slow
def test_oracle_reproduces_readme_gomoku_run():
    """About a minute and a half on 8 host threads (94 million Gomoku playouts)."""
    o = run_oracle("gomoku")
    assert o.u1_events >= 0


# ---- GPU: the engine reproduces the printouts ------------------------------------------------------------------------

def run_engine(name, **kw):
    from helpers import engine_result
    from mcts_numba_cuda_amd import MCTSNC
    ex, board, extra = load(name)
    p = ex["params"]
    shape, E, A = SHAPES[name]
    e = MCTSNC(shape, E if name == "c4" else 0, A, search_time_limit=np.inf, search_steps_limit=ex["steps"], n_trees=p["n_trees"],
               n_playouts=p["n_playouts"], variant=p["variant"], device_memory=p["device_memory"], ucb_c=p["ucb_c"], seed=p["seed"],
               verbose_info=False, game=name, **kw)
    e.init_device_side_arrays()
    assert e.max_tree_size == ex["max_tree_size"]
    assert e._per_state_memory()[0] == ex["per_state_memory"]
    best = e.run(board, extra, ex["turn"])
    res = engine_result(e)
    check_against_printout(ex, e.steps, int(best), res["n_root"], res["actions"], res["trees"])
    assert e.performance_info["playouts"] == ex["playouts"]
    return e


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["c4", "gomoku"])
def test_engine_reproduces_readme_run(name):
    e = run_engine(name)
    if name == "gomoku":   # the whole printed table: 210 empty cells, all expanded by every tree
        assert len([a for a in e.actions_info if a != "best"]) == 210


@pytest.mark.gpu
def test_engine_reproduces_readme_gomoku_run_as_thrifty():
    """acp_thrifty builds the same trees (src/mctsnc.py:1938 keeps the stream indices equal); only the indexing of the
    root table differs, and the Python layer maps it back to actions."""
    from helpers import engine_result
    from mcts_numba_cuda_amd import MCTSNC
    ex, board, extra = load("gomoku")
    p = ex["params"]
    e = MCTSNC((15, 15), 0, 225, search_time_limit=np.inf, search_steps_limit=ex["steps"], n_trees=p["n_trees"], n_playouts=p["n_playouts"],
               variant="acp_thrifty", device_memory=p["device_memory"], ucb_c=p["ucb_c"], seed=p["seed"], verbose_info=False, game="gomoku")
    e.init_device_side_arrays()
    best = e.run(board, extra, ex["turn"])
    res = engine_result(e)
    check_against_printout(ex, e.steps, int(best), res["n_root"], res["actions"], res["trees"])
