"""The benchmark configurations at their full sizes, engine against oracle: every node of every tree, the step scratch,
the reduced root tables and the random streams must agree after the whole search (Connect 4 1x32 ocp_thrifty, 1000
steps; Connect 4 8x256 acp_thrifty, 20000 steps, 16 GiB pools; Gomoku 15x15 4x128 ocp_thrifty, 2000 steps, 16 GiB
pools).  The fourth configuration (Connect 4 4x256 acp_prodigal, 5000 steps) is covered by the recorded A100 games."""
import numpy as np
import pytest

from helpers import compare_with_oracle, make_engine, random_c4_root, random_gomoku_root
from oracle.oracle import Oracle

pytestmark = pytest.mark.gpu


def test_c4_ocp_thrifty_1x32_1000_steps_after_six_random_plies():
    params = dict(n_trees=1, n_playouts=32, variant="ocp_thrifty", device_memory=2.0, ucb_c=2.0, seed=0)
    board, fills, turn = random_c4_root(np.random.default_rng(0), 6)
    e = make_engine(params)
    o = Oracle("c4", (6, 7), 7, 7, 1, 32, "ocp_thrifty", ucb_c=2.0, seed=0, device_memory=2.0, threads=4)
    compare_with_oracle(e, o, board, fills, turn, steps=1000)
    assert e.performance_info["playouts"] == 1000 * 32


def test_c4_acp_thrifty_8x256_20000_steps_empty_board():
    params = dict(n_trees=8, n_playouts=256, variant="acp_thrifty", device_memory=16.0, ucb_c=2.0, seed=0)
    e = make_engine(params)
    assert e.max_tree_size == 16777216            # the reference's cap (src/mctsnc.py:357-358)
    o = Oracle("c4", (6, 7), 7, 7, 8, 256, "acp_thrifty", ucb_c=2.0, seed=0, device_memory=16.0, threads=16)
    board, fills = np.zeros((6, 7), np.int8), np.zeros(7, np.int8)
    compare_with_oracle(e, o, board, fills, 1, steps=20000)
    trees = e.performance_info["trees"]
    assert trees["max_size"] > 100000 and trees["max_depth"] > 30


def test_gomoku_ocp_thrifty_4x128_2000_steps():
    params = dict(n_trees=4, n_playouts=128, variant="ocp_thrifty", device_memory=16.0, ucb_c=2.0, seed=0)
    board, turn = random_gomoku_root(np.random.default_rng(7), 15, 15, 12)
    e = make_engine(params, board_shape=(15, 15), extra=0, actions=225)
    o = Oracle("gomoku", (15, 15), 0, 225, 4, 128, "ocp_thrifty", ucb_c=2.0, seed=0, device_memory=16.0, threads=16)
    compare_with_oracle(e, o, board, None, turn, steps=2000)
    assert e.performance_info["playouts"] == 2000 * 4 * 128
