"""GPU parity tests: the HIP engine (through the C ABI / the MCTSNC class) against the reference's recorded
results and against the CPU oracle, bit-exact for every integer array."""
import os

import numpy as np
import pytest

import replay
from helpers import engine_run_search, make_engine, random_c4_root, compare_with_oracle

pytestmark = pytest.mark.gpu

GOLDEN = replay.GOLDEN


@pytest.mark.parametrize("variant", ["ocp_thrifty", "acp_thrifty"])
def test_reference_tree_dump_1000_steps(variant):
    """extras/mctsnc_<variant>_c4_1000steps.json of the reference: T=4, P=128, seed 0, empty board, 1000 steps."""
    d = np.load(os.path.join(GOLDEN, f"dump_{variant}_c4_1000steps.npz"))
    e = make_engine(dict(n_trees=4, n_playouts=128, variant=variant, device_memory=1.5, ucb_c=2.0, seed=0))
    assert e.max_tree_size == 4238367  # logged by the reference for this configuration
    e.run(np.zeros((6, 7), np.int8), np.zeros(7, np.int8), 1, forced_search_steps_limit=1000)
    for ti in range(4):
        sz = int(d["trees_sizes"][ti])
        assert e.read_array("depths", ti).shape[0] == sz
        np.testing.assert_array_equal(e.read_array("trees", ti), d[f"trees_{ti}"])
        np.testing.assert_array_equal(e.read_array("depths", ti), d[f"depths_{ti}"])
        np.testing.assert_array_equal(e.read_array("turns", ti), d[f"turns_{ti}"])
        np.testing.assert_array_equal(e.read_array("ns", ti), d[f"ns_{ti}"])
        np.testing.assert_array_equal(e.read_array("ns_wins", ti), d[f"ns_wins_{ti}"])
        path = e.read_array("selected_path", ti)
        gp = d["selected_paths"][ti]
        assert gp[-1] == path.size and list(gp[:path.size]) == list(path)
        assert int(e.read_array("node_selected", ti)[0]) == int(d["nodes_selected"][ti])
        np.testing.assert_array_equal(e.read_array("actions_expanded", ti), d["actions_expanded"][ti])
        np.testing.assert_array_equal(e.read_array("playout_outcomes", ti), d["playout_outcomes"][ti])
        if "playout_outcomes_children" in d:
            np.testing.assert_array_equal(e.read_array("playout_outcomes_children", ti), d["playout_outcomes_children"][ti])


def test_north_star_a100_game(archives):
    """Game 1 of the reference's A100 experiment with acp_prodigal 4x256 (5 s per move): every search's root table,
    best action and tree statistics, with the random streams carried from search to search."""
    key = replay.find_archive(archives, "mcts_5_inf_vanilla", "mctsnc_5_inf_4_256_acp_prodigal")
    n = replay.replay_archive(archives[key], make_engine, engine_run_search, max_games=1)
    assert n >= 10


ARCHIVE_PAIRS = [
    ("mcts_5_inf_vanilla", "mctsnc_1_inf_1_32_ocp_thrifty"),
    ("mcts_5_inf_vanilla", "mctsnc_1_inf_2_64_ocp_prodigal"),
    ("mcts_5_inf_vanilla", "mctsnc_1_inf_8_256_ocp_thrifty"),
    ("mcts_5_inf_vanilla", "mctsnc_1_inf_8_256_acp_thrifty"),
    ("mcts_5_inf_vanilla", "mctsnc_1_inf_8_256_acp_prodigal"),
    ("mcts_5_inf_vanilla", "mctsnc_1_inf_1_128_acp_prodigal"),
    ("mcts_5_inf_vanilla", "mctsnc_1_inf_4_32_acp_thrifty"),
    ("mcts_5_inf_vanilla", "mctsnc_5_inf_4_256_ocp_prodigal"),
    ("mcts_5_inf_vanilla", "mctsnc_5_inf_4_128_ocp_thrifty"),
    ("mcts_5_inf_vanilla", "mctsnc_5_inf_4_256_acp_thrifty"),
    ("mctsnc_5_inf_4_128_ocp_thrifty", "mctsnc_5_inf_4_256_acp_prodigal"),
    ("mctsnc_10_inf_4_512_acp_thrifty", "mctsnc_10_inf_4_512_acp_prodigal"),
]


@pytest.mark.parametrize("pair", ARCHIVE_PAIRS, ids=lambda p: p[1] if p[0].startswith("mcts_5") else f"{p[0]}-vs-{p[1]}")
def test_recorded_games(archives, pair):
    key = replay.find_archive(archives, *pair)
    n = replay.replay_archive(archives[key], make_engine, engine_run_search)
    assert n >= 5


@pytest.mark.parametrize("variant", ["ocp_thrifty", "ocp_prodigal", "acp_thrifty", "acp_prodigal"])
@pytest.mark.parametrize("T,P", [(1, 32), (3, 64), (4, 256), (9, 128)])
def test_against_oracle_full_state(variant, T, P):
    """Same seeded roots and step budgets through the oracle and the engine: every per-node array, the step scratch,
    the reduced root table and the random streams afterwards must agree; two runs in a row check the carry-over."""
    rng = np.random.default_rng(1234 + T * 1000 + P)
    params = dict(n_trees=T, n_playouts=P, variant=variant, device_memory=0.25, ucb_c=2.0, seed=7)
    e = make_engine(params)
    from oracle.oracle import Oracle
    o = Oracle("c4", (6, 7), 7, 7, T, P, variant, ucb_c=2.0, seed=7, device_memory=0.25, threads=8)
    for run, plies in enumerate([8, 24]):
        board, fills, turn = random_c4_root(rng, plies)
        compare_with_oracle(e, o, board, fills, turn, steps=150 if P >= 256 else 300)
