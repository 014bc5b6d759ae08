"""The CPU oracle against the reference's own recorded results (no GPU needed).

These are the vectors that pin the oracle: full tree dumps after 1000 steps and the root tables / tree statistics
logged by the reference's A100 experiments, replayed in order so that the random streams carry over as they did."""
import os

import numpy as np
import pytest

import replay
from oracle.oracle import Oracle

GOLDEN = replay.GOLDEN
THREADS = min(8, os.cpu_count() or 1)


def make_oracle(p):
    return Oracle("c4", (6, 7), 7, 7, p["n_trees"], p["n_playouts"], p["variant"], ucb_c=p["ucb_c"], seed=p["seed"],
                  device_memory=p["device_memory"], threads=THREADS)


@pytest.mark.parametrize("variant", ["ocp_thrifty", "acp_thrifty"])
def test_reference_tree_dump_1000_steps(variant):
    d = np.load(os.path.join(GOLDEN, f"dump_{variant}_c4_1000steps.npz"))
    o = make_oracle(dict(n_trees=4, n_playouts=128, variant=variant, device_memory=1.5, ucb_c=2.0, seed=0))
    assert o.S == 4238367  # "calculated max_tree_size" in the reference's log of this run
    o.run(np.zeros((6, 7), np.int8), np.zeros(7, np.int8), 1, 1000)
    for ti in range(4):
        sz = int(d["trees_sizes"][ti])
        assert o.tree_size(ti) == sz
        mine = o.tree(ti, "trees")
        leaves = o.tree(ti, "leaves").astype(bool)
        mine[leaves, 1:] = -1
        np.testing.assert_array_equal(mine, d[f"trees_{ti}"])
        np.testing.assert_array_equal(o.tree(ti, "depths"), d[f"depths_{ti}"])
        np.testing.assert_array_equal(o.tree(ti, "turns"), d[f"turns_{ti}"])
        np.testing.assert_array_equal(o.tree(ti, "ns"), d[f"ns_{ti}"])
        np.testing.assert_array_equal(o.tree(ti, "ns_wins"), d[f"ns_wins_{ti}"])
        p = o.tree(ti, "path")
        gp = d["selected_paths"][ti]
        assert gp[-1] == p[-1] and list(gp[:p[-1]]) == list(p[:p[-1]])
        assert o.tree_selected(ti) == int(d["nodes_selected"][ti])
        np.testing.assert_array_equal(o.tree(ti, "actions_expanded"), d["actions_expanded"][ti])
        np.testing.assert_array_equal(o.tree(ti, "playout_outcomes"), d["playout_outcomes"][ti])
        if "playout_outcomes_children" in d:
            np.testing.assert_array_equal(o.tree(ti, "playout_outcomes_children"), d["playout_outcomes_children"][ti])


def test_dump_root_tables_match_reference_logs():
    """Reduced root tables printed in extras/mctsnc_{ocp,acp}_thrifty_c4_1000steps.log."""
    o = make_oracle(dict(n_trees=4, n_playouts=128, variant="ocp_thrifty", device_memory=1.5, ucb_c=2.0, seed=0))
    assert o.run(np.zeros((6, 7), np.int8), np.zeros(7, np.int8), 1, 1000) == 3
    assert (o.best["n"], o.best["n_wins"]) == (425856, 266268)
    o = make_oracle(dict(n_trees=4, n_playouts=128, variant="acp_thrifty", device_memory=1.5, ucb_c=2.0, seed=0))
    assert o.run(np.zeros((6, 7), np.int8), np.zeros(7, np.int8), 1, 1000) == 3
    assert (o.best["n"], o.best["n_wins"]) == (3309184, 2005327)
    assert int(o.result("root_ns")[0]) == 3581056
    np.testing.assert_array_equal(o.result("actions_ns"), [20224, 41728, 70400, 3309184, 76672, 45312, 17536])
    np.testing.assert_array_equal(o.result("actions_ns_wins"), [10191, 22289, 38687, 2005327, 42600, 24504, 8710])


def test_north_star_first_two_searches(archives):
    """acp_prodigal 4x256 on the A100: searches 1 and 2 of game 1 (5081 and 5027 steps, about 35 M playouts each,
    the second with the random streams left by the first; several draws round to 1.0f on the way)."""
    key = replay.find_archive(archives, "mcts_5_inf_vanilla", "mctsnc_5_inf_4_256_acp_prodigal")
    assert archives[key]["max_tree_sizes_logged"] == [5651185]
    engines = []

    def mk(p):
        engines.append(make_oracle(p))
        assert engines[-1].S == 5651185
        return engines[-1]
    assert replay.replay_archive(archives[key], mk, replay.oracle_run_search, max_games=1, max_searches=2) == 2
    assert engines[0].u1_events > 0


CHEAP = ["mctsnc_1_inf_1_32_ocp_thrifty", "mctsnc_1_inf_2_32_ocp_prodigal", "mctsnc_1_inf_2_64_acp_thrifty",
         "mctsnc_1_inf_1_64_acp_prodigal", "mctsnc_1_inf_4_64_ocp_thrifty", "mctsnc_1_inf_8_32_acp_prodigal",
         "mctsnc_1_inf_4_128_ocp_prodigal", "mctsnc_1_inf_1_256_acp_thrifty"]


@pytest.mark.parametrize("name", CHEAP)
def test_recorded_games_all_variants(archives, name):
    """Whole recorded games (every search from the first move to the decided end game, win flags and terminal
    selections included) for each variant; for four configurations several consecutive games, which checks that the
    streams carry over from game to game."""
    key = replay.find_archive(archives, "mcts_5_inf_vanilla", name)
    n = replay.replay_archive(archives[key], make_oracle, replay.oracle_run_search)
    assert n >= 7 * len(archives[key]["games"])


def test_logged_pool_sizes(archives):
    """max_tree_size printed by the reference for every archived configuration equals the restated sizing formula."""
    from oracle.oracle import max_tree_size
    checked = 0
    for key, entry in archives.items():
        insts = list(entry["engines"].values())
        logged = entry["max_tree_sizes_logged"]
        if len(logged) != len(insts):
            continue
        mine = sorted(max_tree_size((6, 7), 7, 7, p["n_trees"], p["variant"], p["device_memory"]) for p in insts)
        assert mine == sorted(logged), key
        checked += 1
    assert checked > 60
