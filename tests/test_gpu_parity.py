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


@pytest.mark.parametrize("variant", ["ocp_thrifty", "acp_thrifty"])
def test_json_dump_equals_reference_dump(variant, tmp_path):
    """MCTSNC._json_dump (src/mctsnc.py:2377-2462) of the same run, condensed by the routine that condensed the
    reference's own dump file into the fixture: every array and the recorded parameters come out identical."""
    import importlib.util
    from mcts_numba_cuda_amd import MCTSNC
    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(GOLDEN, "make_fixtures.py"))
    make_fixtures = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(make_fixtures)
    e = MCTSNC((6, 7), 7, 7, search_time_limit=np.inf, search_steps_limit=1000, n_trees=4, n_playouts=128, variant=variant,
               device_memory=1.5, ucb_c=2.0, seed=0, verbose_info=False)
    e.init_device_side_arrays()
    e.run(np.zeros((6, 7), np.int8), np.zeros(7, np.int8), 1)
    e._json_dump(str(tmp_path / "dump.json"))
    make_fixtures.condense_dump(str(tmp_path / "dump.json"), str(tmp_path / "dump.npz"))
    mine, ref = np.load(tmp_path / "dump.npz"), np.load(os.path.join(GOLDEN, f"dump_{variant}_c4_1000steps.npz"))
    assert sorted(mine.files) == sorted(ref.files)
    for key in ref.files:
        if key == "selected_paths":     # entries past a path's length are whatever earlier steps left there
            for ti in range(4):
                length = int(ref[key][ti, -1])
                assert int(mine[key][ti, -1]) == length
                np.testing.assert_array_equal(mine[key][ti, :length], ref[key][ti, :length])
        else:
            np.testing.assert_array_equal(mine[key], ref[key], err_msg=key)


def test_north_star_a100_game(archives):
    """Game 1 of the reference's A100 experiment with acp_prodigal 4x256 (5 s per move): every search's root table,
    best action and tree statistics, with the random streams carried from search to search."""
    key = replay.find_archive(archives, "mcts_5_inf_vanilla", "mctsnc_5_inf_4_256_acp_prodigal")
    n = replay.replay_archive(archives[key], make_engine, engine_run_search, max_games=1)
    assert n >= 10


def test_north_star_whole_experiment():
    """All 100 games of that experiment, 1362 searches with 7.4 million MCTS steps in the recorded order: the engine's
    random streams run on from search to search and from game to game as the reference's single instance did."""
    entry = replay.load_whole_experiment()
    assert len(entry["games"]) == 100
    n = replay.replay_archive(entry, make_engine, engine_run_search)
    assert n == 1362


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


def test_first_recorded_game_of_every_archive(archives):
    """The reference's experiments cover every (variant, n_trees, n_playouts) combination it was run with on
    Connect 4; the first game of each archive (root tables, best actions and tree statistics of every search, in the
    recorded order and with the recorded step counts) must come out of the HIP engine unchanged."""
    total = 0
    for key in sorted(archives):
        n = replay.replay_archive(archives[key], make_engine, engine_run_search, max_games=1)
        assert n >= 3, key
        total += n
    assert total > 700


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


@pytest.mark.parametrize("variant", ["ocp_thrifty", "ocp_prodigal", "acp_thrifty", "acp_prodigal"])
def test_widest_search_512_trees(variant):
    """n_trees = 512 is the reference's MAX_N_TREES (src/mctsnc.py:195): more trees than the device holds sets of
    workgroups for, so the all-children kernel takes trees from its queue within one search."""
    rng = np.random.default_rng(77)
    params = dict(n_trees=512, n_playouts=32, variant=variant, device_memory=1.0, ucb_c=2.0, seed=5)
    e = make_engine(params)
    from oracle.oracle import Oracle
    o = Oracle("c4", (6, 7), 7, 7, 512, 32, variant, ucb_c=2.0, seed=5, device_memory=1.0, threads=8)
    for plies in (10, 3):
        board, fills, turn = random_c4_root(rng, plies)
        compare_with_oracle(e, o, board, fills, turn, steps=40)


@pytest.mark.parametrize("variant", ["acp_thrifty", "acp_prodigal"])
def test_one_search_of_slightly_more_trees_than_cus(variant):
    """288 trees x 128 playouts: between one and 1.4 trees per CU a single all-children search runs on teams whose
    workgroups play their playouts as a pool of jobs (64 lanes for 128 playouts here)."""
    rng = np.random.default_rng(78)
    params = dict(n_trees=288, n_playouts=128, variant=variant, device_memory=1.0, ucb_c=2.0, seed=5)
    e = make_engine(params)
    from oracle.oracle import Oracle
    o = Oracle("c4", (6, 7), 7, 7, 288, 128, variant, ucb_c=2.0, seed=5, device_memory=1.0, threads=8)
    for plies in (12, 2):
        board, fills, turn = random_c4_root(rng, plies)
        compare_with_oracle(e, o, board, fills, turn, steps=30)


@pytest.mark.parametrize("m,n", [(4, 5), (5, 6), (8, 7), (7, 8), (6, 8), (12, 4), (13, 4), (10, 5)])
@pytest.mark.parametrize("variant", ["ocp_thrifty", "acp_prodigal"])
def test_other_connect4_boards(m, n, variant):
    """Boards other than 6x7 up to what a 64-bit column-major bitboard with one spare row holds: small ones end in
    draws and full columns within a few steps, 7x8 and 8x7 use the last bits, 13 rows is the tallest board."""
    rng = np.random.default_rng(100 * m + n)
    params = dict(n_trees=3, n_playouts=64, variant=variant, device_memory=0.25, ucb_c=2.0, seed=9)
    e = make_engine(params, board_shape=(m, n), extra=n, actions=n)
    from oracle.oracle import Oracle
    o = Oracle("c4", (m, n), n, n, 3, 64, variant, ucb_c=2.0, seed=9, device_memory=0.25, threads=8)
    for plies in (2, m * n // 2):
        board, fills, turn = random_c4_root(rng, plies, m, n)
        compare_with_oracle(e, o, board, fills, turn, steps=250)


@pytest.mark.parametrize("m,n", [(4, 5), (7, 8), (8, 7), (13, 4)])
def test_other_connect4_boards_one_workgroup_per_tree(m, n):
    """The same boards' extremes with every tree searched by a single workgroup (the pool of playout jobs)."""
    rng = np.random.default_rng(100 * m + n + 1)
    params = dict(n_trees=3, n_playouts=64, variant="acp_prodigal", device_memory=0.25, ucb_c=2.0, seed=9)
    e = make_engine(params, board_shape=(m, n), extra=n, actions=n, options=dict(solo_trees=1))
    from oracle.oracle import Oracle
    o = Oracle("c4", (m, n), n, n, 3, 64, "acp_prodigal", ucb_c=2.0, seed=9, device_memory=0.25, threads=8)
    for plies in (2, m * n // 2):
        board, fills, turn = random_c4_root(rng, plies, m, n)
        compare_with_oracle(e, o, board, fills, turn, steps=250)


@pytest.mark.parametrize("variant", ["ocp_thrifty", "ocp_prodigal", "acp_thrifty", "acp_prodigal"])
def test_small_playout_counts_and_exploration_constants(variant):
    """n_playouts below a wavefront (down to one playout per node), ucb_c = 0 (pure exploitation: ties everywhere) and
    other constants, a budget of a single step, on both games."""
    from helpers import random_gomoku_root
    from oracle.oracle import Oracle
    rng = np.random.default_rng(5)
    for P, c in ((1, 2.0), (2, 0.0), (4, 0.5), (16, 7.25)):
        params = dict(n_trees=2, n_playouts=P, variant=variant, device_memory=0.25, ucb_c=c, seed=13)
        e = make_engine(params)
        o = Oracle("c4", (6, 7), 7, 7, 2, P, variant, ucb_c=c, seed=13, device_memory=0.25, threads=8)
        for plies, steps in ((6, 1), (14, 300)):
            board, fills, turn = random_c4_root(rng, plies)
            compare_with_oracle(e, o, board, fills, turn, steps=steps)
    for P, c in ((1, 2.0), (8, 0.0), (16, 1.0)):
        params = dict(n_trees=2, n_playouts=P, variant=variant, device_memory=0.5, ucb_c=c, seed=13)
        e = make_engine(params, board_shape=(15, 15), extra=0, actions=225, game="gomoku")
        o = Oracle("gomoku", (15, 15), 0, 225, 2, P, variant, ucb_c=c, seed=13, device_memory=0.5, threads=8)
        for stones, steps in ((3, 1), (10, 30 if variant.startswith("ocp") else 4)):
            board, turn = random_gomoku_root(rng, 15, 15, stones)
            compare_with_oracle(e, o, board, None, turn, steps)


def test_search_ends_before_visit_counters_overflow():
    """512 playouts on each of 7 children add up to 3584 visits of the root per step: its int32 counter (the reference's
    dtype, src/mctsnc.py:334) would overflow after 599 186 steps, which this engine reaches within seconds.  The search
    ends there, whatever the limits say, with every count still exact."""
    from mcts_numba_cuda_amd import MCTSNC
    e = MCTSNC((6, 7), 7, 7, search_time_limit=60.0, search_steps_limit=np.inf, n_trees=1, n_playouts=512, variant="acp_prodigal",
               device_memory=1.0, ucb_c=2.0, seed=1, verbose_info=False)
    e.init_device_side_arrays()
    e.run(np.zeros((6, 7), np.int8), np.zeros(7, np.int8), 1)
    cap = (2**31 - 1) // (512 * 7)
    assert e.steps == cap
    info = e.actions_info
    n_root = info["best"]["n_root"]
    assert 2**30 < n_root <= cap * 512 * 7 < 2**31    # fewer than 7 children deep in the tree
    assert sum(entry["n"] for a, entry in info.items() if a != "best") == n_root
    assert e.time_total < 30.0


@pytest.mark.parametrize("threads", [0, 64, 192, 512], ids=["default-workgroup", "one-wavefront", "three-wavefronts", "eight-wavefronts"])
@pytest.mark.parametrize("variant", ["acp_thrifty", "acp_prodigal"])
def test_one_workgroup_per_tree_gives_the_same_trees(variant, threads):
    """With many trees in one pass the all-children search of a tree is done by a single workgroup instead of one per
    column (option solo_trees sets from how many trees on), which runs all playouts of a step as one pool of jobs that
    its lanes take one after the other (solo_threads overrides its size).  Forced here for small searches: full
    state against the oracle over two runs, a pool that fills up, late-game roots, and a batch against single runs."""
    from mcts_numba_cuda_amd import MCTSNC, run_batch
    from oracle.oracle import Oracle
    forced = dict(solo_trees=1, solo_threads=threads)
    rng = np.random.default_rng(41)
    for T, P, steps in ((3, 64, 300), (4, 256, 150), (2, 16, 200)):
        params = dict(n_trees=T, n_playouts=P, variant=variant, device_memory=0.25, ucb_c=2.0, seed=7)
        e = make_engine(params, options=forced)
        o = Oracle("c4", (6, 7), 7, 7, T, P, variant, ucb_c=2.0, seed=7, device_memory=0.25, threads=8)
        for plies in (8, 24):
            board, fills, turn = random_c4_root(rng, plies)
            compare_with_oracle(e, o, board, fills, turn, steps=steps)
    e = MCTSNC((6, 7), 7, 7, search_time_limit=np.inf, search_steps_limit=np.inf, n_trees=2, n_playouts=64, variant=variant,
               device_memory=2.0, ucb_c=2.0, seed=4, verbose_info=False)
    e.device_memory = float(2 * 95 * 50 + 2 * 8300)  # room for about 50 nodes per tree
    e.init_device_side_arrays()
    for name, value in forced.items():
        e.set_option(name, value)
    o = Oracle("c4", (6, 7), 7, 7, 2, 64, variant, ucb_c=2.0, seed=4, max_tree_size_override=e.max_tree_size, threads=4)
    for plies in (5, 30):
        board, fills, turn = random_c4_root(rng, plies)
        compare_with_oracle(e, o, board, fills, turn, steps=200)
    params = dict(n_trees=4, n_playouts=128, variant=variant, device_memory=0.1, ucb_c=2.0, seed=11)
    roots = [random_c4_root(rng, p) for p in (4, 9, 15, 22, 12)]
    batch = [make_engine(params, options=forced) for _ in roots]
    run_batch(batch, [r[0] for r in roots], [r[1] for r in roots], [r[2] for r in roots], forced_search_steps_limit=400)
    for eb, r in zip(batch, roots):
        es = make_engine(params, options=dict(solo_trees=0))
        es.run(r[0], r[1], r[2], forced_search_steps_limit=400)
        assert eb.actions_info == es.actions_info
        for ti in range(4):
            np.testing.assert_array_equal(eb.read_array("ns", ti), es.read_array("ns", ti))
            np.testing.assert_array_equal(eb.read_array("trees", ti), es.read_array("trees", ti))


@pytest.mark.parametrize("threads", [0, 64, 192], ids=["half-the-playouts", "one-wavefront", "three-wavefronts"])
@pytest.mark.parametrize("variant", ["acp_thrifty", "acp_prodigal"])
def test_teams_with_playout_pools_give_the_same_trees(variant, threads):
    """A pass of a few hundred trees runs teams whose workgroups play their child's playouts as a pool of jobs on fewer
    lanes than playouts (option team_pool forces the form on or off, team_pool_threads sets the lanes).  Forced here
    for small searches: full state against the oracle over two runs, a pool that fills up, late-game roots, a playout
    count smaller than a wavefront, and a batch through the queue against single runs without pools."""
    from mcts_numba_cuda_amd import MCTSNC, run_batch
    from oracle.oracle import Oracle
    forced = dict(team_pool=1, solo_trees=0, team_pool_threads=threads)
    rng = np.random.default_rng(43)
    for T, P, steps in ((3, 64, 300), (4, 256, 150), (2, 16, 200)):
        params = dict(n_trees=T, n_playouts=P, variant=variant, device_memory=0.25, ucb_c=2.0, seed=7)
        e = make_engine(params, options=forced)
        o = Oracle("c4", (6, 7), 7, 7, T, P, variant, ucb_c=2.0, seed=7, device_memory=0.25, threads=8)
        for plies in (8, 24):
            board, fills, turn = random_c4_root(rng, plies)
            compare_with_oracle(e, o, board, fills, turn, steps=steps)
    e = MCTSNC((6, 7), 7, 7, search_time_limit=np.inf, search_steps_limit=np.inf, n_trees=2, n_playouts=64, variant=variant,
               device_memory=2.0, ucb_c=2.0, seed=4, verbose_info=False)
    e.device_memory = float(2 * 95 * 50 + 2 * 8300)  # room for about 50 nodes per tree
    e.init_device_side_arrays()
    for name, value in forced.items():
        e.set_option(name, value)
    o = Oracle("c4", (6, 7), 7, 7, 2, 64, variant, ucb_c=2.0, seed=4, max_tree_size_override=e.max_tree_size, threads=4)
    for plies in (5, 30):
        board, fills, turn = random_c4_root(rng, plies)
        compare_with_oracle(e, o, board, fills, turn, steps=200)
    params = dict(n_trees=4, n_playouts=128, variant=variant, device_memory=0.1, ucb_c=2.0, seed=11)
    roots = [random_c4_root(rng, int(rng.integers(4, 24))) for _ in range(96)]
    batch = [make_engine(params, options=forced) for _ in roots]
    run_batch(batch, [r[0] for r in roots], [r[1] for r in roots], [r[2] for r in roots], forced_search_steps_limit=300)
    es = make_engine(params, options=dict(team_pool=0, solo_trees=0))
    for k in range(0, len(roots), 7):
        eb, r = batch[k], roots[k]
        es.reseed()
        es.run(r[0], r[1], r[2], forced_search_steps_limit=300)
        assert eb.actions_info == es.actions_info
        for ti in range(4):
            np.testing.assert_array_equal(eb.read_array("ns", ti), es.read_array("ns", ti))
            np.testing.assert_array_equal(eb.read_array("trees", ti), es.read_array("trees", ti))


@pytest.mark.parametrize("variant", ["ocp_thrifty", "ocp_prodigal", "acp_thrifty", "acp_prodigal"])
def test_nearly_full_boards(variant):
    """Roots with one to four empty cells on both games (trees of a handful of nodes, every playout a few plies, draws
    by a full board), and a Gomoku root that already holds a five, which neither the reference nor the engine looks
    for (only lines through the last stone placed are tested)."""
    from helpers import random_gomoku_root
    from oracle.oracle import Oracle
    rng = np.random.default_rng(8)
    params = dict(n_trees=2, n_playouts=32, variant=variant, device_memory=0.1, ucb_c=2.0, seed=3)
    e = make_engine(params)
    o = Oracle("c4", (6, 7), 7, 7, 2, 32, variant, ucb_c=2.0, seed=3, device_memory=0.1, threads=4)
    for plies in (38, 40, 41):
        board, fills, turn = random_c4_root(rng, plies)
        compare_with_oracle(e, o, board, fills, turn, steps=30)
    e = make_engine(params, board_shape=(6, 6), extra=0, actions=36, game="gomoku")
    o = Oracle("gomoku", (6, 6), 0, 36, 2, 32, variant, ucb_c=2.0, seed=3, device_memory=0.1, threads=4)
    for stones in (35, 34, 30):
        board, turn = random_gomoku_root(rng, 6, 6, stones)
        compare_with_oracle(e, o, board, None, turn, 20)
    board = np.zeros((6, 6), np.int8)
    board[2, 0:5] = 1
    board[3, 0:4] = -1
    compare_with_oracle(e, o, board, None, -1, 20)


def test_run_batch_equals_single_runs():
    """Several engines searched concurrently in one device pass end in exactly the state separate runs leave."""
    from mcts_numba_cuda_amd import run_batch
    rng = np.random.default_rng(5)
    params = dict(n_trees=4, n_playouts=128, variant="acp_prodigal", device_memory=0.1, ucb_c=2.0, seed=11)
    roots = [random_c4_root(rng, p) for p in (4, 9, 15, 22, 12)]
    batch = [make_engine(params) for _ in roots]
    single = [make_engine(params) for _ in roots]
    for rounds in range(2):  # second round: random streams carried over on both sides
        run_batch(batch, [r[0] for r in roots], [r[1] for r in roots], [r[2] for r in roots], forced_search_steps_limit=400)
        for e, r in zip(single, roots):
            e.run(r[0], r[1], r[2], forced_search_steps_limit=400)
        for eb, es in zip(batch, single):
            assert eb.actions_info == es.actions_info
            assert eb.performance_info["trees"] == es.performance_info["trees"]
            for ti in range(4):
                for name in ("trees", "ns", "ns_wins", "depths"):
                    np.testing.assert_array_equal(eb.read_array(name, ti), es.read_array(name, ti))
            np.testing.assert_array_equal(eb.read_array("rng_playout"), es.read_array("rng_playout"))


def test_run_batch_larger_than_the_device_takes_trees_from_the_queue():
    """A batch whose workgroups cannot all be resident at once (80 searches x 4 trees x 7 columns = 2240 workgroups of
    256 threads): the resident sets of workgroups start on one tree each and take the others from a queue as they
    finish; every search still ends exactly where a separate run ends."""
    from mcts_numba_cuda_amd import run_batch
    rng = np.random.default_rng(17)
    params = dict(n_trees=4, n_playouts=256, variant="acp_thrifty", device_memory=0.02, ucb_c=2.0, seed=3)
    roots = [random_c4_root(rng, int(rng.integers(0, 24))) for _ in range(80)]
    batch = [make_engine(params) for _ in roots]
    run_batch(batch, [r[0] for r in roots], [r[1] for r in roots], [r[2] for r in roots], forced_search_steps_limit=120)
    single = make_engine(params)
    for k in (0, 7, 31, 43, 44, 45, 62, 79):
        single.reseed()
        single.run(*roots[k], forced_search_steps_limit=120)
        assert batch[k].actions_info == single.actions_info
        for ti in range(4):
            for name in ("trees", "ns", "ns_wins"):
                np.testing.assert_array_equal(batch[k].read_array(name, ti), single.read_array(name, ti))


def test_time_limited_run_and_chunking():
    """A time budget is honoured within a few percent and splitting a search over several kernel launches changes
    nothing: the same number of steps in one launch gives the identical tree."""
    params = dict(n_trees=4, n_playouts=64, variant="acp_thrifty", device_memory=0.25, ucb_c=2.0, seed=2)
    from mcts_numba_cuda_amd import MCTSNC
    e = MCTSNC((6, 7), 7, 7, search_time_limit=0.25, search_steps_limit=np.inf, n_trees=4, n_playouts=64, variant="acp_thrifty",
               device_memory=0.25, ucb_c=2.0, seed=2, verbose_info=False)
    e.init_device_side_arrays()
    board, fills, turn = random_c4_root(np.random.default_rng(3), 7)
    e.run(board, fills, turn)
    assert 0.25 <= e.time_loop < 0.30
    steps = e.steps
    assert steps > 1000
    ref = make_engine(params)
    ref.run(board, fills, turn, forced_search_steps_limit=steps)
    assert e.actions_info == ref.actions_info
    for ti in range(4):
        np.testing.assert_array_equal(e.read_array("ns", ti), ref.read_array("ns", ti))
        np.testing.assert_array_equal(e.read_array("trees", ti), ref.read_array("trees", ti))


def test_tree_full_and_terminal_paths_match_oracle():
    """A tiny node pool forces the memory-exhausted path; late-game roots force terminal selections."""
    from oracle.oracle import Oracle
    rng = np.random.default_rng(9)
    for variant in ["ocp_thrifty", "ocp_prodigal", "acp_thrifty", "acp_prodigal"]:
        from mcts_numba_cuda_amd import MCTSNC
        e = MCTSNC((6, 7), 7, 7, search_time_limit=np.inf, search_steps_limit=np.inf, n_trees=2, n_playouts=64, variant=variant,
                   device_memory=2.0, ucb_c=2.0, seed=4, verbose_info=False)
        e.device_memory = float(2 * 95 * 50 + 2 * 8300)  # room for about 50 nodes per tree
        e.init_device_side_arrays()
        assert 10 < e.max_tree_size < 120
        o = Oracle("c4", (6, 7), 7, 7, 2, 64, variant, ucb_c=2.0, seed=4, max_tree_size_override=e.max_tree_size, threads=4)
        for plies in (5, 30):
            board, fills, turn = random_c4_root(rng, plies)
            compare_with_oracle(e, o, board, fills, turn, steps=200)
        assert max(e.read_array("depths", t).shape[0] for t in range(2)) <= e.max_tree_size


def test_gomoku_run_batch_in_groups():
    """Three Gomoku all-child-playouts searches in one call.  One such search already fills the device (8 trees x 64
    workgroups of 74 KB of LDS, two per CU), so the host runs them in consecutive groups; results equal separate runs."""
    from mcts_numba_cuda_amd import MCTSNC, run_batch
    rng = np.random.default_rng(23)

    def mk():
        e = MCTSNC((15, 15), 0, 225, search_time_limit=np.inf, n_trees=8, n_playouts=128, variant="acp_prodigal", device_memory=0.5,
                   seed=4, verbose_info=False, game="gomoku")
        e.init_device_side_arrays()
        return e
    from helpers import random_gomoku_root
    roots = [random_gomoku_root(rng, 15, 15, int(rng.integers(0, 12))) for _ in range(3)]
    batch = [mk() for _ in roots]
    run_batch(batch, [r[0] for r in roots], None, [r[1] for r in roots], forced_search_steps_limit=4)
    single = mk()
    for k in range(3):
        single.reseed()
        single.run(roots[k][0], None, roots[k][1], forced_search_steps_limit=4)
        assert batch[k].actions_info == single.actions_info
        for name in ("trees", "ns", "ns_wins"):
            np.testing.assert_array_equal(batch[k].read_array(name, 7), single.read_array(name, 7))


@pytest.mark.parametrize("game,variant", [("c4", "acp_prodigal"), ("c4", "acp_thrifty"), ("gomoku", "acp_prodigal")])
def test_device_scope_fences_give_the_same_trees(game, variant):
    """The all-child kernels skip L2 write-backs and invalidations once a tree's workgroups are known to share an
    XCC.  Option agent_fences keeps them on the general path (full device-scope release and acquire every step), which
    a device that spreads a tree over XCCs would take; results must not depend on it."""
    rng = np.random.default_rng(31)
    if game == "c4":
        from oracle.oracle import Oracle
        params = dict(n_trees=3, n_playouts=64, variant=variant, device_memory=0.25, ucb_c=2.0, seed=5)
        e = make_engine(params, options=dict(agent_fences=1))
        o = Oracle("c4", (6, 7), 7, 7, 3, 64, variant, ucb_c=2.0, seed=5, device_memory=0.25, threads=8)
        board, fills, turn = random_c4_root(rng, 9)
        compare_with_oracle(e, o, board, fills, turn, 300)
    else:
        from oracle.oracle import Oracle
        from helpers import random_gomoku_root
        params = dict(n_trees=2, n_playouts=64, variant=variant, device_memory=0.5, ucb_c=2.0, seed=5)
        e = make_engine(params, board_shape=(9, 9), extra=0, actions=81, game="gomoku", options=dict(agent_fences=1))
        o = Oracle("gomoku", (9, 9), 0, 81, 2, 64, variant, ucb_c=2.0, seed=5, device_memory=0.5, threads=8)
        board, turn = random_gomoku_root(rng, 9, 9, 6)
        compare_with_oracle(e, o, board, None, turn, 12)


def test_device_scope_fences_replay_a_recorded_game(archives):
    """The general path again (option agent_fences), over thousands of steps per search instead of hundreds: the first
    game of the reference's experiment with acp_prodigal 4 x 256 (17 searches of 5000 to 5900 steps with carried random
    streams) and of the one with acp_thrifty 8 x 256 (10 searches) must give the recorded root tables and tree statistics."""
    for a in ("mctsnc_5_inf_4_256_acp_prodigal", "mctsnc_1_inf_8_256_acp_thrifty"):
        key = replay.find_archive(archives, "mcts_5_inf_vanilla", a)
        n = replay.replay_archive(archives[key], lambda params: make_engine(params, options=dict(agent_fences=1)), engine_run_search, max_games=1)
        assert n >= 3, key


def test_time_limited_batch_over_several_launches_through_the_queue():
    """A time budget splits a batch into several kernel launches, each of which hands the trees beyond the resident
    workgroup sets out through the queue again: every search must end where a single search of as many steps ends."""
    from mcts_numba_cuda_amd import MCTSNC, run_batch
    rng = np.random.default_rng(41)

    def mk(limit):
        e = MCTSNC((6, 7), 7, 7, search_time_limit=limit, search_steps_limit=np.inf, n_trees=4, n_playouts=256,
                   variant="acp_prodigal", device_memory=0.05, ucb_c=2.0, seed=9, verbose_info=False)
        e.init_device_side_arrays()
        return e
    roots = [random_c4_root(rng, int(rng.integers(4, 20))) for _ in range(72)]
    batch = [mk(0.05) for _ in roots]
    run_batch(batch, [r[0] for r in roots], [r[1] for r in roots], [r[2] for r in roots])
    steps = batch[0].steps
    assert steps > 64 and all(e.steps == steps for e in batch)   # more than the first chunk: at least two launches
    single = mk(np.inf)
    for k in (0, 43, 44, 71):
        single.reseed()
        single.run(*roots[k], forced_search_steps_limit=steps)
        assert batch[k].actions_info == single.actions_info
        for ti in range(4):
            for name in ("trees", "ns", "ns_wins"):
                np.testing.assert_array_equal(batch[k].read_array(name, ti), single.read_array(name, ti))
