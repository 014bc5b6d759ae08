"""GPU parity of the Gomoku engine against the CPU oracle, array for array.  The oracle is pinned end to end on Gomoku by
the reference's one recorded Gomoku search (its README printout, tests/test_readme_examples.py, which the engine also
reproduces directly), on Connect 4 by the reference's tree dumps and recorded games, and for the Gomoku rules by brute
force (the reference's Gomoku archives are missing from its checkout)."""
import numpy as np
import pytest

from helpers import compare_with_oracle, make_engine, random_gomoku_root

pytestmark = pytest.mark.gpu


def engines(variant, T, P, m, n, seed=3, device_memory=0.5, **okw):
    from oracle.oracle import Oracle
    params = dict(n_trees=T, n_playouts=P, variant=variant, device_memory=device_memory, ucb_c=2.0, seed=seed)
    e = make_engine(params, board_shape=(m, n), extra=0, actions=m * n, game="gomoku")
    o = Oracle("gomoku", (m, n), 0, m * n, T, P, variant, ucb_c=2.0, seed=seed, device_memory=device_memory, threads=8, **okw)
    return e, o


@pytest.mark.parametrize("variant,T,P,steps", [("ocp_thrifty", 4, 128, 60), ("ocp_prodigal", 2, 64, 80),
                                               ("acp_thrifty", 2, 64, 6), ("acp_prodigal", 1, 128, 5),
                                               ("acp_prodigal", 3, 64, 4), ("acp_thrifty", 5, 64, 3)])
def test_gomoku_15x15_full_state(variant, T, P, steps):
    """Two consecutive searches on 15x15 (random streams carried over): every per-node array, the step scratch,
    the reduced root table and the generator states must equal the oracle's."""
    rng = np.random.default_rng(11)
    e, o = engines(variant, T, P, 15, 15)
    for stones in (0, 12):
        board, turn = random_gomoku_root(rng, 15, 15, stones)
        compare_with_oracle(e, o, board, None, turn, steps)


@pytest.mark.parametrize("variant", ["ocp_thrifty", "ocp_prodigal", "acp_thrifty", "acp_prodigal"])
def test_gomoku_small_boards_deep_trees(variant):
    """Small boards give deep trees, draws, terminal selections and, on 5x5, frequent exactly-five wins."""
    rng = np.random.default_rng(12)
    for (m, n), steps in (((6, 6), 250), ((5, 7), 150), ((8, 5), 100)):
        e, o = engines(variant, 2, 64, m, n)
        board, turn = random_gomoku_root(rng, m, n, 4)
        compare_with_oracle(e, o, board, None, turn, steps if variant.startswith("ocp") else steps // 3)


@pytest.mark.parametrize("variant,steps", [("acp_prodigal", 6), ("ocp_thrifty", 150)])
def test_gomoku_children_that_complete_lines(variant, steps):
    """A root whose children decide games at creation: a cell that completes exactly five (open four in a row; a gapped
    four; a diagonal that ends in the board's corner region), a cell that would make six (no win), and a four of the
    other side that the grandchildren complete.  Outcomes and terminal flags of every node against the oracle."""
    board = np.zeros((15, 15), np.int8)
    board[7, 3:7] = 1                                   # open four: (7,2) and (7,7) win for +1
    board[9, [2, 3, 5, 6, 7]] = 1                       # (9,4) makes six: not a win
    board[3, [8, 9, 11, 12]] = 1                        # gapped four: (3,10) wins
    for k in range(4):
        board[10 + k, k] = 1                            # diagonal (10,0)..(13,3): (14,4) wins, the other end is off the board
        board[1 + k, 12] = -1                           # four of -1 in a column: its replies at (0,12) and (5,12) win
    board[[0, 0, 5, 12, 14], [0, 5, 2, 9, 14]] = -1     # a few more stones of -1
    e, o = engines(variant, 2, 64, 15, 15, seed=9)
    compare_with_oracle(e, o, board, None, 1, steps)


@pytest.mark.parametrize("levels", [0, 2])
def test_gomoku_one_child_backup_of_paths_too_deep_to_prepare(levels):
    """One-child variants prepare the backup's arg-max during the playouts for paths of up to 48 levels; deeper ones are
    backed up after the playouts from memory.  Option prep_levels lowers the limit so that ordinary searches take that
    path at every step (0) or at the steps that select below the second level (2)."""
    rng = np.random.default_rng(21)
    for variant, (m, n), steps in (("ocp_thrifty", (15, 15), 80), ("ocp_prodigal", (6, 6), 250)):
        e, o = engines(variant, 2, 64, m, n)
        e.set_option("prep_levels", levels)
        board, turn = random_gomoku_root(rng, m, n, 5)
        compare_with_oracle(e, o, board, None, turn, steps)


@pytest.mark.parametrize("P", [1, 8, 32, 256])
def test_gomoku_one_child_other_playout_counts(P):
    """A one-child workgroup has 256 threads whatever the playout count: with fewer playouts the other wavefronts help
    (LDS columns, children, the backup's arg-max), with 256 every wavefront plays and none is left to help."""
    e, o = engines("ocp_thrifty", 2, P, 9, 9, seed=4)
    board, turn = random_gomoku_root(np.random.default_rng(P), 9, 9, 6)
    compare_with_oracle(e, o, board, None, turn, 60 if P < 256 else 25)


def test_gomoku_tree_full_path():
    from mcts_numba_cuda_amd import MCTSNC
    from oracle.oracle import Oracle
    for variant in ("ocp_prodigal", "acp_thrifty"):
        e = MCTSNC((6, 6), 0, 36, search_time_limit=np.inf, n_trees=2, n_playouts=64, variant=variant, seed=5, verbose_info=False, game="gomoku")
        e.device_memory = float(2 * 194 * 80 + 2 * 8500)
        e.init_device_side_arrays()
        assert 40 < e.max_tree_size < 120
        o = Oracle("gomoku", (6, 6), 0, 36, 2, 64, variant, seed=5, max_tree_size_override=e.max_tree_size, threads=4)
        board, turn = random_gomoku_root(np.random.default_rng(1), 6, 6, 3)
        compare_with_oracle(e, o, board, None, turn, 40)


def test_gomoku_large_playout_count_runs_in_rounds():
    """n_playouts = 512 exceeds the 256 threads of a workgroup; the playouts then run in two rounds."""
    e, o = engines("ocp_thrifty", 1, 512, 15, 15)
    board, turn = random_gomoku_root(np.random.default_rng(2), 15, 15, 8)
    compare_with_oracle(e, o, board, None, turn, 12)


@pytest.mark.parametrize("variant", ["ocp_prodigal", "acp_thrifty"])
def test_gomoku_sixteen_wide_boards(variant):
    """16 is the widest line the engine holds (one 16-bit half per side and line): fives and longer runs that touch
    the last cell of a row, column or diagonal must be judged as on any other board."""
    rng = np.random.default_rng(16)
    for (m, n), steps in (((16, 16), 30), ((5, 16), 120), ((16, 5), 120), ((16, 6), 60)):
        e, o = engines(variant, 2, 64, m, n)
        board, turn = random_gomoku_root(rng, m, n, 6)
        compare_with_oracle(e, o, board, None, turn, steps if variant.startswith("ocp") else max(3, steps // 10))


@pytest.mark.parametrize("variant,steps", [("ocp_thrifty", 40), ("ocp_prodigal", 40), ("acp_thrifty", 3), ("acp_prodigal", 3)])
def test_gomoku_boards_beyond_sixteen(variant, steps):
    """Boards with a side beyond 16 are held in the engine's second format (12 words per colour, 16-bit list entries,
    one line word per colour): 19 x 19, a rectangle, the 384 cells that still fit the 128-byte record, and boards one line of
    which is 24 long while the other side is short (deep trees, wins, draws).  Two consecutive searches each, every
    array against the oracle; more than 256 children per node exercise the arg-max tie rule on nine bits."""
    rng = np.random.default_rng(19)
    for (m, n), scale in (((19, 19), 1.0), ((17, 20), 1.0), ((24, 16), 0.5), ((5, 24), 3.0), ((20, 5), 3.0)):
        e, o = engines(variant, 2, 64, m, n, seed=7)
        for stones in (0, 12):
            board, turn = random_gomoku_root(rng, m, n, stones)
            compare_with_oracle(e, o, board, None, turn, max(2, int(steps * scale)))


@pytest.mark.parametrize("variant,steps", [("ocp_thrifty", 30), ("ocp_prodigal", 30), ("acp_thrifty", 2), ("acp_prodigal", 2)])
def test_gomoku_boards_up_to_the_references_caps(variant, steps):
    """Boards of more than 384 cells need 16 words per colour and a 256-byte node record: 22 x 22, the two extreme shapes
    of the reference's caps (512 actions, sides of 32: src/mctsnc.py:191-193), 20 x 25, and 32 x 5 (a line of 32 cells in a
    32-bit line word; the format is chosen by the cell count, so this one runs in the 12-word format)."""
    rng = np.random.default_rng(32)
    for (m, n), scale in (((22, 22), 1.0), ((32, 16), 1.0), ((16, 32), 1.0), ((20, 25), 0.5), ((32, 5), 3.0), ((5, 32), 3.0)):
        e, o = engines(variant, 2, 64, m, n, seed=11)
        for stones in (0, 14):
            board, turn = random_gomoku_root(rng, m, n, stones)
            compare_with_oracle(e, o, board, None, turn, max(2, int(steps * scale)))


def test_gomoku_fives_at_the_far_end_of_32_cell_lines():
    """32 x 16: runs of five that end on the last cell of a 32-cell column (bit 31 of a line word), a six there, and a row
    of five on the last row."""
    board = np.zeros((32, 16), np.int8)
    board[27:31, 3] = 1                                 # column 3, rows 27..30: (31,3) and (26,3) win
    board[26:31, 9] = 1; board[25, 9] = -1              # five already there is not checked; (31,9) would make six: no win
    board[31, 10:14] = 1                                # last row: (31,9)? occupied later; (31,14) wins, (31,9) makes a row five too
    for k in range(4):
        board[27 + k, 12 - k] = -1                      # anti-diagonal of -1 towards the last row
    board[[0, 2, 9, 14, 20], [0, 7, 2, 9, 10]] = -1
    for variant, steps in (("acp_prodigal", 3), ("ocp_thrifty", 100)):
        e, o = engines(variant, 2, 64, 32, 16, seed=9)
        compare_with_oracle(e, o, board, None, 1, steps)


def test_gomoku_wide_board_children_that_complete_lines():
    """19 x 19: cells that complete exactly five in the part of the board the 16-wide format does not reach (columns and
    rows 16 to 18, the diagonals that end there), a cell that would make six, and a row of five that ends on the last
    column."""
    board = np.zeros((19, 19), np.int8)
    board[17, 14:18] = 1                                # four in row 17, columns 14..17: (17,13) and (17,18) win
    board[2, [12, 13, 15, 16, 17]] = 1                  # (2,14) makes six: not a win
    board[14:18, 18] = 1                                # column 18, rows 14..17: (13,18) and (18,18) win
    for k in range(4):
        board[14 + k, 3 - k] = 1                        # anti-diagonal (14,3)..(17,0): (13,4) wins, the other end is off the board
        board[5 + k, 14 + k] = -1                       # diagonal of -1 (5,14)..(8,17): its replies at (4,13) and (9,18) win
    board[[0, 0, 9, 12, 18], [0, 7, 2, 9, 10]] = -1
    for variant, steps in (("acp_prodigal", 4), ("ocp_thrifty", 120)):
        e, o = engines(variant, 2, 64, 19, 19, seed=9)
        compare_with_oracle(e, o, board, None, 1, steps)


def test_gomoku_wide_board_other_playout_counts_and_batches():
    """19 x 19 with 256 playouts (the workgroup holds 64 at a time: four rounds) and with 16; three searches in one
    pass against separate runs."""
    from mcts_numba_cuda_amd import MCTSNC, run_batch
    rng = np.random.default_rng(23)
    for variant, P, steps in (("ocp_prodigal", 256, 12), ("acp_thrifty", 256, 2), ("ocp_thrifty", 16, 40)):
        e, o = engines(variant, 2, P, 19, 19, seed=2)
        board, turn = random_gomoku_root(rng, 19, 19, 20)
        compare_with_oracle(e, o, board, None, turn, steps)

    def mk():
        e = MCTSNC((19, 19), 0, 361, search_time_limit=np.inf, n_trees=2, n_playouts=64, variant="acp_prodigal", device_memory=0.5,
                   seed=6, verbose_info=False, game="gomoku")
        e.init_device_side_arrays()
        return e
    roots = [random_gomoku_root(rng, 19, 19, stones) for stones in (30, 2, 11)]
    batch, single = [mk() for _ in roots], [mk() for _ in roots]
    run_batch(batch, [r[0] for r in roots], None, [r[1] for r in roots], forced_search_steps_limit=3)
    for e, r in zip(single, roots):
        e.run(r[0], None, r[1], forced_search_steps_limit=3)
    for eb, es in zip(batch, single):
        assert eb.actions_info == es.actions_info
        for name in ("trees", "ns", "ns_wins", "boards"):
            np.testing.assert_array_equal(eb.read_array(name, 1), es.read_array(name, 1))


@pytest.mark.parametrize("variant,steps", [("ocp_prodigal", 20), ("acp_thrifty", 3)])
def test_gomoku_largest_board_with_256_playouts(variant, steps):
    """On 16x16 the lists and line words of 256 playouts do not fit the LDS of a CU: the workgroup then holds 128 at a
    time and plays 256 in two rounds."""
    e, o = engines(variant, 2, 256, 16, 16, seed=8)
    board, turn = random_gomoku_root(np.random.default_rng(3), 16, 16, 30)
    compare_with_oracle(e, o, board, None, turn, steps)


def test_gomoku_all_child_playouts_in_rounds():
    """n_playouts = 512 with all-child-playouts: every child's playouts run in two rounds of 256, one tree spread over
    all XCDs."""
    e, o = engines("acp_thrifty", 1, 512, 9, 9)
    board, turn = random_gomoku_root(np.random.default_rng(5), 9, 9, 5)
    compare_with_oracle(e, o, board, None, turn, 3)


@pytest.mark.parametrize("variant,T,steps", [("acp_thrifty", 20, 3), ("acp_prodigal", 40, 3), ("acp_prodigal", 512, 2),
                                             ("ocp_thrifty", 512, 12)])
def test_gomoku_many_trees(variant, T, steps):
    """More trees than the device holds 32 workgroups each for: fewer workgroups per tree, down to one, and past that
    consecutive launches over groups of trees (n_trees = 512 is the reference's MAX_N_TREES, src/mctsnc.py:195)."""
    rng = np.random.default_rng(21)
    e, o = engines(variant, T, 32, 15, 15, seed=5, device_memory=2.0)
    for stones in (8, 1):
        board, turn = random_gomoku_root(rng, 15, 15, stones)
        compare_with_oracle(e, o, board, None, turn, steps)


def test_gomoku_engines_of_different_shapes_alive_together():
    """The dynamic-LDS limit is a setting of the kernel function, not of an engine: an engine created earlier, whose
    playouts need more LDS than the latest one's, must still launch.  Three engines (16 x 16 with 128 slots: 81 KB;
    6 x 6: 3 KB; 19 x 19 in the other board format: 104 KB) are created first and then used in turn, twice."""
    rng = np.random.default_rng(31)
    made = []
    for variant, (m, n), P, steps in (("acp_thrifty", (16, 16), 256, 2), ("ocp_prodigal", (6, 6), 64, 60), ("acp_prodigal", (19, 19), 64, 2),
                                      ("ocp_thrifty", (15, 15), 128, 30)):
        e, o = engines(variant, 2, P, m, n, seed=13)
        made.append((e, o, random_gomoku_root(rng, m, n, 6), steps))
    for _ in range(2):
        for e, o, (board, turn), steps in made:
            compare_with_oracle(e, o, board, None, turn, steps)


def test_gomoku_one_child_batch_equals_single_runs():
    """Five one-child searches of positions with different numbers of stones in one pass (the library orders the trees
    of a batch by stones on the board) against separate runs, twice, so that the generators carry over on both sides."""
    from mcts_numba_cuda_amd import MCTSNC, run_batch
    rng = np.random.default_rng(29)

    def mk():
        e = MCTSNC((15, 15), 0, 225, search_time_limit=np.inf, n_trees=3, n_playouts=64, variant="ocp_prodigal", device_memory=0.5,
                   seed=6, verbose_info=False, game="gomoku")
        e.init_device_side_arrays()
        return e
    roots = [random_gomoku_root(rng, 15, 15, stones) for stones in (14, 2, 9, 0, 21)]
    batch, single = [mk() for _ in roots], [mk() for _ in roots]
    for _ in range(2):
        run_batch(batch, [r[0] for r in roots], None, [r[1] for r in roots], forced_search_steps_limit=40)
        for e, r in zip(single, roots):
            e.run(r[0], None, r[1], forced_search_steps_limit=40)
        for eb, es in zip(batch, single):
            assert eb.actions_info == es.actions_info
            for name in ("trees", "ns", "ns_wins"):
                np.testing.assert_array_equal(eb.read_array(name, 2), es.read_array(name, 2))
