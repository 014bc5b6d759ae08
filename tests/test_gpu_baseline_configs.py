"""The benchmark configurations at their full sizes, engine against oracle: every node of every tree, the step scratch,
the reduced root tables and the random streams must agree after the whole search (Connect 4 1x32 ocp_thrifty, 1000
steps; Connect 4 8x256 acp_thrifty, 20000 steps, 16 GiB pools; Gomoku 15x15 4x128 ocp_thrifty, 2000 steps, 16 GiB
pools, on a root of its own and on the benchmark's 32 seeded roots: three of them against the oracle, all of them in one
batched pass against their sequential searches; Connect 4 4x256 acp_prodigal, 5000 steps, on the benchmark's own 64
seeded roots: four of them against the oracle, all of them in one batched pass against their sequential searches -- the
same configuration is also covered by the recorded A100 games).  The fifth configuration (PUCT on Gomoku) is in test_gpu_puct_gomoku.py."""
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


GOMOKU_PARAMS = dict(n_trees=4, n_playouts=128, variant="ocp_thrifty", device_memory=16.0, ucb_c=2.0, seed=0)


def gomoku_bench_roots():
    import bench
    return bench.make_gomoku_roots()


def test_gomoku_benchmark_roots_are_what_the_configuration_says():
    roots = gomoku_bench_roots()
    stones = [int(np.count_nonzero(b)) for b, _ in roots]
    assert len(roots) == 32 and 0 <= min(stones) <= 2 and 18 <= max(stones) <= 20
    for board, turn in roots:
        plus, minus = int((board == 1).sum()), int((board == -1).sum())
        assert plus - minus in (0, 1) and turn == (1 if plus == minus else -1)


@pytest.mark.parametrize("stones", [0, 10, 20])
def test_gomoku_ocp_thrifty_4x128_2000_steps_on_a_benchmark_root(stones):
    """Three of the 32 roots bench.py times (the one with the fewest stones, one in the middle, the one with the most),
    the full 2000 steps."""
    roots = gomoku_bench_roots()
    k = min(range(len(roots)), key=lambda i: (abs(int(np.count_nonzero(roots[i][0])) - stones), i))
    board, turn = roots[k]
    e = make_engine(GOMOKU_PARAMS, board_shape=(15, 15), extra=0, actions=225, game="gomoku")
    o = Oracle("gomoku", (15, 15), 0, 225, 4, 128, "ocp_thrifty", ucb_c=2.0, seed=0, device_memory=16.0, threads=16)
    compare_with_oracle(e, o, board, None, turn, steps=2000)
    assert e.performance_info["playouts"] == 2000 * 4 * 128


def test_gomoku_ocp_thrifty_4x128_all_benchmark_roots_batched_equal_sequential():
    """What bench.py times twice: the roots one MCTSNC.run() after the other (streams restarted per root), and all 32 in one
    run_batch pass on 32 engines: root tables, best actions, tree statistics and the visit counts of every tree."""
    from helpers import engine_result
    from mcts_numba_cuda_amd import run_batch
    roots = gomoku_bench_roots()
    mk = lambda: make_engine(GOMOKU_PARAMS, board_shape=(15, 15), extra=0, actions=225, game="gomoku")
    one = mk()
    one.search_steps_limit = 2000.0
    sequential = []
    for board, turn in roots:
        one.reseed()
        one.run(board, None, turn)
        sequential.append((engine_result(one), [one.read_array("ns", t).copy() for t in range(4)]))
    one._release()
    engines = [mk() for _ in roots]
    for e in engines:
        e.search_steps_limit = 2000.0
    run_batch(engines, [r[0] for r in roots], None, [r[1] for r in roots])
    for k, e in enumerate(engines):
        assert e.steps == 2000 and e.performance_info["playouts"] == 2000 * 4 * 128
        assert engine_result(e) == sequential[k][0], f"root {k}"
        for t in range(4):
            np.testing.assert_array_equal(e.read_array("ns", t), sequential[k][1][t], err_msg=f"root {k}, tree {t}")
        e._release()


def bench_roots():
    import bench
    assert (bench.T, bench.P, bench.STEPS, bench.DEVICE_MEMORY) == (4, 256, 5000, 2.0)
    return bench.make_roots(bench.N_ROOTS)


@pytest.mark.parametrize("k", [0, 21, 42, 63])
def test_c4_acp_prodigal_4x256_5000_steps_on_a_benchmark_root(k):
    params = dict(n_trees=4, n_playouts=256, variant="acp_prodigal", device_memory=2.0, ucb_c=2.0, seed=0)
    board, fills, turn = bench_roots()[k]
    e = make_engine(params)
    o = Oracle("c4", (6, 7), 7, 7, 4, 256, "acp_prodigal", ucb_c=2.0, seed=0, device_memory=2.0, threads=16)
    compare_with_oracle(e, o, board, fills, turn, steps=5000)
    assert e.steps == 5000 and e.performance_info["playouts"] > 4 * 256 * 5000


def test_c4_acp_prodigal_4x256_all_benchmark_roots_batched_equal_sequential():
    """What bench.py times twice: the 64 roots one MCTSNC.run() after the other (streams restarted per root), and all
    64 in one run_batch pass on 64 engines."""
    from helpers import engine_result
    from mcts_numba_cuda_amd import run_batch
    params = dict(n_trees=4, n_playouts=256, variant="acp_prodigal", device_memory=2.0, ucb_c=2.0, seed=0)
    roots = bench_roots()
    one = make_engine(params)
    one.search_steps_limit = 5000.0
    sequential = []
    for board, fills, turn in roots:
        one.reseed()
        one.run(board, fills, turn)
        sequential.append((engine_result(one), [one.read_array("ns", t).copy() for t in range(4)]))
    one._release()
    engines = [make_engine(params) for _ in roots]
    for e in engines:
        e.search_steps_limit = 5000.0
    run_batch(engines, [r[0] for r in roots], [r[1] for r in roots], [r[2] for r in roots])
    for k, e in enumerate(engines):
        assert e.steps == 5000
        assert engine_result(e) == sequential[k][0], f"root {k}"
        for t in range(4):
            np.testing.assert_array_equal(e.read_array("ns", t), sequential[k][1][t], err_msg=f"root {k}, tree {t}")
        e._release()
