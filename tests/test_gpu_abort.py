"""The path a search takes when the workgroups of a tree wait for each other in vain (include/mctsnc_hip.h:
MCTSNC_E_DEVICE_SYNC).  No workgroup is made to hang: option spin_limit = 1 makes the first wait that is not met at
once give up, every kernel exits normally, and the host must report the failure and leave the engine in the state of a
newly initialised one."""
import numpy as np
import pytest

from helpers import make_engine, random_c4_root, random_gomoku_root

pytestmark = pytest.mark.gpu


def snapshot(e, trees):
    out = dict(info=e.actions_info, rng=e.read_array("rng_playout").copy())
    for ti in range(trees):
        for name in ("trees", "ns", "ns_wins"):
            out[name, ti] = e.read_array(name, ti).copy()
    return out


def assert_same(a, b):
    assert a["info"] == b["info"]
    for key in a:
        if key != "info":
            np.testing.assert_array_equal(a[key], b[key], err_msg=str(key))


@pytest.mark.parametrize("game,variant", [("c4", "acp_prodigal"), ("c4", "acp_thrifty"), ("gomoku", "acp_prodigal")])
def test_abandoned_search_reports_and_leaves_a_fresh_engine(game, variant):
    from mcts_numba_cuda_amd import _lib
    rng = np.random.default_rng(5)
    if game == "c4":
        params = dict(n_trees=3, n_playouts=64, variant=variant, device_memory=0.25, ucb_c=2.0, seed=5)
        mk = lambda: make_engine(params)
        board, fills, turn = random_c4_root(rng, 9)
        root, steps = (board, fills, turn), 300
    else:
        params = dict(n_trees=2, n_playouts=64, variant=variant, device_memory=0.5, ucb_c=2.0, seed=5)
        mk = lambda: make_engine(params, board_shape=(9, 9), extra=0, actions=81, game="gomoku")
        board, turn = random_gomoku_root(rng, 9, 9, 6)
        root, steps = (board, None, turn), 12
    e = mk()
    e.run(*root, forced_search_steps_limit=steps)          # the streams have moved on from their seeds
    e.set_option("spin_limit", 1)
    with pytest.raises(_lib.EngineError) as err:
        e.run(*root, forced_search_steps_limit=steps)
    assert err.value.code == -5 and "timed out" in str(err.value)    # MCTSNC_E_DEVICE_SYNC
    e.set_option("spin_limit", 0)
    fresh = mk()
    for _ in range(2):                                     # two runs: the carried streams agree as well
        e.run(*root, forced_search_steps_limit=steps)
        fresh.run(*root, forced_search_steps_limit=steps)
        assert_same(snapshot(e, params["n_trees"]), snapshot(fresh, params["n_trees"]))


def test_option_values_are_checked():
    from mcts_numba_cuda_amd import _lib
    e = make_engine(dict(n_trees=1, n_playouts=32, variant="ocp_thrifty", device_memory=0.05, ucb_c=2.0, seed=0))
    for name, value in (("solo_threads", 100), ("solo_threads", 1024), ("team_pool", 2), ("agent_fences", 3), ("spin_limit", -1)):
        with pytest.raises(_lib.EngineError):
            e.set_option(name, value)
    with pytest.raises(ValueError):
        e.set_option("no_such_option", 1)
    e.set_option("solo_threads", 128)
    e.set_option("solo_threads", 0)
