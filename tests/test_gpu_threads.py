"""Two host threads, each with an engine of its own, searching at the same time: the library keeps no shared mutable
state between engines (an error message is per thread, a stream per engine), and the all-children kernels, whose
workgroups wait for each other, still get the whole of their grid resident.  Results equal those of separate runs."""
import threading

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _engine(game):
    from mcts_numba_cuda_amd import MCTSNC
    if game == "gomoku":
        e = MCTSNC((15, 15), 0, 225, search_time_limit=np.inf, search_steps_limit=100, n_trees=8, n_playouts=128,
                   variant="acp_prodigal", device_memory=1.0, verbose_info=False, game="gomoku")
    else:
        e = MCTSNC((6, 7), 7, 7, search_time_limit=np.inf, search_steps_limit=20000, n_trees=8, n_playouts=256,
                   variant="acp_prodigal", device_memory=1.0, verbose_info=False)
    e.init_device_side_arrays()
    return e


def _root(game):
    if game == "gomoku":
        return np.zeros((15, 15), np.int8), None, 1
    return np.zeros((6, 7), np.int8), np.zeros(7, np.int8), 1


@pytest.mark.parametrize("games", [("c4", "c4"), ("c4", "gomoku"), ("gomoku", "gomoku")], ids="-".join)
def test_an_engine_per_host_thread(games):
    engines = [_engine(g) for g in games]
    alone = []
    for e, g in zip(engines, games):
        e.run(*_root(g))
        alone.append((dict(e.actions_info["best"]), e.read_array("ns", 7).copy()))
    together = [None, None]
    errors = []

    def work(i):
        try:
            engines[i].reseed()
            engines[i].run(*_root(games[i]))
            together[i] = (dict(engines[i].actions_info["best"]), engines[i].read_array("ns", 7).copy())
        except Exception as exc:  # reported by the main thread
            errors.append(exc)

    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=120)
    assert not errors, errors
    for a, b in zip(alone, together):
        assert b is not None and a[0] == b[0]
        np.testing.assert_array_equal(a[1], b[1])
