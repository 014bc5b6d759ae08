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


def test_a_failed_initialisation_keeps_no_device_memory():
    """An engine whose node pool cannot be allocated (512 trees x 2^24 nodes x 128 bytes is over a terabyte) must give
    back what it had allocated before the failure (stream, events, 0.9 GB of generator states), both on the failing
    call and on destroy; the free device memory afterwards is what it was before."""
    import ctypes
    from mcts_numba_cuda_amd import _lib
    L = _lib.lib()
    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipMemGetInfo.argtypes = [ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]

    def free_bytes():
        free, total = ctypes.c_size_t(), ctypes.c_size_t()
        assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
        return free.value

    warm = _engine("c4")     # the runtime's own first-use allocations happen here, not inside the measurement
    warm.close()
    before = free_bytes()
    cfg = _lib.Config(game=0, board_m=6, board_n=7, extra_info_memory=7, max_actions=7, n_trees=512, n_playouts=512, variant=3, ucb_c=2.0,
                      seed=0, max_tree_size=2**24, device=0)
    for _ in range(2):
        h = ctypes.c_void_p()
        assert L.mctsnc_create(ctypes.byref(cfg), ctypes.byref(h)) == 0
        assert L.mctsnc_init_device(h) == -2 and b"hipMalloc" in L.mctsnc_last_error()
        assert free_bytes() >= before - (8 << 20)          # nothing of the half-built engine is still held
        assert L.mctsnc_init_device(h) == -2                # a second attempt on the same handle fails the same way
        L.mctsnc_destroy(h)
    assert free_bytes() >= before - (8 << 20)
