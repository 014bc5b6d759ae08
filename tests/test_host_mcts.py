"""The host-side State / C4 / Gomoku / MCTS classes against the reference's recorded CPU searches: the archive of the
north-star experiment logs, for every search of the CPU player, the step count, the visit and win counts of all root
actions and the size and depth of the search tree (A100 box, seed 0).  Replaying the first searches of the first game
with the recorded step counts must reproduce them exactly, which pins the selection rule, the expansion order, the
playout mechanics and the consumption of numpy's legacy random stream."""
import contextlib
import io

import numpy as np
import pytest

from replay import find_archive


def mcts_events(game, count):
    out, moves = [], []
    for ev in game["events"]:
        if ev["type"] == "move":
            moves.append(ev["action"])
        elif ev["type"] == "mcts":
            out.append((list(moves), ev))
            if len(out) == count:
                break
    return out


def test_cpu_mcts_reproduces_recorded_searches(archives):
    from mcts_numba_cuda_amd.c4 import C4
    from mcts_numba_cuda_amd.mcts import MCTS
    arch = archives[find_archive(archives, "mcts_5_inf_vanilla", "mctsnc_5_inf_4_256_acp_prodigal")]
    game = arch["games"][0]
    assert game["black"] == "MCTS(search_time_limit=5.0, search_steps_limit=inf, vanilla=True, ucb_c=2.0, seed: 0)"
    ai = MCTS(search_time_limit=5.0, search_steps_limit=np.inf, vanilla=True, ucb_c=2.0, seed=0)
    assert str(ai) == game["black"]
    for moves, ev in mcts_events(game, 2):
        state = C4()
        for a in moves:
            state = state.take_action(a)
        with contextlib.redirect_stdout(io.StringIO()):
            best = ai.run(state, forced_search_steps_limit=ev["steps"])
        info = ai.root_actions_info
        assert best == ev["best"] and ai.steps == ev["steps"] and state.n == ev["n_root"]
        for key, (n, n_wins, win_flag) in ev["actions"].items():
            got = info[int(key)]
            assert (got["n"], got["n_wins"], int(got["win_flag"])) == (n, n_wins, win_flag), key
        tree = ai.performance_info["tree"]
        assert tree["size"] == ev["tree"]["size"] and tree["max_depth"] == ev["tree"]["max_depth"]
        assert tree["mean_depth"] == pytest.approx(ev["tree"]["mean_depth"], rel=1e-12)


def test_state_classes_match_the_device_rules():
    """The host rules agree with the oracle's outcome routine (the device rules) on random games of both kinds."""
    from mcts_numba_cuda_amd.c4 import C4
    from mcts_numba_cuda_amd.gomoku import Gomoku
    from oracle import oracle
    rng = np.random.default_rng(4)
    L = oracle.lib()
    for cls, game in ((C4, 0), (Gomoku, 1)):
        for _ in range(30):
            state = cls()
            while True:
                legal = [a for a in range(cls.get_max_actions())
                         if (state.column_fills[a] < cls.M if cls is C4 else state.board.reshape(-1)[a] == 0)]
                a = int(rng.choice(legal))
                if cls is Gomoku:
                    assert state.take_action(cls.get_max_actions() + 3) is None      # off the board
                state = state.take_action(a)
                assert state.parent.take_action(a) is state                           # memoised child
                board = np.ascontiguousarray(state.board)
                extra = state.column_fills.ctypes.data if cls is C4 else None
                want = L.mo_game_outcome(game, cls.M, cls.N, board.ctypes.data, extra, int(state.turn), a)
                got = state.compute_outcome()
                assert (2 if got is None else got) == want
                if got is not None:
                    assert state.win_flag == (got == -state.turn)
                    break
    assert C4.class_repr() == "C4_6x7" and Gomoku.class_repr() == "Gomoku_15x15"
    assert Gomoku.action_name_to_index("B4") == 3 * 15 + 1 and Gomoku.action_index_to_name(46) == "B4"
    assert (C4.get_board_shape(), C4.get_extra_info_memory(), C4.get_max_actions()) == ((6, 7), 7, 7)
    assert (Gomoku.get_board_shape(), Gomoku.get_extra_info_memory(), Gomoku.get_max_actions()) == ((15, 15), 0, 225)


@pytest.mark.gpu
def test_host_states_drive_the_gpu_engine():
    """The call sequence of the reference's game runner (src/game_runner.py:89-135): states produce board / extra info,
    MCTSNC searches, the chosen action is applied to the state."""
    from mcts_numba_cuda_amd import MCTSNC
    from mcts_numba_cuda_amd.c4 import C4
    ai = MCTSNC(C4.get_board_shape(), C4.get_extra_info_memory(), C4.get_max_actions(), search_time_limit=np.inf,
                search_steps_limit=200, n_trees=2, n_playouts=64, variant="ocp_thrifty", device_memory=0.1,
                action_index_to_name_function=C4.action_index_to_name, verbose_info=False)
    ai.init_device_side_arrays()
    state = C4()
    with contextlib.redirect_stdout(io.StringIO()):
        for _ in range(6):
            move = ai.run(state.get_board(), state.get_extra_info(), state.get_turn())
            state = state.take_action(int(move))
            assert state is not None
            if state.compute_outcome() is not None:
                break
    assert int(np.abs(state.board).sum()) >= 6 or state.compute_outcome() is not None
