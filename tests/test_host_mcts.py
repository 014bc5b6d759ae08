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


def test_archive_log_parser_reads_the_runner_format():
    """A log fragment in the format the reference's runner prints (src/game_runner.py, src/mctsnc.py:1255-1257,
    src/utils.py:23-30), with a numpy-2 style scalar repr as some archives have."""
    from mcts_numba_cuda_amd.archive import parse_instance, parse_log
    inst = "MCTSNC(search_time_limit=5.0, search_steps_limit=inf, n_trees=4, n_playouts=256, variant='acp_prodigal', device_memory=2.0, ucb_c=2.0, seed: 0)"
    assert parse_instance(inst) == dict(n_trees=4, n_playouts=256, variant="acp_prodigal", device_memory=2.0, ucb_c=2.0, seed=0)
    log = "\n".join([
        "GAME 1/100:", "BLACK: " + inst, "WHITE: MCTS(search_time_limit=5.0, search_steps_limit=inf, vanilla=True, ucb_c=2.0, seed: 0)",
        "MCTSNC RUN... [" + inst + "]", "[actions info:", "{",
        "  0: {'name': '0', 'n_root': 512, 'win_flag': False, 'n': 256, 'n_wins': 100, 'q': np.float64(0.39), 'ucb': 1.5},",
        "  3: {'name': '3', 'n_root': 512, 'win_flag': True, 'n': 256, 'n_wins': 256, 'q': 1.0, 'ucb': inf},",
        "  best: {'index': 3, 'name': '3', 'n_root': 512, 'win_flag': True, 'n': 256, 'n_wins': 256, 'q': 1.0, 'ucb': inf}",
        "}]", "[performance info:", "{", "  steps: 1,", "  steps_per_second: 10.0,", "  playouts: 512,", "  playouts_per_second: 5120.0,",
        "  times_[ms]: {'total': 1.0},", "  trees: {'count': 4, 'mean_depth': 0.75, 'max_depth': 1, 'mean_size': 3.0, 'max_size': 3}", "}]",
        "MCTSNC RUN DONE. [time: 0.1 s; best action: 3]", "MOVE PLAYED: 3", "GAME OUTCOME: BLACK WINS"])
    games = parse_log(log, 5)
    assert len(games) == 1 and games[0]["outcome"] == "BLACK WINS"
    search, move = games[0]["events"]
    assert search == {"type": "mctsnc", "side": "black", "steps": 1, "playouts": 512, "best": 3, "n_root": 512,
                      "actions": {"0": [256, 100, 0], "3": [256, 256, 1]},
                      "trees": {"mean_depth": 0.75, "max_depth": 1, "mean_size": 3.0, "max_size": 3}}
    assert move == {"type": "move", "action": 3}


@pytest.mark.gpu
def test_archive_replay_tool_reproduces_a_recorded_game(archives):
    """The replay tool on the fixture of the north-star archive: every MCTSNC search of the first game reproduces the
    logged root table, best action and tree statistics."""
    from mcts_numba_cuda_amd import archive
    entry = archives[find_archive(archives, "mcts_5_inf_vanilla", "mctsnc_5_inf_4_256_acp_prodigal")]
    checked, failures = archive.replay(entry, max_games=1)
    assert checked >= 10 and failures == []
