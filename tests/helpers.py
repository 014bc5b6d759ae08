"""Shared helpers of the test suite."""
import numpy as np

M, N = 6, 7


def make_engine(params, board_shape=(M, N), extra=N, actions=N, options=None, **kw):
    """An initialised MCTSNC engine (HIP) for Connect 4 from a parameter dict as stored in the archive fixture;
    `options`: {name: value} for MCTSNC.set_option()."""
    from mcts_numba_cuda_amd import MCTSNC
    e = MCTSNC(board_shape, extra, actions, search_time_limit=np.inf, search_steps_limit=np.inf,
               n_trees=params["n_trees"], n_playouts=params["n_playouts"], variant=params["variant"],
               device_memory=params["device_memory"], ucb_c=params["ucb_c"], seed=params["seed"], verbose_info=False, **kw)
    e.init_device_side_arrays()
    for name, value in (options or {}).items():
        e.set_option(name, value)
    return e


def engine_result(e):
    acts = {}
    for a, entry in e.actions_info.items():
        if a == "best":
            continue
        acts[int(a)] = (entry["n"], entry["n_wins"], int(entry["win_flag"]))
    best = e.actions_info["best"]
    tr = e.performance_info["trees"]
    return dict(best=int(e.best_action), actions=acts, n_root=best["n_root"] if best else 0,
                trees=dict(mean_depth=tr["mean_depth"], max_depth=tr["max_depth"], mean_size=tr["mean_size"], max_size=tr["max_size"]))


def engine_run_search(e, board, fills, turn, steps):
    e.run(board, fills, turn, forced_search_steps_limit=steps)
    return engine_result(e)


def c4_has_four(board, token):
    m, n = board.shape
    for i in range(m):
        for j in range(n):
            for di, dj in ((0, 1), (1, 0), (1, 1), (1, -1)):
                ok = True
                for k in range(4):
                    ii, jj = i + di * k, j + dj * k
                    if not (0 <= ii < m and 0 <= jj < n and board[ii, jj] == token):
                        ok = False
                        break
                if ok:
                    return True
    return False


def random_c4_root(rng, plies, m=M, n=N):
    """A non-terminal Connect 4 position after `plies` uniformly random legal moves (rejection on decided games)."""
    while True:
        board = np.zeros((m, n), np.int8)
        fills = np.zeros(n, np.int8)
        turn = 1
        ok = True
        for _ in range(plies):
            legal = np.flatnonzero(fills < m)
            if legal.size == 0:
                ok = False
                break
            j = int(rng.choice(legal))
            board[m - 1 - fills[j], j] = turn
            fills[j] += 1
            if c4_has_four(board, turn):
                ok = False
                break
            turn = -turn
        if ok and (fills < m).any():
            return board, fills, turn


def compare_with_oracle(e, o, board, fills, turn, steps):
    """Runs the same search on engine and oracle and compares everything observable."""
    e.run(board, fills, turn, forced_search_steps_limit=steps)
    o.run(board, fills, turn, steps)
    T = o.T
    for ti in range(T):
        sz = o.tree_size(ti)
        assert e.read_array("depths", ti).shape[0] == sz, f"tree {ti}: size {e.read_array('depths', ti).shape[0]} vs {sz}"
        leaves = o.tree(ti, "leaves").astype(bool)
        ot = o.tree(ti, "trees").copy()
        ot[leaves, 1:] = -1
        np.testing.assert_array_equal(e.read_array("trees", ti), ot, err_msg=f"trees[{ti}]")
        for mine, theirs in [("depths", "depths"), ("turns", "turns"), ("leaves", "leaves"), ("terminals", "terminals"),
                             ("ns", "ns"), ("ns_wins", "ns_wins"), ("boards", "boards"), ("extra_infos", "extras")]:
            np.testing.assert_array_equal(e.read_array(mine, ti), o.tree(ti, theirs), err_msg=f"{mine}[{ti}]")
        oc_e, oc_o = e.read_array("outcomes", ti), o.tree(ti, "outcomes")
        np.testing.assert_array_equal(oc_e[1:], oc_o[1:], err_msg=f"outcomes[{ti}]")
        p = o.tree(ti, "path")
        np.testing.assert_array_equal(e.read_array("selected_path", ti), p[:p[-1]], err_msg=f"path[{ti}]")
        assert int(e.read_array("node_selected", ti)[0]) == o.tree_selected(ti)
        np.testing.assert_array_equal(e.read_array("playout_outcomes", ti), o.tree(ti, "playout_outcomes"))
        np.testing.assert_array_equal(e.read_array("actions_expanded", ti), o.tree(ti, "actions_expanded"), err_msg=f"actions_expanded[{ti}]")
        if o.variant.startswith("acp"):
            np.testing.assert_array_equal(e.read_array("playout_outcomes_children", ti), o.tree(ti, "playout_outcomes_children"))
    best = o.best
    assert int(e.best_action) == best["action"] and bool(e.best_win_flag) == best["win_flag"]
    assert int(e.best_n) == best["n"] and int(e.best_n_wins) == best["n_wins"]
    np.testing.assert_array_equal(e._root_actions_expanded, o.result("root_actions_expanded"))
    np.testing.assert_array_equal(e._root_ns, o.result("root_ns"))
    np.testing.assert_array_equal(e._actions_ns, o.result("actions_ns"))
    np.testing.assert_array_equal(e._actions_ns_wins, o.result("actions_ns_wins"))
    np.testing.assert_array_equal(e._actions_win_flags.astype(np.uint8), o.result("actions_win_flags"))
    np.testing.assert_array_equal(e.read_array("rng_playout"), o.rng_states("playout"))


def random_gomoku_root(rng, m, n, stones):
    """`stones` stones placed alternately on distinct random cells (no rule check: the engine, like the reference,
    only tests lines through the last stone placed)."""
    board = np.zeros((m, n), np.int8)
    turn = 1
    for c in rng.permutation(m * n)[:stones]:
        board[c // n, c % n] = turn
        turn = -turn
    return board, turn
