"""Gomoku PUCT loop on the GPU through the C ABI (include/puct_gomoku.h): with one traversal per tree a search is
deterministic and must equal the sequential oracle array for array, in one launch and in three launches per step;
with concurrent traversals the trees must satisfy the structural invariants.  The reference has no such loop, so
nothing here is pinned against reference output."""
import numpy as np
import pytest

import puct_gomoku_checks as gc
from helpers import random_gomoku_root
from oracle import puct_oracle as po

pytestmark = pytest.mark.gpu

COMPARED = ("node_count", "node_expanded", "node_expand_inflight", "node_legal", "node_turn", "node_value", "node_board",
            "edge_child", "edge_n", "edge_w", "edge_prior", "edge_action", "edge_inflight")


def read_all(e):
    from mcts_numba_cuda_amd.puct_gomoku import ARRAYS
    return {name: e.read_array(name) for name in ARRAYS}


def assert_same_trees(got, want):
    """Compares everything that belongs to created nodes (rows of nodes that were never created are uninitialised on
    the device)."""
    assert np.array_equal(got["node_count"], want["node_count"])
    for t, count in enumerate(want["node_count"]):
        for name in COMPARED[1:7]:
            assert np.array_equal(got[name][t, :count], want[name][t, :count]), (name, t)
        for node in range(count):
            k = int(want["node_legal"][t, node])
            if want["node_expanded"][t, node] == -1:
                continue
            for name in COMPARED[7:]:
                assert np.array_equal(got[name][t, node, :k], want[name][t, node, :k]), (name, t, node)
    for name in ("out_selected", "out_len"):
        assert np.array_equal(got[name], want[name]), name
    for t in range(want["out_len"].shape[0]):
        for w in range(want["out_len"].shape[1]):
            k = max(int(want["out_len"][t, w]) - 1, 0)
            assert np.array_equal(got["out_path"][t, w, :k], want["out_path"][t, w, :k])
            assert np.array_equal(got["path_values"][t, w, :k], want["path_values"][t, w, :k])


@pytest.mark.parametrize("shape,stones,steps,max_nodes,depth,c_pw", [
    ((15, 15), 0, 400, 1024, 64, 1.0), ((15, 15), 14, 300, 1024, 64, 2.0), ((6, 6), 6, 500, 2048, 64, 1.0),
    ((5, 5), 17, 300, 1024, 64, 1.0), ((9, 9), 0, 300, 120, 64, 1.0), ((7, 7), 2, 300, 1024, 3, 1.0)])
def test_single_traversal_equals_oracle(shape, stones, steps, max_nodes, depth, c_pw):
    from mcts_numba_cuda_amd.puct_gomoku import PUCTGomoku
    rng = np.random.default_rng(shape[0] * 31 + stones)
    board, turn = random_gomoku_root(rng, shape[0], shape[1], stones)
    kw = dict(trees=5, traversals=1, max_nodes=max_nodes, path_depth=depth, cpuct=1.5, c_pw=c_pw, dirichlet_alpha=0.3, seed=9)
    want = po.gomoku_search(board, turn, steps, **kw)
    for fused in (True, False):
        e = PUCTGomoku(board_shape=shape, **kw)
        best = e.run(board, turn, steps, fused=fused)
        got = read_all(e)
        assert_same_trees(got, want)
        assert [e.selections[k] for k in ("invalid", "expand", "terminal", "depth_limit", "busy")] == want["tally"][:, :5].sum(axis=0).tolist()
        assert e.result.expansions_committed == int(want["tally"][:, 5].sum())
        # the reported root table is the sum over trees of the root rows
        root_n = np.zeros(shape[0] * shape[1], np.int64)
        for t in range(5):
            ne = max(int(want["node_expanded"][t, 0]), 0)
            np.add.at(root_n, want["edge_action"][t, 0, :ne].astype(int), want["edge_n"][t, 0, :ne])
        assert np.array_equal(e.root_n, root_n) and best == int(np.argmax(root_n))
        e.close()


@pytest.mark.parametrize("shape,stones,trees,traversals,steps,soft", [
    ((15, 15), 0, 16, 16, 250, False), ((15, 15), 20, 16, 16, 250, True), ((6, 6), 8, 4, 16, 300, False),
    ((9, 9), 3, 8, 5, 200, False)])
def test_concurrent_traversals_build_consistent_trees(shape, stones, trees, traversals, steps, soft):
    from mcts_numba_cuda_amd.puct_gomoku import PUCTGomoku
    rng = np.random.default_rng(shape[0] + stones)
    board, turn = random_gomoku_root(rng, shape[0], shape[1], stones)
    e = PUCTGomoku(board_shape=shape, trees=trees, traversals=traversals, max_nodes=16384, path_depth=64, cpuct=1.5,
                   c_pw=1.0, soft_winner=soft, seed=1)
    best = e.run(board, turn, steps)
    h = read_all(e)
    gc.check_trees(h, board, turn, shape[0], shape[1], 16384, 64, tree_not_full_required=True)
    gc.check_visit_flow(h, 64)
    sel = e.selections
    assert sum(sel.values()) == steps * trees * traversals and sel["invalid"] == 0 and sel["depth_limit"] == 0
    assert sum(gc.visits_below(h, t, 0) for t in range(trees)) == sel["expand"] + sel["terminal"]
    assert e.result.nodes_total == int(h["node_count"].sum()) == e.result.expansions_committed + trees
    assert board.reshape(-1)[best] == 0 and e.root_n[best] == e.root_n.max()
    # a second search on the same engine starts from a clean tree and, being racy, may differ, but stays consistent
    e.run(board, turn, 50)
    gc.check_trees(read_all(e), board, turn, shape[0], shape[1], 16384, 64)
    e.close()


def test_expanded_edges_stay_contiguous_when_tickets_leave_holes():
    """The selections of one step can hold expansion tickets with a hole between them (a traversal whose widening limit
    is smaller hands its ticket back after another has drawn the next one; frequent with the soft winner, where many
    traversals pile on one node).  The expansion takes the node's next free edge slot whatever the ticket says, so the
    first `node_expanded` slots of every node always have children.  Twenty-five searches of the configuration that
    used to leave a hole in about one search in ten."""
    from mcts_numba_cuda_amd.puct_gomoku import PUCTGomoku
    board, turn = random_gomoku_root(np.random.default_rng(35), 15, 15, 20)
    for _ in range(25):
        e = PUCTGomoku(board_shape=(15, 15), trees=16, traversals=16, max_nodes=16384, path_depth=64, cpuct=1.5, c_pw=1.0, soft_winner=True, seed=1)
        e.run(board, turn, 250)
        expanded, children, counts = e.read_array("node_expanded"), e.read_array("edge_child"), e.read_array("node_count")
        legal = e.read_array("node_legal")
        for t in range(16):
            k = expanded[t, :counts[t]]
            slots = np.arange(256)[None, :] < np.maximum(k, 0)[:, None]
            assert np.all(children[t, :counts[t]][slots] > 0), f"tree {t}: an expanded slot without a child"
            assert np.all(children[t, :counts[t]][~slots & (np.arange(256)[None, :] < legal[t, :counts[t], None]) & (k >= 0)[:, None]] == -1)
        e.close()


def test_baseline_config_at_full_size():
    """The benchmark configuration for PUCT with virtual loss on Gomoku at its size: 15x15 empty board, 16 trees x 16
    traversals = 256 leaves per step, 4000 steps, node limit 16384 per tree (which this search approaches but does not
    reach: about 13 000 nodes per tree).  Racy by design, so what is checked are the invariants: structure of every
    node of every tree, nothing in flight, conservation of visits from every edge to the child's edges."""
    from mcts_numba_cuda_amd.puct_gomoku import PUCTGomoku
    trees, traversals, steps, max_nodes = 16, 16, 4000, 16384
    board = np.zeros((15, 15), np.int8)
    e = PUCTGomoku(trees=trees, traversals=traversals, max_nodes=max_nodes, path_depth=64, cpuct=1.5, c_pw=1.0, alpha_pw=0.5,
                   recalc_attempts=16, dirichlet_alpha=0.3, seed=0)
    best = e.run(board, 1, steps)
    h = read_all(e)
    print(f"nodes per tree: {h['node_count'].tolist()}", flush=True)
    gc.check_trees(h, board, 1, 15, 15, max_nodes, 64, tree_not_full_required=True)
    gc.check_visit_flow(h, 64)
    sel = e.selections
    assert sum(sel.values()) == steps * trees * traversals and sel["invalid"] == 0 and sel["depth_limit"] == 0
    assert sum(gc.visits_below(h, t, 0) for t in range(trees)) == sel["expand"] + sel["terminal"]
    assert e.result.steps == steps and e.result.nodes_total == int(h["node_count"].sum()) == e.result.expansions_committed + trees
    assert e.result.expansions_committed == sel["expand"]        # every selected expansion was committed: no tree filled up
    assert e.result.max_nodes_in_tree == int(h["node_count"].max()) > 8000
    assert board.reshape(-1)[best] == 0 and e.root_n[best] == e.root_n.max() and int(e.root_n.sum()) == sel["expand"] + sel["terminal"]
    e.close()


@pytest.mark.parametrize("traversals", [16, 1])
def test_node_limit_stops_growth_and_the_search_goes_on(traversals):
    """With the benchmark's shape but room for 2048 nodes per tree, the trees fill up well before the last step.
    From then on the expansions of a step are committed together or not at all, the traversals evaluate the node they
    reached instead, and the search continues on trees that no longer grow."""
    from mcts_numba_cuda_amd.puct_gomoku import PUCTGomoku
    trees, steps, max_nodes = 16, 1500 if traversals > 1 else 6000, 2048
    board = np.zeros((15, 15), np.int8)
    e = PUCTGomoku(trees=trees, traversals=traversals, max_nodes=max_nodes, path_depth=64, cpuct=1.5, c_pw=1.0, recalc_attempts=16, seed=2)
    e.run(board, 1, steps)
    h = read_all(e)
    counts = h["node_count"]
    assert np.all(counts <= max_nodes) and np.all(counts > max_nodes - traversals), counts.tolist()
    gc.check_trees(h, board, 1, 15, 15, max_nodes, 64)     # structure, and nothing left in flight on any node
    sel = e.selections
    assert sum(sel.values()) == steps * trees * traversals and sel["invalid"] == 0
    assert e.result.nodes_total == int(counts.sum()) == e.result.expansions_committed + trees
    assert e.result.expansions_committed < sel["expand"]      # expansions selected after the trees were full were not committed ...
    # ... but were evaluated and backed up along their paths: the root saw more visits than there are nodes, though not
    # one per selection (a selection whose widening step asked the root itself for another child has an empty path)
    root_visits = sum(gc.visits_below(h, t, 0) for t in range(trees))
    assert e.result.expansions_committed < root_visits <= sel["expand"] + sel["terminal"] + sel["depth_limit"]
    assert int(e.root_n.sum()) == root_visits
    if traversals == 1:     # deterministic: equal to the sequential oracle, array for array
        want = po.gomoku_search(board, 1, steps, trees=trees, traversals=1, max_nodes=max_nodes, path_depth=64, cpuct=1.5, c_pw=1.0,
                                dirichlet_alpha=0.3, seed=2)
        assert_same_trees(h, want)
    e.close()


def test_finds_the_winning_move():
    """Four in a row with both ends open for the player to move: every expansion of an end cell is a terminal win worth
    +1, so the search concentrates its visits there."""
    from mcts_numba_cuda_amd.puct_gomoku import PUCTGomoku
    board = np.zeros((15, 15), np.int8)
    board[7, 4:8] = 1
    board[8, 4:7] = -1
    board[3, 3] = -1
    e = PUCTGomoku(trees=16, traversals=8, max_nodes=8192, cpuct=1.5, c_pw=4.0, seed=3)
    best = e.run(board, 1, 600)
    assert best in (7 * 15 + 3, 7 * 15 + 8)
    assert e.root_q[best] == 1.0
    e.close()


def test_configuration_and_root_errors():
    from mcts_numba_cuda_amd.puct_gomoku import EngineError, PUCTGomoku
    for bad in (dict(board_shape=(17, 17)), dict(traversals=17), dict(max_nodes=20000), dict(dirichlet_alpha=1.5),
                dict(path_depth=0), dict(trees=0)):
        with pytest.raises(EngineError):
            PUCTGomoku(**bad)
    e = PUCTGomoku(board_shape=(5, 5), trees=1, traversals=1, max_nodes=16)
    with pytest.raises(EngineError):
        e.run(np.full((5, 5), 1, np.int8), 1, 10)         # no empty cell
    with pytest.raises(EngineError):
        e.run(np.full((5, 5), 3, np.int8), 1, 10)         # not a stone
    with pytest.raises(EngineError):
        e.run(np.zeros((5, 5), np.int8), 0, 10)           # no such player
    assert e.run(np.zeros((5, 5), np.int8), 1, 0) == -1   # no steps: no visits
    e.close()
