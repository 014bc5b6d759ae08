"""Gomoku PUCT loop on the GPU through the C ABI (include/puct_gomoku.h).  The loop takes the claims of a step's
traversals in a fixed order, so a search is reproducible and must equal the host oracle array for array, for any number
of traversals per tree, in one launch and in three launches per step; the trees must also satisfy the structural
invariants.  The reference has no such loop, so nothing here is pinned against reference output."""
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


def created_rows(h):
    """Boolean masks [T, N] of created nodes and [T, N, E] of the edge slots that belong to them."""
    T, N = h["node_legal"].shape
    nodes = np.arange(N)[None, :] < h["node_count"][:, None]
    inner = nodes & (h["node_expanded"] != -1)
    edges = inner[:, :, None] & (np.arange(256)[None, None, :] < np.where(inner, h["node_legal"], 0)[:, :, None])
    return nodes, edges


def assert_same_trees(got, want):
    """Compares everything that belongs to created nodes (rows of nodes that were never created are uninitialised on
    the device) and what the traversals of the last step ended with."""
    assert np.array_equal(got["node_count"], want["node_count"])
    nodes, edges = created_rows(want)
    for name in COMPARED[1:7]:
        assert np.array_equal(got[name][nodes], want[name][nodes]), name
    for name in COMPARED[7:]:
        assert np.array_equal(got[name][edges], want[name][edges]), name
    for name in ("out_selected", "out_len"):
        assert np.array_equal(got[name], want[name]), name
    on_path = np.arange(want["out_path"].shape[2])[None, None, :] < (want["out_len"] - 1)[:, :, None]
    for name in ("out_path", "path_values"):
        assert np.array_equal(got[name][on_path], want[name][on_path]), name


@pytest.mark.parametrize("shape,stones,traversals,steps,max_nodes,depth,c_pw", [
    ((15, 15), 0, 1, 400, 1024, 64, 1.0), ((15, 15), 14, 1, 300, 1024, 64, 2.0), ((6, 6), 6, 1, 500, 2048, 64, 1.0),
    ((5, 5), 17, 1, 300, 1024, 64, 1.0), ((9, 9), 0, 1, 300, 120, 64, 1.0), ((7, 7), 2, 1, 300, 1024, 3, 1.0),
    ((15, 15), 0, 16, 250, 8192, 64, 1.0), ((15, 15), 20, 16, 250, 8192, 64, 16.0), ((6, 6), 8, 16, 300, 8192, 64, 4.0),
    ((9, 9), 3, 5, 200, 4096, 64, 2.0), ((15, 15), 3, 16, 300, 2000, 64, 16.0), ((7, 7), 0, 7, 300, 8192, 2, 8.0),
    ((16, 16), 1, 13, 200, 8192, 256, 3.0)])
def test_search_equals_oracle(shape, stones, traversals, steps, max_nodes, depth, c_pw):
    """Any number of traversals per tree: every array of every created node, the last step's selections and paths and
    the tallies equal the host oracle's, in one launch (with the new nodes' priors worked out by evaluator workgroups or
    by the tree's own) and in three launches per step; includes trees that fill up, paths cut by the depth limit,
    boards that fill up (draws) and the widest board."""
    from mcts_numba_cuda_amd.puct_gomoku import PUCTGomoku
    rng = np.random.default_rng(shape[0] * 31 + stones)
    board, turn = random_gomoku_root(rng, shape[0], shape[1], stones)
    kw = dict(trees=5, traversals=traversals, max_nodes=max_nodes, path_depth=depth, cpuct=1.5, c_pw=c_pw, dirichlet_alpha=0.3, seed=9)
    want = po.gomoku_search(board, turn, steps, **kw)
    gc.check_trees(want, board, turn, shape[0], shape[1], max_nodes, depth)
    for fused, evaluators, agent_fences in ((True, 4, False), (True, 0, False), (True, 8, False), (True, 4, True), (False, 0, False)):
        e = PUCTGomoku(board_shape=shape, evaluators=evaluators, agent_fences=agent_fences, **kw)
        best = e.run(board, turn, steps, fused=fused)
        got = read_all(e)
        assert_same_trees(got, want)
        assert [e.selections[k] for k in ("invalid", "expand", "terminal", "depth_limit", "busy")] == want["tally"][:, :5].sum(axis=0).tolist()
        assert e.result.expansions_committed == int(want["tally"][:, 5].sum())
        assert e.result.nodes_read == int(want["tally"][:, 6].sum()) and e.result.edges_scored == int(want["tally"][:, 7].sum())
        # the reported root table is the sum over trees of the root rows
        root_n = np.zeros(shape[0] * shape[1], np.int64)
        for t in range(5):
            ne = max(int(want["node_expanded"][t, 0]), 0)
            np.add.at(root_n, want["edge_action"][t, 0, :ne].astype(int), want["edge_n"][t, 0, :ne])
        assert np.array_equal(e.root_n, root_n) and best == (int(np.argmax(root_n)) if root_n.any() else -1)
        e.close()


@pytest.mark.parametrize("shape,stones,trees,traversals,steps,c_pw", [
    ((15, 15), 0, 16, 16, 250, 1.0), ((15, 15), 20, 16, 16, 250, 16.0), ((6, 6), 8, 4, 16, 300, 1.0), ((9, 9), 3, 8, 5, 200, 2.0)])
def test_traversals_of_a_step_build_consistent_trees(shape, stones, trees, traversals, steps, c_pw):
    from mcts_numba_cuda_amd.puct_gomoku import PUCTGomoku
    rng = np.random.default_rng(shape[0] + stones)
    board, turn = random_gomoku_root(rng, shape[0], shape[1], stones)
    e = PUCTGomoku(board_shape=shape, trees=trees, traversals=traversals, max_nodes=16384, path_depth=64, cpuct=1.5, c_pw=c_pw, seed=1)
    best = e.run(board, turn, steps)
    h = read_all(e)
    gc.check_trees(h, board, turn, shape[0], shape[1], 16384, 64, tree_not_full_required=True)
    gc.check_visit_flow(h, 64)
    sel = e.selections
    assert sum(sel.values()) == steps * trees * traversals and sel["invalid"] == 0 and sel["depth_limit"] == 0
    if c_pw >= traversals:
        assert sel["busy"] == 0      # a node without children admits one ticket per traversal
    assert sum(gc.visits_below(h, t, 0) for t in range(trees)) == sel["expand"] + sel["terminal"]
    assert e.result.nodes_total == int(h["node_count"].sum()) == e.result.expansions_committed + trees
    assert board.reshape(-1)[best] == 0 and e.root_n[best] == e.root_n.max()
    # a second search on the same engine starts from a clean tree and gives the same trees again
    e.run(board, turn, steps)
    assert_same_trees(read_all(e), h)
    e.close()


def test_repeated_searches_give_the_same_trees():
    """Twenty searches of one configuration (many traversals meeting on few nodes, trees of some thousand nodes) must all
    equal the host oracle's: a result that depends on when a store becomes visible to another wavefront shows up as a
    search that differs.  (An earlier form of the loop, which let the traversals race for their claims, handed out an
    expansion slot twice once in some thousand searches because a barrier did not wait for the stores before it.)"""
    from mcts_numba_cuda_amd.puct_gomoku import PUCTGomoku
    board, turn = random_gomoku_root(np.random.default_rng(35), 15, 15, 20)
    kw = dict(trees=16, traversals=16, max_nodes=4096, path_depth=64, cpuct=1.5, c_pw=3.0, dirichlet_alpha=0.3, seed=1)
    want = po.gomoku_search(board, turn, 250, **kw)
    for evaluators in (4, 0):
        e = PUCTGomoku(board_shape=(15, 15), evaluators=evaluators, **kw)
        for _ in range(10):
            e.run(board, turn, 250)
            assert_same_trees(read_all(e), want)
        e.close()


def test_expanded_edges_stay_contiguous_when_tickets_leave_holes():
    """The selections of one step can hold expansion tickets with a hole between them (a traversal whose widening limit
    is smaller does not get the ticket that one with a larger limit, counting more claims in flight, draws after it).
    The expansion takes the node's next free edge slot whatever the ticket says, so the first `node_expanded` slots of
    every node always have children."""
    from mcts_numba_cuda_amd.puct_gomoku import PUCTGomoku
    board, turn = random_gomoku_root(np.random.default_rng(35), 15, 15, 20)
    for c_pw in (1.0, 3.0):
        e = PUCTGomoku(board_shape=(15, 15), trees=16, traversals=16, max_nodes=16384, path_depth=64, cpuct=1.5, c_pw=c_pw, seed=1)
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
    traversals = 256 leaves per step, 4000 steps, c_pw = 16 (a node without children admits a ticket per traversal, so no
    traversal ends busy and every step evaluates 256 leaves), room for 65536 nodes per tree (64001 get used).  Every field
    of every created node of every tree equals the host oracle's; the structural invariants are checked on two trees."""
    from mcts_numba_cuda_amd.puct_gomoku import ARRAYS, PUCTGomoku
    trees, traversals, steps, max_nodes = 16, 16, 4000, 65536
    board = np.zeros((15, 15), np.int8)
    kw = dict(trees=trees, traversals=traversals, max_nodes=max_nodes, path_depth=64, cpuct=1.5, c_pw=16.0, alpha_pw=0.5,
              dirichlet_alpha=0.3, seed=0)
    e = PUCTGomoku(**kw)
    best = e.run(board, 1, steps)
    print(f"device: {e.performance_info['leaves_per_second'] / 1e6:.2f} M leaves/s, {e.performance_info['leaves_per_step']:.1f} leaves per step", flush=True)
    want = po.gomoku_search(board, 1, steps, threads=16, **kw)
    small = {name: e.read_array(name) for name in ARRAYS if ARRAYS[name][2] in ("T", "TN", "TW")}
    for name in small:
        if name in ("node_count", "out_selected", "out_len"):
            assert np.array_equal(small[name], want[name]), name
    nodes, edges = created_rows(want)
    for name in ("node_expanded", "node_expand_inflight", "node_legal", "node_turn", "node_value"):
        assert np.array_equal(small[name][nodes], want[name][nodes]), name
    assert np.array_equal(e.read_array("node_board")[nodes], want["node_board"][nodes])
    for name in ("edge_child", "edge_n", "edge_w", "edge_prior", "edge_action", "edge_inflight"):
        got = e.read_array(name)
        assert np.array_equal(got[edges], want[name][edges]), name
        del got
    sel = e.selections
    assert sum(sel.values()) == steps * trees * traversals and sel["expand"] == steps * trees * traversals   # nothing busy
    assert e.performance_info["leaves_per_step"] == trees * traversals
    assert e.result.steps == steps and e.result.nodes_total == int(want["node_count"].sum()) == e.result.expansions_committed + trees
    assert e.result.max_nodes_in_tree == steps * traversals + 1
    assert board.reshape(-1)[best] == 0 and e.root_n[best] == e.root_n.max() and int(e.root_n.sum()) == sel["expand"]
    two = {name: (a[:2] if name != "tally" else a) for name, a in want.items()}
    gc.check_trees(two, board, 1, 15, 15, max_nodes, 64, tree_not_full_required=True)
    gc.check_visit_flow(two, 64)
    e.close()


def test_reference_default_widening_at_full_size():
    """The same shape with the reference's default widening constant (c_pw = 1, src/puct/puct_gpu_v3_cpp.py:121): a node
    without children admits one ticket, so most of a step's 16 traversals per tree end busy behind the first to arrive
    (the host oracle shows the same share: it follows from the rule, not from timing).  GPU == oracle on every tree."""
    from mcts_numba_cuda_amd.puct_gomoku import PUCTGomoku
    trees, traversals, steps, max_nodes = 16, 16, 4000, 16384
    board = np.zeros((15, 15), np.int8)
    kw = dict(trees=trees, traversals=traversals, max_nodes=max_nodes, path_depth=64, cpuct=1.5, c_pw=1.0, dirichlet_alpha=0.3, seed=0)
    e = PUCTGomoku(**kw)
    e.run(board, 1, steps)
    want = po.gomoku_search(board, 1, steps, threads=16, **kw)
    assert_same_trees(read_all(e), want)
    sel = e.selections
    assert [sel[k] for k in ("invalid", "expand", "terminal", "depth_limit", "busy")] == want["tally"][:, :5].sum(axis=0).tolist()
    assert 0.5 < e.performance_info["busy_share"] < 0.9
    e.close()


@pytest.mark.parametrize("traversals", [16, 1])
def test_node_limit_stops_growth_and_the_search_goes_on(traversals):
    """With the benchmark's shape but room for 2048 nodes per tree, the trees fill up well before the last step.
    From then on the expansions of a step are committed together or not at all, the traversals evaluate the node they
    reached instead, and the search continues on trees that no longer grow."""
    from mcts_numba_cuda_amd.puct_gomoku import PUCTGomoku
    trees, steps, max_nodes = 16, 1500 if traversals > 1 else 6000, 2048
    board = np.zeros((15, 15), np.int8)
    kw = dict(trees=trees, traversals=traversals, max_nodes=max_nodes, path_depth=64, cpuct=1.5, c_pw=4.0, dirichlet_alpha=0.3, seed=2)
    e = PUCTGomoku(**kw)
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
    assert_same_trees(h, po.gomoku_search(board, 1, steps, **kw))
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
    for bad in (dict(board_shape=(17, 17)), dict(traversals=17), dict(max_nodes=(1 << 20) + 1), dict(dirichlet_alpha=1.5),
                dict(path_depth=0), dict(path_depth=257), dict(trees=0), dict(evaluators=9), dict(evaluators=-1)):
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
