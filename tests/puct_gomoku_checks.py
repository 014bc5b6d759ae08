"""Structural checks of a finished Gomoku PUCT search that hold for the sequential oracle and for every interleaving
of concurrent traversals on the GPU; `h` maps array names (include/puct_gomoku.h) to host arrays."""
import numpy as np


def cells_of(words, cells):
    bits = np.unpackbits(words.view(np.uint8), bitorder="little")
    return bits[:cells].astype(bool)


def run_through(stones, m, n, cell):
    """Longest run through `cell` in each of the four directions on a boolean [m * n] array that holds the stone."""
    r0, c0 = divmod(cell, n)
    runs = []
    for dr, dc in ((0, 1), (1, 0), (1, 1), (1, -1)):
        run = 1
        for s in (-1, 1):
            k = 1
            while True:
                r, c = r0 + s * k * dr, c0 + s * k * dc
                if not (0 <= r < m and 0 <= c < n and stones[r * n + c]):
                    break
                run += 1
                k += 1
        runs.append(run)
    return runs


def check_trees(h, root_board, root_turn, m, n, max_nodes, path_depth, tree_not_full_required=False):
    cells = m * n
    T = h["node_count"].shape[0]
    # nothing is left in flight on any created node (rows of nodes that were never created are uninitialised)
    for t in range(T):
        count = int(h["node_count"][t])
        assert not np.any(h["node_expand_inflight"][t, :count])
        for node in range(count):
            assert not np.any(h["edge_inflight"][t, node, :int(h["node_legal"][t, node])]), (t, node)
    root_pos = (root_board.reshape(-1) == 1)
    root_neg = (root_board.reshape(-1) == -1)
    for t in range(T):
        count = int(h["node_count"][t])
        assert 1 <= count <= max_nodes
        if tree_not_full_required:
            assert count < max_nodes
        pos0, neg0 = cells_of(h["node_board"][t, 0, :8], cells), cells_of(h["node_board"][t, 0, 8:], cells)
        assert np.array_equal(pos0, root_pos) and np.array_equal(neg0, root_neg) and h["node_turn"][t, 0] == root_turn
        seen_children = set()
        for node in range(count):
            ne = int(h["node_expanded"][t, node])
            pos, neg = cells_of(h["node_board"][t, node, :8], cells), cells_of(h["node_board"][t, node, 8:], cells)
            assert not np.any(pos & neg)
            legal = np.flatnonzero(~(pos | neg))
            turn = int(h["node_turn"][t, node])
            if ne == -1:
                continue
            assert 0 <= ne <= legal.size
            # the edge slots are a permutation of the legal cells in descending prior order, priors sum to one
            acts = h["edge_action"][t, node, :legal.size].astype(int)
            assert sorted(acts.tolist()) == legal.tolist()
            pri = h["edge_prior"][t, node, :legal.size].astype(np.float64)
            assert np.all(np.diff(pri) <= 0) and abs(pri.sum() - 1.0) < 1e-4
            child_visits = 0
            for s in range(ne):
                child = int(h["edge_child"][t, node, s])
                assert 0 < child < count and child not in seen_children, (
                    t, node, s, child, count, ne, h["edge_child"][t, node, :ne + 3].tolist(), h["edge_n"][t, node, :ne + 3].tolist(),
                    int(h["node_expand_inflight"][t, node]), int(h["node_legal"][t, node]))
                seen_children.add(child)
                a = acts[s]
                cpos, cneg = cells_of(h["node_board"][t, child, :8], cells), cells_of(h["node_board"][t, child, 8:], cells)
                epos, eneg = pos.copy(), neg.copy()
                (epos if turn > 0 else eneg)[a] = True
                assert np.array_equal(cpos, epos) and np.array_equal(cneg, eneg)
                assert h["node_turn"][t, child] == -turn
                five = 5 in run_through(epos if turn > 0 else eneg, m, n, a)
                full = legal.size == 1
                assert (h["node_expanded"][t, child] == -1) == (five or full)
                if five:
                    assert h["node_value"][t, child] == -1.0
                    # every visit of the winning move scores +1 for the mover
                    assert h["edge_w"][t, node, s] == h["edge_n"][t, node, s]
                elif full:
                    assert h["node_value"][t, child] == 0.0 and h["edge_w"][t, node, s] == 0.0
                assert h["edge_n"][t, node, s] >= 1 and abs(h["edge_w"][t, node, s]) <= h["edge_n"][t, node, s] + 1e-3
                child_visits += int(h["edge_n"][t, node, s])
            for s in range(ne, legal.size):
                assert h["edge_child"][t, node, s] == -1 and h["edge_n"][t, node, s] == 0
            if node != 0:
                continue
        assert len(seen_children) == count - 1
    return True


def visits_below(h, t, node):
    ne = int(h["node_expanded"][t, node])
    return 0 if ne <= 0 else int(h["edge_n"][t, node, :ne].sum())


def check_visit_flow(h, path_depth):
    """Without a full tree and without depth-limit evaluations every visit of an edge beyond the one that created it
    went on to an edge of the child: N(edge) - 1 == sum of the child's edge visits (terminal children excepted)."""
    T = h["node_count"].shape[0]
    for t in range(T):
        count = int(h["node_count"][t])
        for node in range(count):
            ne = int(h["node_expanded"][t, node])
            for s in range(max(ne, 0)):
                child = int(h["edge_child"][t, node, s])
                if h["node_expanded"][t, child] == -1:
                    continue
                assert int(h["edge_n"][t, node, s]) - 1 == visits_below(h, t, child), (t, node, s)
