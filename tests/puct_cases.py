"""Known-answer cases of the PUCT select / backup path, restated from the reference's kernel tests
(src/puct/test_puct_gpu_v3.py:1154-1416, src/puct/test_puct_gpu_v2.py:1085-1119).  Every case is a host-side tree, the
launch parameters and a check of the state after selection and after the claims were released; `runner` is either the
CPU oracle or the HIP library, so both are held to the same answers.  Cases with several traversals only assert what
every interleaving of the traversals satisfies."""
import numpy as np

TERMINAL = -1
NODE_LIMIT = 16384
INVALID, EXPAND, TERMINAL_KIND, DEPTH_LIMIT, BUSY = range(5)
PACKED_INVALID = 0x3FFF


def decode(raw):
    raw = int(raw)
    return (raw >> 22) & 7, (raw >> 14) & 0xFF, raw & 0x3FFF


def reason(raw):
    return (int(raw) >> 25) & 0x3F


def make_case(trees=1, nodes=4, actions=4, warps=1, path_depth=4):
    """Empty trees with prior 1 everywhere (the layout of src/puct/test_puct_gpu_v3.py:85-111)."""
    return {
        "edge_child": np.full((trees, nodes, actions), -1, np.int32),
        "edge_prior": np.ones((trees, nodes, actions), np.float32),
        "edge_w": np.zeros((trees, nodes, actions), np.float32),
        "edge_n": np.zeros((trees, nodes, actions), np.int32),
        "edge_inflight": np.zeros((trees, nodes, actions), np.int32),
        "node_expand_inflight": np.zeros((trees, nodes), np.int32),
        "node_expanded": np.zeros((trees, nodes), np.int32),
        "node_count": np.full((trees,), nodes, np.int32),
        "out_selected": np.full((trees, warps), PACKED_INVALID, np.int32),
        "out_path": np.full((trees, warps, max(1, path_depth)), -1, np.int32),
        "out_len": np.zeros((trees, warps), np.int32),
    }


def inflight_sum(h):
    return int(h["edge_inflight"].sum()) + int(h["node_expand_inflight"].sum())


def inflight_nonnegative(h):
    return not np.any(h["edge_inflight"] < 0) and not np.any(h["node_expand_inflight"] < 0)


class Runner:
    """select(case, **params) -> host arrays after selection; release() -> host arrays after the claims of that
    selection were released (no statistics); backup(values) -> host arrays after an edge-level backup."""

    def select(self, case, **params):
        raise NotImplementedError

    def release(self):
        raise NotImplementedError

    def backup(self, values):
        raise NotImplementedError


def kinds(h):
    return [decode(r)[0] for r in h["out_selected"][0]]


# ---- the cases (each returns None or raises AssertionError) -------------------------------------------------------
def case_fresh_root_expand(r):
    h = r.select(make_case(nodes=2, actions=4, path_depth=2))
    assert decode(h["out_selected"][0, 0]) == (EXPAND, 0, 0) and reason(h["out_selected"][0, 0]) == 1
    assert h["out_len"][0, 0] == 1 and h["node_expand_inflight"][0, 0] == 1
    assert inflight_sum(r.release()) == 0


def case_terminal_root(r):
    c = make_case(nodes=2, actions=4, path_depth=2)
    c["node_expanded"][0, 0] = TERMINAL
    h = r.select(c)
    kind, _, node = decode(h["out_selected"][0, 0])
    assert (kind, node) == (TERMINAL_KIND, 0) and h["out_len"][0, 0] == 1 and inflight_sum(h) == 0
    assert reason(h["out_selected"][0, 0]) == 2


def case_invalid_child_rolls_back(r):
    c = make_case(nodes=2, actions=4, path_depth=4)
    c["node_expanded"][0, 0] = 1
    c["node_expanded"][0, 1] = -2
    c["edge_child"][0, 0, 0] = 1
    c["edge_n"][0, 0, 0] = 1
    h = r.select(c)
    assert decode(h["out_selected"][0, 0])[0] == INVALID and reason(h["out_selected"][0, 0]) == 11
    assert inflight_sum(h) == 0 and h["out_len"][0, 0] == 0


def case_child_beyond_node_count(r):
    c = make_case(nodes=4, actions=4, path_depth=3)
    c["node_count"][0] = 2
    c["node_expanded"][0, 0] = 1
    c["edge_child"][0, 0, 0] = 3
    c["edge_n"][0, 0, 0] = 1
    h = r.select(c)
    assert decode(h["out_selected"][0, 0])[0] == INVALID and reason(h["out_selected"][0, 0]) == 15
    assert inflight_sum(h) == 0


def case_progressive_widening_unique_slots(r):
    c = make_case(nodes=3, actions=4, warps=4, path_depth=2)
    c["node_expanded"][0, 0] = 1
    c["edge_child"][0, 0, 0] = 1
    c["edge_n"][0, 0, 0] = 16
    h = r.select(c, c_pw=1.0, alpha_pw=0.5)
    root_slots, child_expands = [], 0
    for wid in range(4):
        kind, slot, node = decode(h["out_selected"][0, wid])
        if kind == EXPAND:
            assert node in (0, 1)
            if node == 0:
                root_slots.append(slot)
            else:
                child_expands += 1
        else:
            assert kind == BUSY
    assert sorted(root_slots) == [1, 2, 3] and child_expands <= 1
    assert h["node_expand_inflight"][0, 0] == 3
    assert inflight_sum(r.release()) == 0


def case_single_edge_contention(r):
    c = make_case(nodes=2, actions=4, warps=8, path_depth=2)
    c["node_expanded"][0, 0] = 1
    c["edge_child"][0, 0, 0] = 1
    c["edge_n"][0, 0, 0] = 1
    c["node_expanded"][0, 1] = TERMINAL
    h = r.select(c, c_pw=0.0)
    k = kinds(h)
    valid, busy = k.count(TERMINAL_KIND), k.count(BUSY)
    assert valid > 0 and valid + busy == 8 and h["edge_inflight"][0, 0, 0] == valid
    assert inflight_sum(r.release()) == 0


def case_full_ticket_quota_falls_through(r):
    c = make_case(nodes=3, actions=4, warps=2, path_depth=2)
    c["node_expanded"][0, 0] = 1
    c["node_expand_inflight"][0, 0] = 3
    c["edge_child"][0, 0, 0] = 1
    c["edge_n"][0, 0, 0] = 16
    c["node_expanded"][0, 1] = TERMINAL
    h = r.select(c, c_pw=1.0, alpha_pw=0.5)
    k = kinds(h)
    valid, busy = k.count(TERMINAL_KIND), k.count(BUSY)
    assert valid > 0 and valid + busy == 2
    assert all(decode(x)[2] in (0, 1) for x in h["out_selected"][0])
    assert h["edge_inflight"][0, 0, 0] == valid and h["node_expand_inflight"][0, 0] == 3
    h2 = r.release()
    assert h2["node_expand_inflight"][0, 0] == 3 and h2["edge_inflight"][0, 0, 0] == 0


def _two_terminal_children():
    c = make_case(nodes=4, actions=4, warps=8, path_depth=2)
    c["node_expanded"][0, 0] = 2
    for slot, child in enumerate((1, 2)):
        c["edge_child"][0, 0, slot] = child
        c["edge_n"][0, 0, slot] = 1
        c["node_expanded"][0, child] = TERMINAL
    return c


def case_strict_winner(r):
    h = r.select(_two_terminal_children(), c_pw=0.0, soft_winner=0)
    k = kinds(h)
    assert k.count(TERMINAL_KIND) > 0 and k.count(TERMINAL_KIND) + k.count(BUSY) == 8
    assert int(h["edge_inflight"][0, 0].sum()) == k.count(TERMINAL_KIND)
    assert inflight_sum(r.release()) == 0


def case_soft_winner(r):
    h = r.select(_two_terminal_children(), c_pw=0.0, soft_winner=1)
    assert kinds(h) == [TERMINAL_KIND] * 8 and int(h["edge_inflight"][0, 0].sum()) == 8
    assert inflight_sum(r.release()) == 0


def case_fully_expanded_select_release(r):
    c = make_case(nodes=3, actions=4, path_depth=4)
    c["node_expanded"][0, 0] = 2
    c["edge_child"][0, 0, :2] = (1, 2)
    c["edge_prior"][0, 0, :2] = (0.1, 0.9)
    c["edge_n"][0, 0, :2] = 1
    h = r.select(c)
    assert decode(h["out_selected"][0, 0]) == (EXPAND, 0, 2)
    assert h["out_path"][0, 0, 0] == 1 and h["out_len"][0, 0] == 2
    assert h["edge_inflight"][0, 0, 1] == 1 and h["node_expand_inflight"][0, 2] == 1
    assert inflight_sum(r.release()) == 0


def case_fully_expanded_select_backup(r):
    """Statistics after a backup with value 0.7 on the one path edge (src/puct/test_puct_gpu_v2.py:1085-1119)."""
    c = make_case(nodes=3, actions=4, path_depth=4)
    c["node_expanded"][0, 0] = 2
    c["edge_child"][0, 0, :2] = (1, 2)
    c["edge_prior"][0, 0, :2] = (0.1, 0.9)
    c["edge_n"][0, 0, :2] = 1
    r.select(c)
    values = np.zeros((1, 1, 4), np.float32)
    values[0, 0, 0] = 0.7
    h2 = r.backup(values)
    assert inflight_sum(h2) == 0 and h2["edge_n"][0, 0, 1] == 2 and h2["edge_n"][0, 0, 0] == 1
    assert h2["edge_w"][0, 0, 1] == np.float32(0.7) and h2["edge_w"][0, 0, 0] == 0


def case_depth_limit(r):
    c = make_case(nodes=3, actions=4, path_depth=1)
    c["node_expanded"][0, :2] = 1
    c["edge_child"][0, 0, 0] = 1
    c["edge_child"][0, 1, 0] = 2
    c["edge_n"][0, 0, 0] = 1
    c["edge_n"][0, 1, 0] = 1
    h = r.select(c)
    kind, _, node = decode(h["out_selected"][0, 0])
    assert (kind, node) == (DEPTH_LIMIT, 1) and h["out_len"][0, 0] == 2 and h["edge_inflight"][0, 0, 0] == 1
    assert inflight_sum(r.release()) == 0


def case_zero_n_edge_selectable(r):
    c = make_case(nodes=3, actions=4, path_depth=3)
    c["node_expanded"][0, 0] = 1
    c["edge_child"][0, 0, 0] = 1
    h = r.select(c)
    kind, _, node = decode(h["out_selected"][0, 0])
    assert (kind, node) == (EXPAND, 1) and h["out_len"][0, 0] == 2


def case_encoding_boundaries(r):
    assert decode(r.select(make_case(nodes=2, actions=256, path_depth=2))["out_selected"][0, 0])[0] == EXPAND
    h = r.select(make_case(nodes=2, actions=257, path_depth=2))
    assert decode(h["out_selected"][0, 0])[0] == INVALID and reason(h["out_selected"][0, 0]) == 10
    assert decode(r.select(make_case(nodes=NODE_LIMIT + 1, actions=4, path_depth=2))["out_selected"][0, 0])[0] == INVALID
    c = make_case(nodes=NODE_LIMIT + 1, actions=4, path_depth=2)
    c["node_count"][0] = NODE_LIMIT
    assert decode(r.select(c)["out_selected"][0, 0])[0] == EXPAND


# ---- cases beyond the reference's: what the arithmetic fixes -----------------------------------------------------
def case_hand_computed_scores(r):
    """Three edges, parent_n_eff = 2 + 5 + 9 = 16, sqrt = 4, cpuct = 1.5, no widening (c_pw = 0 with 3 edges expanded
    gives allowed = 1).  Scores: e0 = 1.0/2 + 1.5*0.2*4/3 = 0.9, e1 = 3.5/5 + 1.5*0.3*4/6 = 1.0,
    e2 = 2.7/9 + 1.5*0.5*4/10 = 0.6  ->  edge 1."""
    c = make_case(nodes=4, actions=4, path_depth=3)
    c["node_expanded"][0, 0] = 3
    c["node_expanded"][0, 1:] = TERMINAL
    c["edge_child"][0, 0, :3] = (1, 2, 3)
    c["edge_n"][0, 0, :3] = (2, 5, 9)
    c["edge_w"][0, 0, :3] = (1.0, 3.5, 2.7)
    c["edge_prior"][0, 0, :3] = (0.2, 0.3, 0.5)
    h = r.select(c, cpuct=1.5, c_pw=0.0)
    assert decode(h["out_selected"][0, 0]) == (TERMINAL_KIND, 0, 2) and h["out_path"][0, 0, 0] == 1


def case_virtual_loss_lowers_score(r):
    """Same tree with 3 visits in flight on edge 1: parent_n_eff = 19, sqrt(19) = 4.3589; e0 = 0.5 + 0.3*4.3589/3 =
    0.936, e1 = 0.7 + 0.45*4.3589/9 = 0.918, e2 = 0.3 + 0.75*4.3589/10 = 0.627  ->  edge 0."""
    c = make_case(nodes=4, actions=4, path_depth=3)
    c["node_expanded"][0, 0] = 3
    c["node_expanded"][0, 1:] = TERMINAL
    c["edge_child"][0, 0, :3] = (1, 2, 3)
    c["edge_n"][0, 0, :3] = (2, 5, 9)
    c["edge_w"][0, 0, :3] = (1.0, 3.5, 2.7)
    c["edge_prior"][0, 0, :3] = (0.2, 0.3, 0.5)
    c["edge_inflight"][0, 0, 1] = 3
    h = r.select(c, cpuct=1.5, c_pw=0.0)
    assert decode(h["out_selected"][0, 0]) == (TERMINAL_KIND, 0, 1) and h["out_path"][0, 0, 0] == 0
    assert h["edge_inflight"][0, 0, 0] == 1 and h["edge_inflight"][0, 0, 1] == 3


def case_tie_rotation_by_wid(r):
    """Five edges with prior 0 and equal Q: the exploration term is 0 whatever is in flight, so all scores stay tied and
    traversal wid takes the edge whose rotated index (eid - wid mod 5) is smallest, i.e. edge wid, under every
    interleaving (no two of the five traversals ever claim the same edge)."""
    span = 5
    c = make_case(nodes=span + 1, actions=8, warps=span, path_depth=2)
    c["node_expanded"][0, 0] = span
    c["node_expanded"][0, 1:] = TERMINAL
    c["edge_child"][0, 0, :span] = np.arange(1, span + 1)
    c["edge_n"][0, 0, :span] = 4
    c["edge_w"][0, 0, :span] = 1.0
    c["edge_prior"][0, 0, :span] = 0.0
    h = r.select(c, c_pw=0.0)
    for wid in range(span):
        assert decode(h["out_selected"][0, wid]) == (TERMINAL_KIND, 0, wid + 1)
        assert h["out_path"][0, wid, 0] == wid
    assert np.array_equal(h["edge_inflight"][0, 0, :span], np.ones(span, np.int32))
    assert inflight_sum(r.release()) == 0


def case_tie_rotation_across_slices_and_around(r):
    """200 expanded edges with prior 0 (scores do not depend on what is in flight); the best Q sits on edges 3, 70 and
    130.  Traversal wid takes the first of them at or after index wid, and edge 3 again once wid is beyond 130 (the
    rotated index eid - wid mod 200 is smallest there), whatever the interleaving; with the soft winner every claim
    lands, so the counts are known too.  140 traversals: offsets in every 64-edge slice, spread over nine workgroups."""
    span, warps, best = 200, 140, (3, 70, 130)
    c = make_case(nodes=span + 1, actions=256, warps=warps, path_depth=2)
    c["node_expanded"][0, 0] = span
    c["node_expanded"][0, 1:] = TERMINAL
    c["edge_child"][0, 0, :span] = np.arange(1, span + 1)
    c["edge_n"][0, 0, :span] = 4
    c["edge_w"][0, 0, :span] = 1.0
    c["edge_w"][0, 0, list(best)] = 2.0
    c["edge_prior"][0, 0, :span] = 0.0
    h = r.select(c, c_pw=0.0, soft_winner=1)
    want = [next((e for e in best if e >= wid), best[0]) for wid in range(warps)]
    assert h["out_path"][0, :, 0].tolist() == want
    assert [decode(x) for x in h["out_selected"][0]] == [(TERMINAL_KIND, 0, e + 1) for e in want]
    counts = np.zeros(256, np.int32)
    np.add.at(counts, want, 1)
    assert np.array_equal(h["edge_inflight"][0, 0], counts)
    assert inflight_sum(r.release()) == 0


def case_wide_node_beyond_one_wavefront(r):
    """200 expanded edges; the single best one sits at index 137 (beyond the first 64 lanes) because of its prior."""
    e = 200
    c = make_case(nodes=e + 1, actions=256, path_depth=2)
    c["node_expanded"][0, 0] = e
    c["node_expanded"][0, 1:] = TERMINAL
    c["edge_child"][0, 0, :e] = np.arange(1, e + 1)
    c["edge_n"][0, 0, :e] = 1
    c["edge_prior"][0, 0, :e] = 0.001
    c["edge_prior"][0, 0, 137] = 0.5
    h = r.select(c, c_pw=0.0)
    assert decode(h["out_selected"][0, 0]) == (TERMINAL_KIND, 0, 138)
    assert h["out_path"][0, 0, 0] == 137 and h["edge_inflight"][0, 0, 137] == 1 and inflight_sum(h) == 1


def case_nan_and_minus_inf_never_win(r):
    """An edge whose score is NaN or -inf never beats the initial (-FLT_MAX, none) of the reference's scan
    (src/puct/puct_gpu_v3_cpp.cu:58-71,189-191), so a node with only such edges reports NO_VALID_EDGE."""
    c = make_case(nodes=3, actions=4, path_depth=2)
    c["node_expanded"][0, 0] = 2
    c["edge_child"][0, 0, :2] = (1, 2)
    c["edge_n"][0, 0, :2] = 1
    c["edge_w"][0, 0, 0] = np.nan
    c["edge_w"][0, 0, 1] = -np.inf
    h = r.select(c, c_pw=0.0)
    assert decode(h["out_selected"][0, 0])[0] == INVALID and reason(h["out_selected"][0, 0]) == 14
    assert inflight_sum(h) == 0


def case_deep_chain_rollback(r):
    """A chain of 100 single-edge nodes ending in an invalid node word: all 100 claims are taken back (the rollback
    spans more path entries than a wavefront has lanes)."""
    n = 102
    c = make_case(nodes=n, actions=2, path_depth=128)
    c["node_expanded"][0, :100] = 1
    c["edge_child"][0, np.arange(100), 0] = np.arange(1, 101)
    c["edge_n"][0, :100, 0] = 1
    c["node_expanded"][0, 100] = -7
    h = r.select(c, c_pw=0.0)
    assert decode(h["out_selected"][0, 0])[0] == INVALID and reason(h["out_selected"][0, 0]) == 11
    assert inflight_sum(h) == 0 and h["out_len"][0, 0] == 0


def case_deep_chain_terminal(r):
    n = 102
    c = make_case(nodes=n, actions=2, path_depth=128)
    c["node_expanded"][0, :100] = 1
    c["edge_child"][0, np.arange(100), 0] = np.arange(1, 101)
    c["edge_n"][0, :100, 0] = 1
    c["node_expanded"][0, 100] = TERMINAL
    h = r.select(c, c_pw=0.0)
    assert decode(h["out_selected"][0, 0]) == (TERMINAL_KIND, 0, 100) and h["out_len"][0, 0] == 101
    assert np.array_equal(h["out_path"][0, 0, :100], np.arange(100) << 8)
    assert int(h["edge_inflight"].sum()) == 100
    assert inflight_sum(r.release()) == 0


REFERENCE_CASES = [case_fresh_root_expand, case_terminal_root, case_invalid_child_rolls_back,
                   case_child_beyond_node_count, case_progressive_widening_unique_slots, case_single_edge_contention,
                   case_full_ticket_quota_falls_through, case_strict_winner, case_soft_winner,
                   case_fully_expanded_select_release, case_fully_expanded_select_backup, case_depth_limit,
                   case_zero_n_edge_selectable, case_encoding_boundaries]
ARITHMETIC_CASES = [case_hand_computed_scores, case_virtual_loss_lowers_score, case_tie_rotation_by_wid,
                    case_tie_rotation_across_slices_and_around, case_wide_node_beyond_one_wavefront, case_nan_and_minus_inf_never_win, case_deep_chain_rollback,
                    case_deep_chain_terminal]
ALL_CASES = REFERENCE_CASES + ARITHMETIC_CASES


def random_forest(rng, trees, nodes, actions, warps, path_depth, terminal_fraction=0.2, fill=0.6):
    """Random consistent trees: node i > 0 hangs under an earlier node with free edge slots; a share of the leaves is
    terminal; statistics are random but consistent in sign and size.  Used to compare the library with the oracle."""
    c = make_case(trees=trees, nodes=nodes, actions=actions, warps=warps, path_depth=path_depth)
    for t in range(trees):
        used = int(max(2, nodes * fill))
        c["node_count"][t] = used
        expanded = np.zeros(nodes, np.int32)
        for i in range(1, used):
            while True:
                p = int(rng.integers(0, i))
                if expanded[p] < actions:
                    break
            s = expanded[p]
            expanded[p] += 1
            c["edge_child"][t, p, s] = i
            n = int(rng.integers(0, 20))
            c["edge_n"][t, p, s] = n
            c["edge_w"][t, p, s] = np.float32(rng.uniform(-1, 1) * n)
            c["edge_prior"][t, p, s] = np.float32(rng.uniform(0.01, 1.0))
        c["node_expanded"][t] = expanded
        leaves = np.flatnonzero(expanded[:used] == 0)
        term = leaves[rng.random(leaves.size) < terminal_fraction]
        c["node_expanded"][t, term] = TERMINAL
    return c


def wide_forest(rng, trees, nodes, actions, warps, path_depth, hubs=2, claims=0.05, terminal_fraction=0.15, fill=0.8):
    """Random consistent trees with wide nodes: four new nodes in five hang under one of the first `hubs` nodes while
    those have free edge slots, so the top levels fill several 64-edge slices; half of the priors come from four values
    (equal scores in different slices), a fifth of the edges is unvisited, and a share `claims` of all edge slots
    already holds one to three claims."""
    c = make_case(trees=trees, nodes=nodes, actions=actions, warps=warps, path_depth=path_depth)
    for t in range(trees):
        used = int(max(2, nodes * fill))
        c["node_count"][t] = used
        expanded = np.zeros(nodes, np.int32)
        for i in range(1, used):
            while True:
                p = int(rng.integers(0, min(i, hubs))) if rng.random() < 0.8 else int(rng.integers(0, i))
                if expanded[p] < actions:
                    break
            s = expanded[p]
            expanded[p] += 1
            c["edge_child"][t, p, s] = i
            n = int(rng.integers(0, 20)) if rng.random() < 0.8 else 0
            c["edge_n"][t, p, s] = n
            c["edge_w"][t, p, s] = np.float32(rng.uniform(-1, 1) * n)
            c["edge_prior"][t, p, s] = np.float32(rng.choice([0.1, 0.25, 0.5, 1.0]) if rng.random() < 0.5 else rng.uniform(0.01, 1.0))
        c["node_expanded"][t] = expanded
        leaves = np.flatnonzero(expanded[:used] == 0)
        term = leaves[rng.random(leaves.size) < terminal_fraction]
        c["node_expanded"][t, term] = TERMINAL
    if claims:
        held = rng.random(c["edge_inflight"].shape) < claims
        c["edge_inflight"][held] = rng.integers(1, 4, int(held.sum()))
    return c
