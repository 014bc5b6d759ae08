"""Known-answer cases of PUCT selection with node-level virtual loss (the two select kernels of
src/puct/puct_gpu_v2.py:573-840) and the backup that takes it back, restated from the reference's kernel tests
(src/puct/test_puct_gpu_v2.py:1006-1166) plus cases whose answer the arithmetic fixes.  `runner` is either the CPU oracle
or the HIP library, so both are held to the same answers; `variant` is "preclaim" or "winner_recalc".  Cases with several
traversals only assert what every interleaving of the traversals satisfies."""
import numpy as np

import puct_cases as pc
from puct_cases import DEPTH_LIMIT, EXPAND, INVALID, PACKED_INVALID, TERMINAL, TERMINAL_KIND

VARIANTS = ("preclaim", "winner_recalc")


def decode(raw):
    """src/puct/test_puct_gpu_v2.py:71-75: the v2 word has no reason field."""
    raw = int(raw)
    return raw >> 22, (raw >> 14) & 0xFF, raw & 0x3FFF


def make_case(trees=1, nodes=4, actions=4, warps=1, path_depth=4):
    """src/puct/test_puct_gpu_v2.py:78-106."""
    c = pc.make_case(trees=trees, nodes=nodes, actions=actions, warps=warps, path_depth=path_depth)
    del c["edge_inflight"]
    c["node_inflight"] = np.zeros((trees, nodes), np.int32)
    return c


def inflight_sum(h):
    return int(h["node_inflight"].sum()) + int(h["node_expand_inflight"].sum())


def inflight_nonnegative(h):
    return not np.any(h["node_inflight"] < 0) and not np.any(h["node_expand_inflight"] < 0)


class Runner:
    """select(case, variant, **params) -> host arrays after selection; backup(values) -> host arrays after the node-level
    backup of that selection (values: float32 [trees, warps, path_depth])."""

    sequential = False   # True: the traversals of a launch run one after another, wid ascending

    def select(self, case, variant, **params):
        raise NotImplementedError

    def backup(self, values):
        raise NotImplementedError


def zeros_like_path(h):
    return np.zeros(h["out_path"].shape, np.float32)


def score(cpuct, prior, w, n, inflight, parent_eff):
    """src/puct/puct_gpu_v2.py:271-287 in float32, operation for operation."""
    f = np.float32
    q = f(w) / f(n) if n > 0 else f(0)
    u = f(f(f(cpuct) * f(prior)) * np.sqrt(f(parent_eff))) / f(n + inflight + 1)
    return f(q + u)


# ---- the reference's cases ------------------------------------------------------------------------------------------
def case_fresh_root_expand_roundtrip(r, variant):
    """:1006-1020"""
    h = r.select(make_case(nodes=2, actions=4, path_depth=2), variant)
    assert decode(h["out_selected"][0, 0]) == (EXPAND, 0, 0) and h["out_len"][0, 0] == 1
    assert h["node_expand_inflight"][0, 0] == 1
    assert inflight_sum(r.backup(zeros_like_path(h))) == 0


def case_terminal_root(r, variant):
    """:1023-1034"""
    c = make_case(nodes=2, actions=4, path_depth=2)
    c["node_expanded"][0, 0] = TERMINAL
    h = r.select(c, variant)
    assert decode(h["out_selected"][0, 0]) == (TERMINAL_KIND, 0, 0) and h["out_len"][0, 0] == 1 and inflight_sum(h) == 0


def case_invalid_child_rolls_back(r, variant):
    """:1037-1047: the child's node word is neither a count nor the terminal mark; the claim on it is given back."""
    c = make_case(nodes=2, actions=4, path_depth=4)
    c["node_expanded"][0, 0] = 1
    c["node_expanded"][0, 1] = -2
    c["edge_child"][0, 0, 0] = 1
    c["edge_n"][0, 0, 0] = 1
    h = r.select(c, variant)
    assert h["out_selected"][0, 0] == PACKED_INVALID and h["out_len"][0, 0] == 0 and inflight_sum(h) == 0


def case_child_beyond_node_count(r, variant):
    """:1050-1059"""
    c = make_case(nodes=4, actions=4, path_depth=3)
    c["node_count"][0] = 2
    c["node_expanded"][0, 0] = 1
    c["edge_child"][0, 0, 0] = 3
    c["edge_n"][0, 0, 0] = 1
    h = r.select(c, variant)
    assert decode(h["out_selected"][0, 0])[0] == INVALID and inflight_sum(h) == 0


def case_progressive_widening_unique_slots(r, variant):
    """:1062-1088: sqrt(16) = 4 children allowed, one there: three of the four traversals get slots 1, 2, 3."""
    c = make_case(nodes=3, actions=4, warps=4, path_depth=2)
    c["node_expanded"][0, 0] = 1
    c["edge_child"][0, 0, 0] = 1
    c["edge_n"][0, 0, 0] = 16
    h = r.select(c, variant, c_pw=1.0, alpha_pw=0.5)
    slots = []
    for wid in range(4):
        kind, slot, node = decode(h["out_selected"][0, wid])
        assert kind in (EXPAND, INVALID)
        if kind == EXPAND:
            assert node == 0
            slots.append(slot)
    assert sorted(slots) == [1, 2, 3] and h["node_expand_inflight"][0, 0] == 3
    assert inflight_sum(r.backup(zeros_like_path(h))) == 0


def case_fully_expanded_select_and_backup(r, variant):
    """:1091-1119: the edge with prior 0.9 wins, its child is fresh and takes an expansion ticket; the backup turns the
    virtual visit into a real one with value 0.7."""
    c = make_case(nodes=3, actions=4, path_depth=4)
    c["node_expanded"][0, 0] = 2
    c["edge_child"][0, 0, :2] = (1, 2)
    c["edge_prior"][0, 0, :2] = (0.1, 0.9)
    c["edge_n"][0, 0, :2] = 1
    h = r.select(c, variant)
    assert decode(h["out_selected"][0, 0]) == (EXPAND, 0, 2)
    assert h["out_path"][0, 0, 0] == 1 and h["out_len"][0, 0] == 2
    assert h["node_inflight"][0, 2] == 1 and h["node_inflight"][0, 1] == 0 and h["node_expand_inflight"][0, 2] == 1
    values = zeros_like_path(h)
    values[0, 0, 0] = 0.7
    h2 = r.backup(values)
    assert inflight_sum(h2) == 0 and h2["edge_n"][0, 0, 1] == 2 and h2["edge_w"][0, 0, 1] == np.float32(0.7)
    assert h2["edge_n"][0, 0, 0] == 1


def case_depth_limit(r, variant):
    """:1122-1139"""
    c = make_case(nodes=3, actions=4, path_depth=1)
    c["node_expanded"][0, :2] = 1
    c["edge_child"][0, 0, 0] = 1
    c["edge_child"][0, 1, 0] = 2
    c["edge_n"][0, :2, 0] = 1
    h = r.select(c, variant)
    assert decode(h["out_selected"][0, 0]) == (DEPTH_LIMIT, 0, 1) and h["out_len"][0, 0] == 2
    assert h["node_inflight"][0, 1] == 1
    assert inflight_sum(r.backup(zeros_like_path(h))) == 0


def case_encoding_boundaries(r, variant):
    """:1142-1166: 256 actions fit the packing, 257 do not; node_count, not the array size, gates the packed node id."""
    assert decode(r.select(make_case(nodes=2, actions=256, path_depth=2), variant)["out_selected"][0, 0])[0] == EXPAND
    assert decode(r.select(make_case(nodes=2, actions=257, path_depth=2), variant)["out_selected"][0, 0])[0] == INVALID
    big = make_case(nodes=pc.NODE_LIMIT + 1, actions=4, path_depth=2)
    assert decode(r.select(big, variant)["out_selected"][0, 0])[0] == INVALID
    big["node_count"][0] = pc.NODE_LIMIT
    assert decode(r.select(big, variant)["out_selected"][0, 0])[0] == EXPAND


# ---- what the arithmetic fixes ----------------------------------------------------------------------------------------
def _three_children(path_depth=2):
    c = make_case(nodes=4, actions=4, path_depth=path_depth)
    c["node_expanded"][0, 0] = 3
    c["node_expanded"][0, 1:] = TERMINAL
    c["edge_child"][0, 0, :3] = (1, 2, 3)
    return c


def case_hand_computed_scores(r, variant):
    """Scores worked out here in float32, :271-287; parent count = sum of visits and virtual visits, :407-416."""
    c = _three_children()
    c["edge_n"][0, 0, :3] = (10, 3, 6)
    c["edge_w"][0, 0, :3] = (6.0, 1.2, 4.5)
    c["edge_prior"][0, 0, :3] = (0.2, 0.5, 0.3)
    c["node_inflight"][0, 2] = 2
    parent = 10 + 3 + 6 + 2
    s = [score(1.7, c["edge_prior"][0, 0, e], c["edge_w"][0, 0, e], c["edge_n"][0, 0, e], c["node_inflight"][0, e + 1], parent)
         for e in range(3)]
    best = int(np.argmax(s))
    assert len(set(s)) == 3 and best == 2          # (the virtual visits on child 2 cost edge 1 the lead)
    h = r.select(c, variant, cpuct=1.7, c_pw=0.0)
    assert decode(h["out_selected"][0, 0]) == (TERMINAL_KIND, 0, best + 1) and h["out_path"][0, 0, 0] == best
    assert h["node_inflight"][0, best + 1] == 1 and h["node_inflight"][0, 2] == 2
    c["node_inflight"][0, 2] = 0                     # without them edge 1 leads
    s = [score(1.7, c["edge_prior"][0, 0, e], c["edge_w"][0, 0, e], c["edge_n"][0, 0, e], 0, 19) for e in range(3)]
    assert int(np.argmax(s)) == 1
    h = r.select(c, variant, cpuct=1.7, c_pw=0.0)
    assert h["out_path"][0, 0, 0] == 1


def case_edges_that_lead_nowhere_are_no_candidates(r, variant):
    """An expanded edge whose child id is -1 or beyond node_count is skipped: not scored, not counted (:407-445)."""
    c = _three_children()
    c["edge_child"][0, 0, 1] = -1
    c["edge_n"][0, 0, :3] = (4, 1000, 4)       # the 1000 visits would change sqrt(parent) and every score if counted
    c["edge_prior"][0, 0, :3] = (0.3, 100.0, 0.31)
    h = r.select(c, variant, c_pw=0.0)
    assert h["out_path"][0, 0, 0] == 2 and h["node_inflight"][0, 3] == 1 and int(h["node_inflight"].sum()) == 1
    c["edge_child"][0, 0, :3] = (-1, 9, -5)    # nothing left: the traversal ends without a selection
    h = r.select(c, variant, c_pw=0.0)
    assert h["out_selected"][0, 0] == PACKED_INVALID and h["out_len"][0, 0] == 0 and inflight_sum(h) == 0


def case_ties(r, variant):
    """Equal scores: the preclaim kernel rotates the edge order by wid (:121-144), the winner-recalc kernel takes the
    smallest edge index (:110-117).  One traversal per tree, wid = 0..3 in separate launches is not possible (wid is the
    position in the launch), so four trees with four traversals each would race; instead the traversals of one launch
    all see three equal edges, and only wid 0's choice is fixed: edge 0 in both kernels."""
    c = _three_children()
    c["edge_n"][0, 0, :3] = 2
    h = r.select(c, variant, c_pw=0.0)
    assert h["out_path"][0, 0, 0] == 0
    # a later equal edge does not displace an earlier one; a better one does
    c["edge_prior"][0, 0, 2] = 1.5
    assert r.select(c, variant, c_pw=0.0)["out_path"][0, 0, 0] == 2


def case_ties_across_slices_and_around(r, variant):
    """200 expanded edges with prior 0 (a score is its Q, whatever the counters hold); the best Q sits on edges 3, 70 and
    130.  Under every interleaving: the preclaim kernel's traversal wid takes the first of them at or after index wid and
    edge 3 again once wid is beyond 130 (:121-144); of the winner-recalc kernel's traversals exactly one keeps edge 3
    (the claim that found the child free), all others meet a conflict there and keep the best of the rest, edge 70
    (:520-560).  140 traversals: rotation offsets in every 64-edge slice, spread over nine workgroups."""
    span, warps, best = 200, 140, (3, 70, 130)
    c = make_case(nodes=span + 1, actions=256, warps=warps, path_depth=2)
    c["node_expanded"][0, 0] = span
    c["node_expanded"][0, 1:] = TERMINAL
    c["edge_child"][0, 0, :span] = np.arange(1, span + 1)
    c["edge_n"][0, 0, :span] = 4
    c["edge_w"][0, 0, :span] = 1.0
    c["edge_w"][0, 0, list(best)] = 2.0
    c["edge_prior"][0, 0, :span] = 0.0
    h = r.select(c, variant, c_pw=0.0)
    got = h["out_path"][0, :, 0].tolist()
    if variant == "preclaim":
        want = [next((e for e in best if e >= wid), best[0]) for wid in range(warps)]
        assert got == want
    else:
        want = [3] + [70] * (warps - 1)
        assert sorted(got) == want
    assert [decode(x) for x in h["out_selected"][0]] == [(TERMINAL_KIND, 0, e + 1) for e in got]
    counts = np.zeros(span + 1, np.int32)
    np.add.at(counts, [e + 1 for e in want], 1)
    assert np.array_equal(h["node_inflight"][0], counts)
    assert inflight_sum(r.backup(zeros_like_path(h))) == 0


def case_preclaim_rotation_by_wid(r, variant):
    """Four traversals on four equal edges.  One after another (the oracle), the preclaim kernel's traversal wid finds the
    children taken before it one claim heavier and, among the equal rest, prefers edge wid (:121-144): four different
    children.  Concurrently a traversal may also see the passing claims of the others, so only the totals are fixed."""
    c = make_case(nodes=5, actions=4, warps=4, path_depth=2)
    c["node_expanded"][0, 0] = 4
    c["node_expanded"][0, 1:] = TERMINAL
    c["edge_child"][0, 0] = (1, 2, 3, 4)
    c["edge_n"][0, 0] = 1
    h = r.select(c, variant, c_pw=0.0)
    if variant == "preclaim" and r.sequential:
        assert [int(h["out_path"][0, w, 0]) for w in range(4)] == [0, 1, 2, 3]
    assert int(h["node_inflight"].sum()) == 4 and np.all(h["node_inflight"] >= 0)
    assert inflight_sum(r.backup(zeros_like_path(h))) == 0


def case_winner_recalc_conflict(r, variant):
    """Winner-recalc only (:520-560): the best edge's child already carries a claim, so the claim is released and the
    edges are scored once more without it; the runner-up is claimed and kept even if it carries claims too.  With a
    single expanded edge, or when no other edge leads anywhere, the first winner is kept."""
    if variant != "winner_recalc":
        return
    c = _three_children()
    c["edge_n"][0, 0, :3] = 5
    c["edge_prior"][0, 0, :3] = (0.9, 0.05, 0.3)
    c["node_inflight"][0, 1] = 1                 # edge 0 still scores best with one virtual visit
    assert score(1, 0.9, 0, 5, 1, 16) > score(1, 0.3, 0, 5, 0, 16)
    h = r.select(c, variant, c_pw=0.0)
    assert h["out_path"][0, 0, 0] == 2 and h["node_inflight"][0, 1] == 1 and h["node_inflight"][0, 3] == 1
    c["node_inflight"][0, 3] = 4                 # the runner-up carries claims as well: it is kept all the same
    h = r.select(c, variant, c_pw=0.0)
    assert score(1, 0.3, 0, 5, 4, 20) > score(1, 0.05, 0, 5, 0, 20)
    assert h["out_path"][0, 0, 0] == 2 and h["node_inflight"][0, 3] == 5 and h["node_inflight"][0, 1] == 1
    c["edge_child"][0, 0, 1:3] = -1              # no other edge leads anywhere: back to the first winner
    c["node_inflight"][0, 3] = 0
    h = r.select(c, variant, c_pw=0.0)
    assert h["out_path"][0, 0, 0] == 0 and h["node_inflight"][0, 1] == 2
    one = make_case(nodes=2, actions=4, path_depth=2)      # a single expanded edge is taken whatever it carries
    one["node_expanded"][0, 0] = 1
    one["node_expanded"][0, 1] = TERMINAL
    one["edge_child"][0, 0, 0] = 1
    one["edge_n"][0, 0, 0] = 3
    one["node_inflight"][0, 1] = 7
    h = r.select(one, variant, c_pw=0.0)
    assert decode(h["out_selected"][0, 0]) == (TERMINAL_KIND, 0, 1) and h["node_inflight"][0, 1] == 8
    bad = _three_children()                                # a negative counter cannot be claimed (:329-331)
    bad["edge_n"][0, 0, :3] = 1
    bad["edge_prior"][0, 0, 0] = 5.0
    bad["node_inflight"][0, 1] = -1
    h = r.select(bad, variant, c_pw=0.0)
    assert h["out_selected"][0, 0] == PACKED_INVALID and h["node_inflight"][0, 1] == -1 and int(h["node_inflight"].sum()) == -1


def case_fresh_node_quota(r, variant):
    """A node without children: the preclaim kernel allows exactly one child (:640), the winner-recalc kernel what the
    widening formula gives for a count of one, ceil(c_pw) (:775)."""
    c = make_case(nodes=2, actions=8, warps=4, path_depth=2)
    h = r.select(c, variant, c_pw=3.0)
    kinds = [decode(x)[0] for x in h["out_selected"][0]]
    slots = sorted(decode(x)[1] for x in h["out_selected"][0] if decode(x)[0] == EXPAND)
    want = 1 if variant == "preclaim" else 3
    assert kinds.count(EXPAND) == want and slots == list(range(want)) and kinds.count(INVALID) == 4 - want
    assert h["node_expand_inflight"][0, 0] == want
    assert inflight_sum(r.backup(zeros_like_path(h))) == 0


def case_wide_node_beyond_one_wavefront(r, variant):
    c = make_case(nodes=202, actions=256, path_depth=2)
    c["node_expanded"][0, 0] = 200
    c["node_expanded"][0, 1:] = TERMINAL
    c["edge_child"][0, 0, :200] = np.arange(1, 201)
    c["edge_n"][0, 0, :200] = 3
    c["edge_prior"][0, 0, :200] = 0.5
    c["edge_prior"][0, 0, 150] = 0.6
    c["node_inflight"][0, 100] = 1
    h = r.select(c, variant, c_pw=0.0)
    assert decode(h["out_selected"][0, 0]) == (TERMINAL_KIND, 0, 151) and h["out_path"][0, 0, 0] == 150
    assert int(h["node_inflight"].sum()) == 2 and h["node_inflight"][0, 151] == 1


def case_nan_and_minus_inf_never_win(r, variant):
    c = _three_children()
    c["edge_n"][0, 0, :3] = 2
    c["edge_w"][0, 0, :3] = (np.nan, -np.inf, -8.0)
    h = r.select(c, variant, c_pw=0.0)
    assert h["out_path"][0, 0, 0] == 2
    c["edge_w"][0, 0, 2] = np.nan
    h = r.select(c, variant, c_pw=0.0)
    assert h["out_selected"][0, 0] == PACKED_INVALID and inflight_sum(h) == 0


def case_deep_chain(r, variant):
    """100 levels of single children: every child on the way carries one claim at the terminal end; with an inconsistent
    node word at the end instead, all of them are given back (:291-310)."""
    c = make_case(nodes=101, actions=2, path_depth=128)
    c["node_expanded"][0, :100] = 1
    c["edge_child"][0, np.arange(100), 0] = np.arange(1, 101)
    c["edge_n"][0, :100, 0] = 1
    c["node_expanded"][0, 100] = TERMINAL
    h = r.select(c, variant, c_pw=0.0)
    assert decode(h["out_selected"][0, 0]) == (TERMINAL_KIND, 0, 100) and h["out_len"][0, 0] == 101
    assert np.array_equal(h["out_path"][0, 0, :100], np.arange(100) << 8)
    assert np.array_equal(h["node_inflight"][0], np.r_[0, np.ones(100, np.int32)])
    values = zeros_like_path(h)
    values[0, 0, :100] = 0.25
    h2 = r.backup(values)
    assert inflight_sum(h2) == 0 and np.all(h2["edge_n"][0, :100, 0] == 2) and np.all(h2["edge_w"][0, :100, 0] == 0.25)
    c["node_expanded"][0, 100] = -7
    h = r.select(c, variant, c_pw=0.0)
    assert h["out_selected"][0, 0] == PACKED_INVALID and h["out_len"][0, 0] == 0 and inflight_sum(h) == 0


REFERENCE_CASES = [case_fresh_root_expand_roundtrip, case_terminal_root, case_invalid_child_rolls_back,
                   case_child_beyond_node_count, case_progressive_widening_unique_slots,
                   case_fully_expanded_select_and_backup, case_depth_limit, case_encoding_boundaries]
ARITHMETIC_CASES = [case_hand_computed_scores, case_edges_that_lead_nowhere_are_no_candidates, case_ties,
                    case_ties_across_slices_and_around, case_preclaim_rotation_by_wid, case_winner_recalc_conflict, case_fresh_node_quota,
                    case_wide_node_beyond_one_wavefront, case_nan_and_minus_inf_never_win, case_deep_chain]
ALL_CASES = REFERENCE_CASES + ARITHMETIC_CASES


def random_forest(rng, trees, nodes, actions, warps, path_depth, broken_edges=0.05):
    """puct_cases.random_forest with node-level counters and a share of expanded edges that lead nowhere."""
    c = pc.random_forest(rng, trees, nodes, actions, warps, path_depth)
    del c["edge_inflight"]
    c["node_inflight"] = np.zeros((trees, nodes), np.int32)
    expanded = np.arange(actions)[None, None, :] < np.maximum(c["node_expanded"], 0)[:, :, None]
    broken = expanded & (rng.random(c["edge_child"].shape) < broken_edges)
    c["edge_child"][broken] = -1
    return c


def wide_forest(rng, trees, nodes, actions, warps, path_depth, hubs=2, visits=0.05, broken_edges=0.03):
    """puct_cases.wide_forest with node-level counters: a share `visits` of the nodes already carries one to three
    virtual visits, and a share of the expanded edges leads nowhere."""
    c = pc.wide_forest(rng, trees, nodes, actions, warps, path_depth, hubs=hubs, claims=0.0)
    del c["edge_inflight"]
    c["node_inflight"] = np.zeros((trees, nodes), np.int32)
    if visits:
        held = rng.random(c["node_inflight"].shape) < visits
        c["node_inflight"][held] = rng.integers(1, 4, int(held.sum()))
    expanded = np.arange(actions)[None, None, :] < np.maximum(c["node_expanded"], 0)[:, :, None]
    broken = expanded & (rng.random(c["edge_child"].shape) < broken_edges)
    c["edge_child"][broken] = -1
    return c
