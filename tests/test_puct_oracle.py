"""The sequential PUCT oracle against the reference's known answers and against what the arithmetic fixes."""
import copy

import numpy as np
import pytest

import puct_cases as pc
from oracle import puct_oracle as po


class OracleRunner(pc.Runner):
    def select(self, case, **params):
        self.h = copy.deepcopy(case)
        return copy.deepcopy(po.select(self.h, **params))

    def release(self):
        return copy.deepcopy(po.backup(self.h, None))

    def backup(self, values):
        return copy.deepcopy(po.backup(self.h, values))


@pytest.mark.parametrize("case", pc.ALL_CASES, ids=lambda f: f.__name__)
def test_known_answers(case):
    case(OracleRunner())


def test_select_then_backup_conserves_counts():
    rng = np.random.default_rng(3)
    h = pc.random_forest(rng, trees=8, nodes=200, actions=6, warps=8, path_depth=16)
    n_before, w_before = h["edge_n"].copy(), h["edge_w"].copy()
    po.select(h, cpuct=1.5, c_pw=1.0)
    assert pc.inflight_nonnegative(h)
    kinds = (h["out_selected"] >> 22) & 7
    holding = (kinds != pc.INVALID) & (kinds != pc.BUSY)
    # every holding traversal has one claim per path edge, and one ticket if it expands
    assert int(h["edge_inflight"].sum()) == int((h["out_len"][holding] - 1).sum())
    assert int(h["node_expand_inflight"].sum()) == int((kinds == pc.EXPAND).sum())
    values = np.full(h["out_path"].shape, 0.25, np.float32)
    po.backup(h, values)
    assert pc.inflight_sum(h) == 0
    added = h["edge_n"] - n_before
    assert int(added.sum()) == int((h["out_len"][holding] - 1).sum())
    assert np.allclose(h["edge_w"] - w_before, 0.25 * added, atol=1e-4)


def test_node_level_backup_matches_v2_known_answer():
    """src/puct/test_puct_gpu_v2.py:1085-1119: a path through edge (0, 1) into child 2, which holds one virtual visit
    and one expansion ticket; after backup with value 0.7 both are gone, edge_n is 2 and edge_w is 0.7."""
    h = pc.make_case(nodes=3, actions=4, path_depth=4)
    h["edge_child"][0, 0, :2] = (1, 2)
    h["edge_n"][0, 0, :2] = 1
    h["node_inflight"] = np.zeros((1, 3), np.int32)
    h["node_inflight"][0, 2] = 1
    h["node_expand_inflight"][0, 2] = 1
    h["out_selected"][0, 0] = (pc.EXPAND << 22) | 2        # v2 layout: no reason field
    h["out_path"][0, 0, 0] = 1
    h["out_len"][0, 0] = 2
    values = np.zeros((1, 1, 4), np.float32)
    values[0, 0, 0] = 0.7
    po.backup(h, values, node_level=True)
    assert int(h["node_inflight"].sum()) == 0 and int(h["node_expand_inflight"].sum()) == 0
    assert h["edge_n"][0, 0, 1] == 2 and h["edge_w"][0, 0, 1] == np.float32(0.7)


# ---- Gomoku PUCT loop: the evaluator and the sequential search -------------------------------------------------------
import math

import puct_gomoku_checks as gc


def test_single_precision_log_and_exp_within_two_ulp_of_libm():
    """The evaluator's branch-free float32 log (positive normal arguments) and exp (arguments <= 0, zero below -86)
    against numpy's, which are correctly rounded to well below an ulp."""
    ev = po.evaluator()
    rng = np.random.default_rng(0)
    xs = np.concatenate([rng.uniform(0, 1, 20000), np.exp(rng.uniform(-87, 88, 20000)), [1.0, 0.5, 2.0, 1.17549435e-38, 3.4e38,
                         0.70710677, 0.70710683, 1.4142135, 1.4142137]]).astype(np.float32)
    for x in xs:
        got, want = np.float32(ev.po_det_logf(float(x))), np.log(np.float64(x))
        assert abs(np.float64(got) - want) <= 2 * np.spacing(np.float32(abs(want))), x
    assert ev.po_det_logf(1.0) == 0.0
    xs = np.concatenate([-rng.uniform(0, 86, 20000), -rng.uniform(0, 2, 20000), [0.0, -0.0, -1e-10, -0.3465735, -0.3465737, -1.0397, -86.0]]).astype(np.float32)
    for x in xs:
        got, want = np.float32(ev.po_det_expf(float(x))), np.exp(np.float64(x))
        assert abs(np.float64(got) - want) <= 2 * np.spacing(np.float32(want)), x
    assert ev.po_det_expf(0.0) == 1.0 and ev.po_det_expf(-86.5) == 0.0 and ev.po_det_expf(-1000.0) == 0.0


def test_gamma_variates_have_gamma_moments():
    ev = po.evaluator()
    for alpha in (0.3, 0.7):
        g = np.array([ev.po_gamma(alpha, k * 0x9E3779B97F4A7C15 % 2**64) for k in range(200000)])
        assert np.all(g >= 0)
        assert abs(g.mean() - alpha) < 0.01 and abs(g.var() - alpha) < 0.03      # Gamma(alpha, 1): mean = var = alpha
        # third central moment of Gamma(alpha, 1) is 2 alpha
        assert abs(((g - g.mean()) ** 3).mean() - 2 * alpha) < 0.15


def test_root_priors_have_dirichlet_moments():
    """Priors of the empty 15x15 board over 64 trees (64 different evaluators): a permutation of the cells in
    descending order, summing to one, with the marginal variance of Dirichlet(0.3, ..., 0.3)."""
    board = np.zeros((15, 15), np.int8)
    h = po.gomoku_search(board, 1, 0, trees=64, traversals=1, max_nodes=2)
    pri = h["edge_prior"][:, 0, :225].astype(np.float64)
    acts = h["edge_action"][:, 0, :225]
    assert np.all(np.sort(acts, axis=1) == np.arange(225))
    assert np.all(np.diff(pri, axis=1) <= 0) and np.allclose(pri.sum(axis=1), 1.0, atol=1e-5)
    n, alpha = 225, 0.3
    want_var = (1 / n) * (1 - 1 / n) / (n * alpha + 1)
    assert abs(pri.var() / want_var - 1.0) < 0.15          # 14400 samples of a heavy-tailed marginal
    by_cell = np.zeros((64, 225))
    np.put_along_axis(by_cell, acts.astype(int), pri, axis=1)
    assert abs(by_cell.mean(axis=0).mean() - 1 / n) < 1e-9 and by_cell.mean(axis=0).max() < 5 / n   # no favoured cell


def test_exactly_five_rule_against_brute_force():
    ev = po.evaluator()
    rng = np.random.default_rng(2)
    hits = 0
    for _ in range(3000):
        m, n = int(rng.integers(5, 16)), int(rng.integers(5, 17))
        if m * n > 256:
            continue
        stones = rng.random(m * n) < 0.55
        cell = int(rng.integers(0, m * n))
        stones[cell] = True
        words = np.zeros(8, np.uint32)
        for c in np.flatnonzero(stones):
            words[c >> 5] |= np.uint32(1 << (c & 31))
        want = 5 in gc.run_through(stones, m, n, cell)
        hits += want
        assert bool(ev.po_makes_five(words.ctypes.data, cell, m, n)) == want
    assert hits > 100


@pytest.mark.parametrize("shape,stones,traversals,steps,max_nodes,depth", [
    ((15, 15), 0, 1, 300, 4096, 64), ((15, 15), 12, 4, 150, 4096, 64), ((6, 6), 4, 2, 400, 4096, 64),
    ((5, 5), 18, 3, 200, 2048, 64), ((9, 9), 0, 8, 120, 300, 64), ((7, 7), 0, 2, 300, 4096, 3)])
def test_sequential_search_builds_consistent_trees(shape, stones, traversals, steps, max_nodes, depth):
    from helpers import random_gomoku_root
    rng = np.random.default_rng(shape[0] * 100 + stones)
    board, turn = random_gomoku_root(rng, shape[0], shape[1], stones)
    h = po.gomoku_search(board, turn, steps, trees=3, traversals=traversals, max_nodes=max_nodes, path_depth=depth, seed=5)
    gc.check_trees(h, board, turn, shape[0], shape[1], max_nodes, depth)
    tally = h["tally"]
    assert np.all(tally[:, :5].sum(axis=1) == steps * traversals) and np.all(tally[:, 0] == 0)
    assert np.array_equal(tally[:, 5], h["node_count"] - 1)
    # every selection that is not busy adds exactly one visit to one root edge, except an expansion of the root itself
    # that a full tree could not take
    for t in range(3):
        if max_nodes >= 2048:
            assert gc.visits_below(h, t, 0) == int(tally[t, 1:4].sum())
        else:
            assert gc.visits_below(h, t, 0) <= int(tally[t, 1:4].sum())
    if max_nodes >= 2048 and depth >= 64:
        gc.check_visit_flow(h, depth)
    else:
        assert (tally[:, 3].sum() > 0) or np.any(h["node_count"] + traversals > max_nodes)   # the limit was exercised
