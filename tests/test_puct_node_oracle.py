"""The sequential oracle of PUCT selection with node-level virtual loss (src/puct/puct_gpu_v2.py:573-840) against the
reference's known answers, hand-computed scores and the conservation laws of select + backup."""
import copy

import numpy as np
import pytest

import puct_node_cases as nc
from oracle import puct_oracle as po


class OracleRunner(nc.Runner):
    sequential = True

    def select(self, case, variant, **params):
        self.h = copy.deepcopy(case)
        return copy.deepcopy(po.node_select(self.h, variant=variant, **params))

    def backup(self, values):
        return copy.deepcopy(po.backup(self.h, values, node_level=True))


@pytest.mark.parametrize("variant", nc.VARIANTS)
@pytest.mark.parametrize("case", nc.ALL_CASES, ids=lambda f: f.__name__)
def test_known_answers(case, variant):
    case(OracleRunner(), variant)


@pytest.mark.parametrize("variant", nc.VARIANTS)
def test_select_then_backup_conserves_counts(variant):
    """Every traversal that ends with a selection holds one claim per path edge, on the child the edge leads to, and one
    ticket if it expands; the node-level backup takes all of it back and adds one visit and the value per path edge."""
    rng = np.random.default_rng(5)
    h = nc.random_forest(rng, trees=8, nodes=200, actions=6, warps=8, path_depth=16)
    n_before, w_before = h["edge_n"].copy(), h["edge_w"].copy()
    po.node_select(h, cpuct=1.5, c_pw=1.0, variant=variant)
    assert nc.inflight_nonnegative(h)
    kinds = h["out_selected"] >> 22
    holding = kinds != nc.INVALID
    assert np.any(holding) and np.all(h["out_len"][~holding] == 0)
    assert int(h["node_inflight"].sum()) == int((h["out_len"][holding] - 1).sum())
    assert int(h["node_expand_inflight"].sum()) == int((kinds == nc.EXPAND).sum())
    # the claims sit on the nodes the paths pass through
    want = np.zeros_like(h["node_inflight"])
    for t, w in zip(*np.nonzero(holding)):
        node = 0
        for d in range(h["out_len"][t, w] - 1):
            enc = int(h["out_path"][t, w, d])
            assert enc >> 8 == node
            node = int(h["edge_child"][t, node, enc & 0xFF])
            want[t, node] += 1
        assert node == nc.decode(h["out_selected"][t, w])[2]
    assert np.array_equal(want, h["node_inflight"])
    values = np.full(h["out_path"].shape, 0.25, np.float32)
    po.backup(h, values, node_level=True)
    assert nc.inflight_sum(h) == 0
    added = h["edge_n"] - n_before
    assert int(added.sum()) == int((h["out_len"][holding] - 1).sum())
    assert np.allclose(h["edge_w"] - w_before, 0.25 * added, atol=1e-4)


def test_variants_agree_without_contention_and_ties():
    """With one traversal per tree, distinct scores and no claims in flight the two kernels are the same function."""
    rng = np.random.default_rng(9)
    a = nc.random_forest(rng, trees=32, nodes=300, actions=8, warps=1, path_depth=12)
    b = copy.deepcopy(a)
    po.node_select(a, cpuct=1.3, c_pw=0.8, variant="preclaim")
    po.node_select(b, cpuct=1.3, c_pw=0.8, variant="winner_recalc")
    for k in a:
        assert np.array_equal(a[k], b[k]), k
