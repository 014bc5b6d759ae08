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
