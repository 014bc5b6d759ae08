"""PUCT selection with node-level virtual loss (puct_node_select_preclaim_launch, puct_node_select_winner_recalc_launch)
and its backup through the C ABI of libpuct_hip.so on the GPU: the reference's known answers, bit-exact agreement with
the sequential oracle wherever a launch is deterministic (one traversal per tree), and the invariants every interleaving
satisfies where it is not."""
import copy

import numpy as np
import pytest

import puct_node_cases as nc
from oracle import puct_oracle as po

pytestmark = pytest.mark.gpu


def to_device(case):
    from mcts_numba_cuda_amd.hipmem import DeviceArray
    return {k: DeviceArray(v) for k, v in case.items()}


def to_host(d):
    return {k: v.numpy() for k, v in d.items()}


def synchronize():
    from mcts_numba_cuda_amd.hipmem import synchronize as sync
    sync()


class HipRunner(nc.Runner):
    def select(self, case, variant, **params):
        from mcts_numba_cuda_amd import puct
        self.d = to_device(case)
        puct.launch_node_select(self.d, variant=variant, **params)
        synchronize()
        return to_host(self.d)

    def backup(self, values):
        from mcts_numba_cuda_amd import puct
        from mcts_numba_cuda_amd.hipmem import DeviceArray
        puct.launch_node_backup(self.d, DeviceArray(values))
        synchronize()
        return to_host(self.d)


@pytest.mark.parametrize("variant", nc.VARIANTS)
@pytest.mark.parametrize("case", nc.ALL_CASES, ids=lambda f: f.__name__)
def test_known_answers(case, variant):
    case(HipRunner(), variant)


@pytest.mark.parametrize("variant", nc.VARIANTS)
@pytest.mark.parametrize("actions,nodes,depth,cpuct,c_pw", [(6, 300, 16, 1.5, 1.0), (225, 2000, 8, 1.5, 0.0),
                                                            (256, 600, 4, 0.7, 2.0), (3, 4000, 64, 1.0, 0.5),
                                                            (5, 16384, 24, 1.2, 1.0), (5, 16385, 24, 1.2, 1.0)])
def test_single_traversal_matches_oracle_exactly(actions, nodes, depth, cpuct, c_pw, variant):
    """One traversal per tree is deterministic: every array must equal the oracle's, over several select/backup rounds on
    the same trees (the statistics drift apart as soon as one score comparison differs).  In every other round the
    claims of the selection are left in place for the next one, so that the kernels also score against virtual visits.
    (Up to 16384 nodes per tree the kernels keep a tree's virtual-visit counters in LDS during a launch, beyond that in
    device memory: the last two cases sit on either side.)"""
    rng = np.random.default_rng(actions * 1000 + nodes)
    case = nc.random_forest(rng, trees=64, nodes=nodes, actions=actions, warps=1, path_depth=depth)
    h = copy.deepcopy(case)
    r = HipRunner()
    for rnd in range(8):
        got = r.select(case if rnd == 0 else to_host(r.d), variant, cpuct=cpuct, c_pw=c_pw)
        po.node_select(h, cpuct=cpuct, c_pw=c_pw, variant=variant)
        for k in h:
            assert np.array_equal(got[k], h[k], equal_nan=True), (rnd, k)
        if rnd % 2 == 1:
            continue          # keep this round's claims (expansion tickets included) for the next selection
        values = rng.uniform(-1, 1, h["out_path"].shape).astype(np.float32)
        got = r.backup(values)
        po.backup(h, values, node_level=True)
        for k in h:
            assert np.array_equal(got[k], h[k], equal_nan=True), (rnd, k)


@pytest.mark.parametrize("variant", nc.VARIANTS)
@pytest.mark.parametrize("actions,nodes,hubs,visits,cpuct,c_pw", [(256, 1200, 2, 0.05, 1.5, 0.0), (193, 1200, 4, 0.3, 1.0, 16.0),
                                                                 (129, 300, 1, 0.3, 0.5, 0.0), (65, 300, 8, 0.05, 4.0, 2.0),
                                                                 (225, 40, 1, 0.0, 0.0, 100.0)])
def test_wide_nodes_with_virtual_visits_match_oracle_exactly(actions, nodes, hubs, visits, cpuct, c_pw, variant):
    """As above on trees whose top levels fill two to four 64-edge slices, with random statistics, repeated priors,
    virtual visits already on some nodes and some expanded edges that lead nowhere."""
    rng = np.random.default_rng(actions * 1000 + nodes)
    case = nc.wide_forest(rng, trees=32, nodes=nodes, actions=actions, warps=1, path_depth=12, hubs=hubs, visits=visits)
    h = copy.deepcopy(case)
    r = HipRunner()
    for rnd in range(4):
        got = r.select(case if rnd == 0 else to_host(r.d), variant, cpuct=cpuct, c_pw=c_pw)
        po.node_select(h, cpuct=cpuct, c_pw=c_pw, variant=variant)
        for k in h:
            assert np.array_equal(got[k], h[k], equal_nan=True), (rnd, k)
        values = rng.uniform(-1, 1, h["out_path"].shape).astype(np.float32)
        got = r.backup(values)
        po.backup(h, values, node_level=True)
        for k in h:
            assert np.array_equal(got[k], h[k], equal_nan=True), (rnd, k)


@pytest.mark.parametrize("variant", nc.VARIANTS)
@pytest.mark.parametrize("trees,warps", [(16, 8), (16, 16), (4, 40), (128, 4)])
def test_concurrent_traversals_keep_invariants(trees, warps, variant):
    rng = np.random.default_rng(trees * 100 + warps)
    case = nc.random_forest(rng, trees=trees, nodes=400, actions=16, warps=warps, path_depth=12)
    n_before, w_before = case["edge_n"].copy(), case["edge_w"].copy()
    r = HipRunner()
    h = r.select(case, variant, cpuct=1.5, c_pw=1.0)
    assert nc.inflight_nonnegative(h)
    kinds = h["out_selected"] >> 22
    assert np.all(np.isin(kinds, (nc.INVALID, nc.EXPAND, nc.TERMINAL_KIND, nc.DEPTH_LIMIT)))
    holding = kinds != nc.INVALID
    assert np.any(holding)
    assert np.all(h["out_len"][~holding] == 0) and np.all(h["out_selected"][~holding] == nc.PACKED_INVALID)
    assert int(h["node_expand_inflight"].sum()) == int((kinds == nc.EXPAND).sum())
    # expansion slots of one node are distinct and start at its current child count
    for t in range(trees):
        seen = set()
        for w in range(warps):
            k, slot, node = nc.decode(h["out_selected"][t, w])
            if k == nc.EXPAND:
                assert (node, slot) not in seen and slot >= h["node_expanded"][t, node]
                seen.add((node, slot))
    # every recorded path is a chain of existing edges from the root to the selected node, and the claims that are left
    # are exactly one per path edge, on the node the edge leads to (every passing claim of a preclaim was given back)
    want = np.zeros_like(h["node_inflight"])
    for t, w in zip(*np.nonzero(holding)):
        node = 0
        for dd in range(h["out_len"][t, w] - 1):
            enc = int(h["out_path"][t, w, dd])
            assert enc >> 8 == node and (enc & 0xFF) < h["node_expanded"][t, node]
            node = int(h["edge_child"][t, node, enc & 0xFF])
            assert 0 <= node < h["node_count"][t]
            want[t, node] += 1
        assert node == nc.decode(h["out_selected"][t, w])[2]
    assert np.array_equal(want, h["node_inflight"])
    values = np.full(h["out_path"].shape, 0.5, np.float32)
    h2 = r.backup(values)
    assert nc.inflight_sum(h2) == 0 and nc.inflight_nonnegative(h2)
    added = h2["edge_n"] - n_before
    assert int(added.sum()) == int((h["out_len"][holding] - 1).sum())
    assert np.allclose(h2["edge_w"] - w_before, 0.5 * added, atol=1e-3)


@pytest.mark.parametrize("variant", nc.VARIANTS)
def test_deep_wide_shape_of_the_reference_benchmark(variant):
    """The reference's large-scale select benchmark at a size that runs in a moment (src/puct/test_puct_gpu_v2.py:
    1802-1915, shape "wide" of :109-143): every node has `actions` children on the same `actions` nodes, equal priors,
    c_pw = 0, eight traversals per tree walk `depth` levels to the depth limit; its own criterion: full-length paths,
    some valid selections, nothing in flight after the backup."""
    trees, actions, depth, warps = 64, 64, 128, 8
    c = nc.make_case(trees=trees, nodes=actions + 1, actions=actions, warps=warps, path_depth=depth)
    c["node_expanded"][:] = actions
    c["edge_child"][:] = np.arange(1, actions + 1, dtype=np.int32)
    c["edge_n"][:] = 1
    r = HipRunner()
    h = r.select(c, variant, cpuct=1.0, c_pw=0.0)
    kinds = h["out_selected"] >> 22
    assert np.all(kinds == nc.DEPTH_LIMIT) and np.all(h["out_len"] == depth + 1)
    assert int(h["node_inflight"].sum()) == trees * warps * depth and nc.inflight_nonnegative(h)
    h2 = r.backup(nc.zeros_like_path(h))
    assert nc.inflight_sum(h2) == 0 and int(h2["edge_n"].sum()) == int(c["edge_n"].sum()) + trees * warps * depth


def test_launch_errors_are_reported():
    from mcts_numba_cuda_amd import puct
    from mcts_numba_cuda_amd.hipmem import DeviceArray
    case = nc.make_case(nodes=2, actions=4, warps=1, path_depth=2)
    d = to_device(case)
    with pytest.raises(ValueError, match="variant"):
        puct.launch_node_select(d, variant="native")
    d["node_inflight"] = DeviceArray(case["node_inflight"].astype(np.int64))
    with pytest.raises(ValueError):
        puct.launch_node_select(d)
