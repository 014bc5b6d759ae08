"""PUCT select / backup through the C ABI of libpuct_hip.so on the GPU: the reference's known answers, bit-exact
agreement with the sequential oracle wherever a launch is deterministic (one traversal per tree), and the invariants
every interleaving satisfies where it is not."""
import copy

import numpy as np
import pytest

import puct_cases as pc
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


class HipRunner(pc.Runner):
    def select(self, case, **params):
        from mcts_numba_cuda_amd import puct
        self.d = to_device(case)
        puct.launch_select(self.d, **params)
        synchronize()
        return to_host(self.d)

    def release(self):
        return self.backup(None)

    def backup(self, values):
        from mcts_numba_cuda_amd import puct
        from mcts_numba_cuda_amd.hipmem import DeviceArray
        puct.launch_edge_backup(self.d, None if values is None else DeviceArray(values))
        synchronize()
        return to_host(self.d)


@pytest.mark.parametrize("case", pc.ALL_CASES, ids=lambda f: f.__name__)
def test_known_answers(case):
    case(HipRunner())


@pytest.mark.parametrize("actions,nodes,depth,cpuct,c_pw", [(6, 300, 16, 1.5, 1.0), (225, 2000, 8, 1.5, 0.0),
                                                            (256, 600, 4, 0.7, 2.0), (3, 4000, 64, 1.0, 0.5),
                                                            (8, 1024, 24, 1.2, 1.0), (8, 1025, 24, 1.2, 1.0)])
def test_single_traversal_matches_oracle_exactly(actions, nodes, depth, cpuct, c_pw):
    """One traversal per tree is deterministic: every array must equal the oracle's, over several select/backup
    rounds on the same trees (the statistics drift apart as soon as one score comparison differs).  (Up to 8192 edge
    slots per tree the kernel keeps a tree's claims in LDS during a launch, beyond that in device memory: the last two
    cases sit on either side.)"""
    rng = np.random.default_rng(actions * 1000 + nodes)
    case = pc.random_forest(rng, trees=64, nodes=nodes, actions=actions, warps=1, path_depth=depth)
    h = copy.deepcopy(case)
    r = HipRunner()
    for rnd in range(6):
        got = r.select(case if rnd == 0 else to_host(r.d), cpuct=cpuct, c_pw=c_pw)
        po.select(h, cpuct=cpuct, c_pw=c_pw)
        for k in h:
            assert np.array_equal(got[k], h[k], equal_nan=True), (rnd, k)
        values = rng.uniform(-1, 1, h["out_path"].shape).astype(np.float32)
        got = r.backup(values)
        po.backup(h, values)
        for k in h:
            assert np.array_equal(got[k], h[k], equal_nan=True), (rnd, k)
        assert pc.inflight_sum(got) == 0


@pytest.mark.parametrize("actions,nodes,hubs,claims,cpuct,c_pw,soft", [(256, 1200, 2, 0.05, 1.5, 0.0, 0), (193, 1200, 4, 0.3, 1.0, 16.0, 1),
                                                                      (129, 300, 1, 0.3, 0.5, 0.0, 0), (65, 300, 8, 0.05, 4.0, 2.0, 1),
                                                                      (225, 40, 1, 0.0, 0.0, 100.0, 0)])
def test_wide_nodes_with_claims_in_flight_match_oracle_exactly(actions, nodes, hubs, claims, cpuct, c_pw, soft):
    """As above on trees whose top levels fill two to four 64-edge slices, with random statistics, repeated priors and
    claims already held on some edges (so the scores see virtual loss and a strict claim can find its edge taken)."""
    rng = np.random.default_rng(actions * 1000 + nodes)
    case = pc.wide_forest(rng, trees=32, nodes=nodes, actions=actions, warps=1, path_depth=12, hubs=hubs, claims=claims)
    h = copy.deepcopy(case)
    r = HipRunner()
    for rnd in range(4):
        got = r.select(case if rnd == 0 else to_host(r.d), cpuct=cpuct, c_pw=c_pw, soft_winner=soft)
        po.select(h, cpuct=cpuct, c_pw=c_pw, soft_winner=soft)
        for k in h:
            assert np.array_equal(got[k], h[k], equal_nan=True), (rnd, k)
        values = rng.uniform(-1, 1, h["out_path"].shape).astype(np.float32)
        got = r.backup(values)
        po.backup(h, values)
        for k in h:
            assert np.array_equal(got[k], h[k], equal_nan=True), (rnd, k)


@pytest.mark.parametrize("trees,warps,soft", [(16, 8, 0), (16, 16, 0), (4, 40, 0), (16, 16, 1), (128, 4, 0)])
def test_concurrent_traversals_keep_invariants(trees, warps, soft):
    rng = np.random.default_rng(trees * 100 + warps)
    case = pc.random_forest(rng, trees=trees, nodes=400, actions=16, warps=warps, path_depth=12)
    n_before, w_before = case["edge_n"].copy(), case["edge_w"].copy()
    r = HipRunner()
    h = r.select(case, cpuct=1.5, c_pw=1.0, soft_winner=soft)
    assert pc.inflight_nonnegative(h)
    kinds = (h["out_selected"] >> 22) & 7
    assert np.all(np.isin(kinds, (pc.EXPAND, pc.TERMINAL_KIND, pc.DEPTH_LIMIT, pc.BUSY)))
    if soft:
        assert not np.any((kinds == pc.BUSY) & (((h["out_selected"] >> 25) & 0x3F) == 5))
    holding = (kinds != pc.BUSY)
    assert np.any(holding)
    assert np.all(h["out_len"][~holding] == 0)
    assert int(h["edge_inflight"].sum()) == int((h["out_len"][holding] - 1).sum())
    assert int(h["node_expand_inflight"].sum()) == int((kinds == pc.EXPAND).sum())
    # expansion slots of one node are distinct and start at its current child count
    for t in range(trees):
        seen = set()
        for w in range(warps):
            k, slot, node = pc.decode(h["out_selected"][t, w])
            if k == pc.EXPAND:
                assert (node, slot) not in seen and slot >= h["node_expanded"][t, node]
                seen.add((node, slot))
    # every recorded path is a chain of existing edges from the root to the selected node
    for t in range(trees):
        for w in range(warps):
            if not holding[t, w]:
                continue
            node = 0
            for dd in range(h["out_len"][t, w] - 1):
                enc = int(h["out_path"][t, w, dd])
                assert enc >> 8 == node and (enc & 0xFF) < h["node_expanded"][t, node]
                node = int(h["edge_child"][t, node, enc & 0xFF])
            assert node == pc.decode(h["out_selected"][t, w])[2]
    values = np.full(h["out_path"].shape, 0.5, np.float32)
    h2 = r.backup(values)
    assert pc.inflight_sum(h2) == 0 and pc.inflight_nonnegative(h2)
    added = h2["edge_n"] - n_before
    assert int(added.sum()) == int((h["out_len"][holding] - 1).sum())
    assert np.allclose(h2["edge_w"] - w_before, 0.5 * added, atol=1e-3)


def test_node_level_backup_known_answer():
    """src/puct/test_puct_gpu_v2.py:1085-1119 through puct_node_backup_launch."""
    from mcts_numba_cuda_amd import puct
    from mcts_numba_cuda_amd.hipmem import DeviceArray
    h = pc.make_case(nodes=3, actions=4, path_depth=4)
    h["edge_child"][0, 0, :2] = (1, 2)
    h["edge_n"][0, 0, :2] = 1
    h["node_inflight"] = np.zeros((1, 3), np.int32)
    h["node_inflight"][0, 2] = 1
    h["node_expand_inflight"][0, 2] = 1
    h["out_selected"][0, 0] = (pc.EXPAND << 22) | 2
    h["out_path"][0, 0, 0] = 1
    h["out_len"][0, 0] = 2
    values = np.zeros((1, 1, 4), np.float32)
    values[0, 0, 0] = 0.7
    d = to_device(h)
    puct.launch_node_backup(d, DeviceArray(values))
    synchronize()
    g = to_host(d)
    assert int(g["node_inflight"].sum()) == 0 and int(g["node_expand_inflight"].sum()) == 0
    assert g["edge_n"][0, 0, 1] == 2 and g["edge_w"][0, 0, 1] == np.float32(0.7)
    ref = copy.deepcopy(h)
    po.backup(ref, values, node_level=True)
    for k in ref:
        assert np.array_equal(g[k], ref[k]), k


def test_launch_errors_are_reported():
    from mcts_numba_cuda_amd import puct
    from mcts_numba_cuda_amd.hipmem import DeviceArray
    case = pc.make_case(nodes=2, actions=4, warps=1, path_depth=2)
    d = to_device(case)
    d["edge_prior"] = DeviceArray(case["edge_prior"].astype(np.float64))
    with pytest.raises(ValueError):
        puct.launch_select(d)
    d = to_device(case)
    d["out_selected"] = DeviceArray(np.zeros((1, 0), np.int32))
    d["out_len"] = DeviceArray(np.zeros((1, 0), np.int32))
    d["out_path"] = DeviceArray(np.zeros((1, 0, 2), np.int32))
    with pytest.raises(RuntimeError, match="launch failed"):
        puct.launch_select(d)           # zero traversals: the runtime rejects the empty launch, as CUDA does
    assert isinstance(puct._lib().puct_cpp_cuda_error_string(0), bytes)
