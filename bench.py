#!/usr/bin/env python3
"""Benchmark of the MCTS-NC search hot path on one MI355X.

Workload (the headline configuration): Connect 4 6x7, 64 seeded roots each reached by 10..20 uniform-random legal
plies (non-terminal), acp_prodigal, n_trees=4, n_playouts=256, ucb_c=2.0, search_steps_limit=5000,
device_memory=2 GiB, seed 0, random streams restarted for every root.

One bench "step" = one complete search (5000 MCTS steps) of one root through MCTSNC.run(), i.e. the drop-in call the
reference's game_runner makes.  `value` = playouts per second over the timed searches (root visit totals / wall time
of run()), with the engine's pools already resident in HBM.  Extra fields: mcts_steps_per_s, the same workload
batched (all roots concurrently, one device pass) and the per-stage device times.

roofline: the dominant kernel is the persistent search kernel; `achieved` = algorithmic bytes (element sizes of the
reference's arrays: selection gathers, expansion, RNG state traffic of the playouts, backup) divided by the kernel's
duration measured with HIP events on the engine's stream.
cpu_baseline: the CPU oracle (a scalar restatement of the same algorithm, OpenMP over playouts) timed on this host on
a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

M, N, A = 6, 7, 7
T, P, STEPS, DEVICE_MEMORY = 4, 256, 5000, 2.0
N_ROOTS = 64
HBM_PEAK_GBS = 8000.0
# Vector ALU peak of the device in wavefront instructions per second: 256 CUs x 4 SIMDs, each issuing one 64-lane
# instruction per 4 clocks at 2.4 GHz.
SIMDS, CLOCK_HZ = 1024, 2.4e9
VALU_PEAK_G = SIMDS * CLOCK_HZ / 4 / 1e9
PROFILES = os.path.join(ROOT, "profiles")


def profile_json(name):
    """The machine-readable block (first ```json fence) of a counter summary under profiles/, or None.  The summaries
    are written from rocprofv3 --pmc runs of this script; each names the commit it was taken at."""
    path = os.path.join(PROFILES, name)
    if not os.path.exists(path):
        return None
    text = open(path).read()
    start = text.find("```json")
    if start < 0:
        return None
    end = text.find("```", start + 7)
    try:
        d = json.loads(text[start + 7:end])
    except ValueError:
        return None
    d["file"] = "profiles/" + name
    # A summary that records the hashes of its kernel's source files can say whether they have changed since the counters
    # were taken (None: the summary holds no hashes).
    d["stale"] = None
    if isinstance(d.get("kernel_sources"), dict):
        d["stale"] = any(source_hash(path) != h for path, h in d["kernel_sources"].items())
    return d


PLAIN_LAUNCH = False


def apply_launch_options(engine):
    """--plain-launch: the all-children kernels as ordinary launches (profilers and the runtime's cooperative queue do not
    get along: a rocprofv3 process that has made a cooperative launch ends with SIGSEGV in the runtime's exit handler)."""
    if PLAIN_LAUNCH:
        engine.set_option("plain_launch", 1)


def source_hash(path):
    import hashlib
    try:
        return hashlib.sha256(open(os.path.join(ROOT, path), "rb").read()).hexdigest()[:16]
    except OSError:
        return None


def valu_roofline(insts, seconds, source, what):
    """Vector-ALU side of the roofline: SQ_INSTS_VALU (wavefront instructions, from the named counter summary) over the
    kernel time measured in this run, against the device's issue peak."""
    if not insts or not seconds:
        return None
    achieved = insts / seconds / 1e9
    return {"bound": "valu", "achieved": achieved, "peak": VALU_PEAK_G, "unit": "G wavefront instructions/s", "frac": achieved / VALU_PEAK_G,
            "formula": "SQ_INSTS_VALU x 4 / (1024 SIMDs x kernel time x 2.4 GHz)", "what": what,
            "counter_file": source.get("file"), "counter_commit": source.get("commit"),
            # the instruction count comes from the counter summary, the time from this run: true if the kernel's sources
            # have changed since the counters were taken, None if the summary does not record their hashes
            "stale": source.get("stale")}


def has_four(board, token):
    for i in range(M):
        for j in range(N):
            for di, dj in ((0, 1), (1, 0), (1, 1), (1, -1)):
                if all(0 <= i + di * k < M and 0 <= j + dj * k < N and board[i + di * k, j + dj * k] == token for k in range(4)):
                    return True
    return False


def make_roots(n_roots, seed=0):
    """Seeded synthetic roots: 10..20 uniform-random legal plies, rejected when the game got decided on the way."""
    rng = np.random.Generator(np.random.PCG64(seed))
    roots = []
    while len(roots) < n_roots:
        plies = int(rng.integers(10, 21))
        board = np.zeros((M, N), np.int8)
        fills = np.zeros(N, np.int8)
        turn, ok = 1, True
        for _ in range(plies):
            legal = np.flatnonzero(fills < M)
            j = int(rng.choice(legal))
            board[M - 1 - fills[j], j] = turn
            fills[j] += 1
            if has_four(board, turn):
                ok = False
                break
            turn = -turn
        if ok and (fills < M).any():
            roots.append((board, fills, turn))
    return roots


def device_synchronize():
    """hipDeviceSynchronize through the HIP runtime the engine library is linked against (MCTSNC.run() itself
    returns only after its stream has drained)."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    rc = hip.hipDeviceSynchronize()
    if rc != 0:
        raise RuntimeError(f"hipDeviceSynchronize failed with {rc}")


def algorithmic_bytes(res, tree_steps, acp=True, mn_e=M * N + A, A=A, P=P):
    """Bytes the reference's arrays would move for the work counted on the device (element sizes of
    src/mctsnc.py:326-348): selection reads per level a leaf flag, the parent's visit count, the child row and the
    children's (ns, ns_wins); expansion reads the selected state and writes k children; each played-out node reads
    its state and reads + writes P generator states; backup updates k children and L + 1 path nodes."""
    levels, children, expanded, played = res.stat_levels, res.stat_children, res.stat_expanded, res.stat_played
    select = levels * (1 + 4 + 4 * A) + 8 * children + tree_steps * (1 + 4) + 4 * (levels + tree_steps)
    expand = tree_steps * (mn_e + 6 + 4 * A + 2 * (A + 2)) + expanded * (mn_e + 18)
    playout = played * (mn_e + 2 + 32 * P + 8)
    backup = (expanded if acp else tree_steps) * (4 + 1 + 8 + 16) + (levels + tree_steps) * (4 + 1 + 8 + 8)
    return dict(select=select, expand=expand, playout=playout, backup=backup, total=select + expand + playout + backup)


# The reference's large-scale selection benchmark (src/puct/test_puct_gpu_v3.py:2069-2160): name -> (trees, edges per
# node, path depth); 8 traversals per tree, "wide" recurrent trees (every node has all its edges expanded, edge a leads
# to node a + 1, equal priors, N = 1, W = 0), no progressive widening, so every selection walks `depth` levels and ends
# at the depth limit.  Published: 1.63 M / 0.64 M / 0.38 M selections/s (winner_recalc, device unstated).
PUCT_SHAPES = {"eq64_d512": (16384, 64, 512), "eq128_d1024": (8192, 128, 1024), "eq256_d1024": (4096, 256, 1024)}
PUCT_TRAVERSALS = 8


def puct_wide_case(trees, actions, depth, warps):
    nodes = actions + 1
    one = {
        "edge_child": np.broadcast_to(np.arange(1, actions + 1, dtype=np.int32), (nodes, actions)),
        "edge_prior": np.ones((nodes, actions), np.float32), "edge_w": np.zeros((nodes, actions), np.float32),
        "edge_n": np.ones((nodes, actions), np.int32), "edge_inflight": np.zeros((nodes, actions), np.int32),
    }
    case = {k: np.ascontiguousarray(np.broadcast_to(v, (trees,) + v.shape)) for k, v in one.items()}
    case.update({
        "node_expand_inflight": np.zeros((trees, nodes), np.int32), "node_expanded": np.full((trees, nodes), actions, np.int32),
        "node_count": np.full((trees,), nodes, np.int32), "out_selected": np.zeros((trees, warps), np.int32),
        "out_path": np.full((trees, warps, depth), -1, np.int32), "out_len": np.zeros((trees, warps), np.int32)})
    return case


def bench_puct_select(args):
    """One bench step = one selection launch over all trees (timed with HIP events on the launch stream), followed by
    an untimed release of the claims, as the reference times it (src/puct/test_puct_gpu_v3.py:632-650)."""
    from mcts_numba_cuda_amd import puct
    from mcts_numba_cuda_amd.hipmem import DeviceArray, Event, synchronize
    trees, actions, depth = PUCT_SHAPES[args.puct_shape]
    warps = PUCT_TRAVERSALS
    steps = args.steps if args.steps != N_ROOTS else 10
    case = puct_wide_case(trees, actions, depth, warps)
    d = {k: DeviceArray(v) for k, v in case.items()}
    def timed(soft):
        for _ in range(max(args.warmup, 1)):
            puct.launch_select(d, cpuct=1.0, c_pw=0.0, soft_winner=soft)
            puct.launch_edge_backup(d)
        synchronize()
        pairs = []
        t0 = time.perf_counter()
        for _ in range(steps):
            a, b = Event(), Event()
            a.record()
            puct.launch_select(d, cpuct=1.0, c_pw=0.0, soft_winner=soft)
            b.record()
            sel, lens = d["out_selected"], d["out_len"]
            puct.launch_edge_backup(d)
            pairs.append((a, b))
        synchronize()
        wall = time.perf_counter() - t0
        ms = sum(a.elapsed_ms(b) for a, b in pairs)
        kinds = (sel.numpy() >> 22) & 7
        lens = lens.numpy()
        # a traversal either reaches the depth limit or gives up busy (the reference's criterion: some valid
        # selections, full-length paths, nothing left in flight after the release;
        # src/puct/test_puct_gpu_v3.py:2141-2150)
        ok = bool(np.all((kinds == 3) | (kinds == 4)) and lens.max() == depth + 1 and np.all(lens[kinds == 3] == depth + 1)
                  and not d["edge_inflight"].numpy().any())
        return ms, wall, ok, float((kinds == 4).mean())

    ms, wall, ok, busy_share = timed(0)
    ms_soft, _, ok_soft, busy_soft = timed(1)
    selections = steps * trees * warps
    # per level: node word, ticket counter, N / W / prior / in-flight of every edge, where the edges lead (the whole
    # child row for nodes of up to 128 edges, else its first 64 words and the winner's) and one path entry.  Exact
    # for the soft-winner run, in which every traversal walks all `depth` levels; with the strict claim a busy traversal
    # stops early, so only the completed ones are counted.
    level_bytes = 8 + 16 * actions + (4 * actions if actions <= 128 else 4 * 64 + 4) + 4
    alg_bytes = int(trees * warps * (1.0 - busy_share)) * depth * level_bytes
    alg_bytes_soft = trees * warps * depth * level_bytes
    cpu = None
    if not args.no_cpu_baseline:
        from oracle import puct_oracle as po
        sample = 64
        h = {k: np.ascontiguousarray(v[:sample]) for k, v in case.items()}
        t1 = time.perf_counter()
        po.select(h, cpuct=1.0, c_pw=0.0)
        dt = time.perf_counter() - t1
        cpu = {"value": sample * warps / dt, "unit": "selections/s", "cores": 1, "kind": "port",
               "sample": f"first {sample} trees of the same workload, one launch ({sample * warps} selections of {depth} levels), "
                         "sequential CPU oracle"}
    prof = profile_json(f"select_kernel_puct_{args.puct_shape}.md")
    launch_s = ms / steps * 1e-3
    traffic = (prof or {}).get("traffic_bytes_per_launch")
    completed = selections * (1.0 - busy_share)     # busy share of the last launch; the launches are alike
    out = {"metric": "PUCT selections/s that complete (reach the depth limit), deep-wide select benchmark of the reference "
                     "(winner_recalc, 8 traversals per tree)",
           "value": completed / (ms * 1e-3), "unit": "selections/s", "n_gpus": 1, "steps": steps, "warmup": max(args.warmup, 1),
           "ms_per_step": ms / steps, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32 scores + int32 atomics",
           "data": "synthetic",
           "config": {"workload": f"{args.puct_shape}: {trees} trees x {warps} traversals, {actions} edges per node, depth {depth}, "
                                  "equal priors, c_pw=0, terminal by depth limit; one puct_select_winner_recalc_launch per step"},
           "valid": ok and ok_soft, "selections_per_s": {"all": selections / (ms * 1e-3), "completed": completed / (ms * 1e-3),
                                                         "busy": selections * busy_share / (ms * 1e-3)},
           "busy_share_last_launch": busy_share, "wall_s_incl_release": wall,
           "soft_winner": {"value": selections / (ms_soft * 1e-3), "unit": "selections/s", "ms_per_step": ms_soft / steps,
                           "busy_share_last_launch": busy_soft, "levels_per_s": selections * depth / (ms_soft * 1e-3),
                           "l2_level_GB_per_s": alg_bytes_soft / (ms_soft / steps * 1e-3) / 1e9,
                           "note": "bytes requested by the traversals; the 8 traversals of a tree read the same rows, so most "
                                   "of them are served by the L2, not by HBM"},
           # The traversals of a tree read the same edge rows, so the bytes they request (the per-traversal algorithmic
           # count) are an L2-level figure; what HBM delivers is what the counters measured, and that is the roofline entry.
           "roofline": {"bound": "hbm", "achieved": traffic / launch_s / 1e9 if traffic else None, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": traffic / launch_s / 1e9 / HBM_PEAK_GBS if traffic else None, "traffic": traffic,
                        "basis": "HBM bytes per launch from the rocprofv3 FETCH_SIZE / WRITE_SIZE summary over this run's launch time",
                        "traffic_source": {"file": prof["file"], "commit": prof.get("commit"), "stale": prof.get("stale")} if prof else None,
                        "kernel": "select_kernel", "avg_launch_ms": ms / steps,
                        "l2_level": {"requested_bytes_per_launch_completed_traversals": alg_bytes,
                                     "requested_GB_per_s": alg_bytes / launch_s / 1e9,
                                     "note": "node word, ticket counter and the 4-byte fields per edge and level that the kernel asks for "
                                             "(N, W, prior, in-flight; the child of every edge up to 128 edges, of the first 64 and "
                                             "the winner beyond), for the traversals that complete; busy ones stop after a third of "
                                             "the levels on average"}},
           "cpu_baseline": cpu}
    print(json.dumps(out))


# published by the reference for its node-level select kernels on this benchmark (8 traversals per tree; hardware not
# stated, its notes mention an RTX 4090): shape -> (preclaim, winner_recalc) selections/s
PUCT_NODE_PUBLISHED = {"eq256_d1024": (242e3, 376e3), "eq128_d1024": (410e3, 641e3), "eq64_d512": (1.21e6, 1.63e6)}


def bench_puct_node_select(args):
    """The reference's large-scale deep-wide select benchmark on its own two kernels with node-level virtual loss
    (src/puct/test_puct_gpu_v2.py:1802-1915): one bench step = one selection launch over all trees, timed with HIP events
    on the launch stream, followed by an untimed node-level backup (path values zero), as the reference times it."""
    from mcts_numba_cuda_amd import puct
    from mcts_numba_cuda_amd.hipmem import DeviceArray, Event, synchronize
    variant = {"node_preclaim": puct.VARIANT_PRECLAIM, "node_winner_recalc": puct.VARIANT_WINNER_RECALC}[args.select_variant]
    trees, actions, depth = PUCT_SHAPES[args.puct_shape]
    warps = PUCT_TRAVERSALS
    steps = args.steps if args.steps != N_ROOTS else 10
    case = puct_wide_case(trees, actions, depth, warps)
    del case["edge_inflight"]
    case["node_inflight"] = np.zeros((trees, actions + 1), np.int32)
    d = {k: DeviceArray(v) for k, v in case.items()}
    values = DeviceArray(np.zeros((trees, warps, depth), np.float32))
    for _ in range(max(args.warmup, 1)):
        puct.launch_node_select(d, cpuct=1.0, c_pw=0.0, variant=variant)
        puct.launch_node_backup(d, values)
    synchronize()
    pairs = []
    for _ in range(steps):
        a, b = Event(), Event()
        a.record()
        puct.launch_node_select(d, cpuct=1.0, c_pw=0.0, variant=variant)
        b.record()
        sel, lens = d["out_selected"], d["out_len"]
        puct.launch_node_backup(d, values)
        pairs.append((a, b))
    synchronize()
    ms = sum(a.elapsed_ms(b) for a, b in pairs)
    kinds = sel.numpy() >> 22
    lens = lens.numpy()
    # the reference's criterion (:1876-1880): some valid selections, full-length paths, nothing left in flight
    ok = bool(np.any(kinds != 0) and lens.max() == depth + 1 and not d["node_inflight"].numpy().any()
              and not d["node_expand_inflight"].numpy().any())
    invalid_share = float((kinds == 0).mean())
    selections = steps * trees * warps
    # per level: the node word and ticket counter, child / N / W / prior of every edge, one path entry.  The children's
    # virtual-visit counters, which both kernels gather and the preclaim kernel updates twice per edge, are held in the
    # workgroup's LDS for the launch (a tree's 8 traversals are one workgroup): 2 x 4 bytes per node and launch
    level_bytes = 8 + 16 * actions + 4
    alg_bytes = trees * warps * depth * level_bytes + trees * (actions + 1) * 8
    cpu = None
    if not args.no_cpu_baseline:
        from oracle import puct_oracle as po
        sample = 64
        h = {k: np.ascontiguousarray(v[:sample]) for k, v in case.items()}
        t1 = time.perf_counter()
        po.node_select(h, cpuct=1.0, c_pw=0.0, variant=variant)
        dt = time.perf_counter() - t1
        cpu = {"value": sample * warps / dt, "unit": "selections/s", "cores": 1, "kind": "port",
               "sample": f"first {sample} trees of the same workload, one launch ({sample * warps} selections of {depth} levels), "
                         "sequential CPU oracle"}
    launch_s = ms / steps * 1e-3
    prof = profile_json(f"node_select_kernel_{variant}_puct_{args.puct_shape}.md")
    traffic = (prof or {}).get("traffic_bytes_per_launch")
    published = PUCT_NODE_PUBLISHED[args.puct_shape][0 if variant == puct.VARIANT_PRECLAIM else 1]
    value = selections / (ms * 1e-3)
    out = {"metric": f"PUCT selections/s, deep-wide select benchmark of the reference, its {variant} kernel with node-level virtual loss "
                     "(8 traversals per tree)",
           "value": value, "unit": "selections/s", "n_gpus": 1, "steps": steps, "warmup": max(args.warmup, 1),
           "ms_per_step": ms / steps, "higher_is_better": True, "scaling": "weak", "vs_baseline": value / published,
           "baseline": {"value": published, "unit": "selections/s", "hardware": "not stated by the reference (its notes mention an RTX 4090)",
                        "source": "the reference's puct_gpu_v2_select_experiments.md:519-528"},
           "dtype": "f32 scores + int32 atomics", "data": "synthetic",
           "config": {"workload": f"{args.puct_shape}: {trees} trees x {warps} traversals, {actions} edges per node, depth {depth}, equal "
                                  f"priors, c_pw=0, terminal by depth limit; one puct_node_select_{variant}_launch per step"},
           "valid": ok, "invalid_share_last_launch": invalid_share, "levels_per_s": selections * depth / (ms * 1e-3),
           # HBM bytes per launch from the counter summary of this kernel and shape, where one exists, over this run's launch
           # time; the bytes the traversals request (the eight traversals of a tree read the same rows) are an L2-level figure
           "roofline": {"bound": "hbm", "achieved": traffic / launch_s / 1e9 if traffic else None, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": traffic / launch_s / 1e9 / HBM_PEAK_GBS if traffic else None, "traffic": traffic,
                        "traffic_source": {"file": prof["file"], "commit": prof.get("commit"), "stale": prof.get("stale")} if prof else None,
                        "kernel": f"node_select_kernel<{str(variant == puct.VARIANT_PRECLAIM).lower()}, true>", "avg_launch_ms": ms / steps,
                        "l2_level": {"requested_bytes_per_launch": alg_bytes, "requested_GB_per_s": alg_bytes / launch_s / 1e9,
                                     "note": "node word, ticket counter, child / N / W / prior of every edge per level and traversal; "
                                             "the virtual-visit counters are in LDS during the launch"}},
           "cpu_baseline": cpu}
    print(json.dumps(out))


def cpu_oracle_baseline(roots):
    """The CPU oracle (scalar restatement of the reference's kernels, OpenMP over playouts) on a bounded sample of the
    headline workload: the first 8 roots, 400 MCTS steps each."""
    from oracle.oracle import Oracle
    cores = min(16, os.cpu_count() or 1)
    n_sample_roots, sample_steps = 8, 400
    cpu_playouts, dt = 0, 0.0
    for b, f, t in roots[:n_sample_roots]:
        o = Oracle("c4", (M, N), A, A, T, P, "acp_prodigal", ucb_c=2.0, seed=0, device_memory=DEVICE_MEMORY, threads=cores)
        t1 = time.perf_counter()
        o.run(b, f, t, sample_steps)
        dt += time.perf_counter() - t1
        cpu_playouts += int(o.result("root_ns").max())
    return {"value": cpu_playouts / dt, "unit": "playouts/s", "cores": cores, "kind": "port",
            "mcts_steps_per_s": n_sample_roots * sample_steps / dt,
            "sample": f"first {n_sample_roots} roots of the workload, {sample_steps} MCTS steps each ({cpu_playouts} playouts), "
                      "CPU oracle (scalar restatement of the reference's kernels) with OpenMP over playouts"}


def make_gomoku_roots(n_roots=32, seed=0):
    """Seeded synthetic Gomoku roots: 0..20 stones placed alternately on random cells of the 15x15 board."""
    rng = np.random.Generator(np.random.PCG64(seed))
    roots = []
    for _ in range(n_roots):
        board = np.zeros((15, 15), np.int8)
        turn = 1
        for c in rng.permutation(225)[:int(rng.integers(0, 21))]:
            board[c // 15, c % 15] = turn
            turn = -turn
        roots.append((board, turn))
    return roots


def bench_gomoku(args):
    """Gomoku 15x15, 32 seeded roots with 0..20 stones placed alternately on random cells,
    ocp_thrifty, n_trees=4, n_playouts=128, 2000 steps, device_memory=16 GiB; one bench step = one search."""
    import contextlib
    import io
    from mcts_numba_cuda_amd import MCTSNC
    roots = make_gomoku_roots()
    steps = min(args.steps, len(roots)) if args.steps != N_ROOTS else 8
    quiet = io.StringIO()
    prof = profile_json("search_kernel_gomoku_ocp_thrifty_4x128_counters.md")
    with contextlib.redirect_stdout(quiet):
        e = MCTSNC((15, 15), 0, 225, search_time_limit=np.inf, search_steps_limit=2000, n_trees=4, n_playouts=128,
                   variant="ocp_thrifty", device_memory=16.0, ucb_c=2.0, seed=0, verbose_info=False)
        e.init_device_side_arrays()
        apply_launch_options(e)
        for w in range(max(args.warmup, 1)):
            e.reseed()
            e.run(roots[w][0], None, roots[w][1])
        playouts = mcts_steps = plies = 0
        dev = 0.0
        alg = dict(select=0, expand=0, playout=0, backup=0, total=0)
        t0 = time.perf_counter()
        for k in range(steps):
            e.reseed()
            e.run(roots[k][0], None, roots[k][1])
            playouts += e.performance_info["playouts"]
            mcts_steps += e.steps
            plies += e.performance_info["playout_plies"]
            dev += e.time_device_loop
            ab = algorithmic_bytes(e._result, e.steps * 4, acp=False, mn_e=225 + 1, A=225, P=128)
            for key in alg:
                alg[key] += ab[key]
        wall = time.perf_counter() - t0
        # the workload as the batch it is: all 32 roots in one run_batch pass (128 workgroups instead of 4 at a time)
        batched = None
        if not args.no_batched:
            from mcts_numba_cuda_amd import run_batch
            engines = [e]
            for _ in range(len(roots) - 1):
                x = MCTSNC((15, 15), 0, 225, search_time_limit=np.inf, search_steps_limit=2000, n_trees=4, n_playouts=128,
                           variant="ocp_thrifty", device_memory=16.0, ucb_c=2.0, seed=0, verbose_info=False)
                x.init_device_side_arrays()
                apply_launch_options(x)
                engines.append(x)
            for rep in range(2):    # first pass warms the pools up
                for x in engines:
                    x.reseed()
                t1 = time.perf_counter()
                run_batch(engines, [r[0] for r in roots], None, [r[1] for r in roots])
                bt = time.perf_counter() - t1
            bp = sum(x.performance_info["playouts"] for x in engines)
            bplies = sum(x.performance_info["playout_plies"] for x in engines)
            bbytes = sum(algorithmic_bytes(x._result, x.steps * 4, acp=False, mn_e=225 + 1, A=225, P=128)["total"] for x in engines)
            kt = engines[0].time_device_loop
            batched = {"roots_per_pass": len(engines), "playouts_per_s": bp / bt, "searches_per_s": len(engines) / bt,
                       "mcts_steps_per_s_all_roots": sum(x.steps for x in engines) / bt, "ms_per_pass": bt * 1e3, "kernel_ms": kt * 1e3,
                       "playout_plies_per_s": bplies / kt, "algorithmic_GB_per_s": bbytes / kt / 1e9, "hbm_frac": bbytes / kt / 1e9 / HBM_PEAK_GBS,
                       "valu": valu_roofline((prof or {}).get("batched_32_roots", {}).get("sq_insts_valu_per_pass"), kt, prof or {},
                                             "one pass over the 32 roots, gomoku::search_kernel_for<Gomoku, false, 8> with 128 workgroups")}
            for x in engines[1:]:
                x._release()
    per_root = (prof or {}).get("sq_insts_valu_per_root")
    roofline_valu = None
    if per_root and len(per_root) >= steps:
        roofline_valu = valu_roofline(sum(per_root[:steps]), dev, prof, "the timed single searches, gomoku::search_kernel_for<Gomoku, false, 8> on 4 workgroups")
    cpu = None
    if not args.no_cpu_baseline:
        from oracle.oracle import Oracle
        cores = min(16, os.cpu_count() or 1)
        o = Oracle("gomoku", (15, 15), 0, 225, 4, 128, "ocp_thrifty", ucb_c=2.0, seed=0, device_memory=16.0, threads=cores)
        t1 = time.perf_counter()
        o.run(roots[0][0], None, roots[0][1], 300)
        dt = time.perf_counter() - t1
        cpu = {"value": int(o.result("root_ns").max()) / dt, "unit": "playouts/s", "cores": cores, "kind": "port",
               "mcts_steps_per_s": 300 / dt, "sample": "first root, 300 MCTS steps, CPU oracle with OpenMP over playouts"}
    out = {"metric": "playouts/s + steps/s, Gomoku 15x15 OCP-thrifty 4x128 on 1 MI355X", "value": playouts / wall,
           "unit": "playouts/s", "n_gpus": 1, "steps": steps, "warmup": max(args.warmup, 1), "ms_per_step": wall / steps * 1e3,
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bit boards + int32 counters (UCB in f64 rounded to f32)",
           "data": "synthetic",
           "config": {"workload": "Gomoku 15x15, seeded roots with 0-20 random stones, ocp_thrifty n_trees=4 n_playouts=128 ucb_c=2.0 "
                                  "search_steps_limit=2000 device_memory=16GiB seed=0; one MCTSNC.run() per root, sequential"},
           "mcts_steps_per_s": mcts_steps / wall, "playout_plies_per_s": plies / dev, "device_loop_share": dev / wall,
           "batched": batched, "roofline_valu": roofline_valu,
           "roofline": {"bound": "hbm", "achieved": alg["total"] / dev / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": alg["total"] / dev / 1e9 / HBM_PEAK_GBS, "traffic": (prof or {}).get("traffic_bytes_per_launch"),
                        "kernel": "mctsnc::gomoku::search_kernel_for<Gomoku, false, 8>", "algorithmic_bytes_per_launch": alg["total"] / steps,
                        "avg_launch_ms": dev / steps * 1e3,
                        "stage_bytes_per_launch": {k: v / steps for k, v in alg.items() if k != "total"},
                        "note": "four workgroups of two wavefronts: bound by the length of the longest playout "
                                "(about 105 instructions per ply on a lone wavefront), not by memory"},
           "cpu_baseline": cpu}
    e._release()
    print(json.dumps(out))


def readme_gomoku_position():
    """The position of the reference's README showcase ("Example usage 2": 15 stones on 15x15, white to move), kept as data
    with the run's printed results in tests/golden/readme_examples.json."""
    with open(os.path.join(ROOT, "tests", "golden", "readme_examples.json")) as f:
        ex = json.load(f)["gomoku"]
    board = np.array([[{"X": 1, "O": -1, ".": 0}[ch] for ch in row] for row in ex["board_rows"]], dtype=np.int8)
    return ex, board


def bench_gomoku_acp(args):
    """The reference's README showcase: Gomoku 15x15, acp_prodigal, n_trees=8, n_playouts=128, device_memory=2 GiB, seed 0,
    from its 15-stone position for the 442 steps its 5 s run took (the engine reproduces the printed root table:
    tests/test_readme_examples.py).  All 210 children of every expanded node are played out: 210 x 128 playouts per
    tree and step.  One bench step = one such search."""
    import contextlib
    import io
    from mcts_numba_cuda_amd import MCTSNC
    ex, board = readme_gomoku_position()
    p = ex["params"]
    steps = args.steps if args.steps != N_ROOTS else 8
    prof = profile_json("search_kernel_gomoku_acp_prodigal_8x128_counters.md")
    quiet = io.StringIO()
    with contextlib.redirect_stdout(quiet):
        e = MCTSNC((15, 15), 0, 225, search_time_limit=np.inf, search_steps_limit=ex["steps"], n_trees=p["n_trees"], n_playouts=p["n_playouts"],
                   variant=p["variant"], device_memory=p["device_memory"], ucb_c=p["ucb_c"], seed=p["seed"], verbose_info=False, game="gomoku")
        e.init_device_side_arrays()
        apply_launch_options(e)
        for _ in range(max(args.warmup, 1)):
            e.reseed()
            e.run(board, None, ex["turn"])
        assert e.performance_info["playouts"] == ex["playouts"]      # the printed run
        playouts = mcts_steps = plies = 0
        dev = 0.0
        stage = dict(select=0.0, expand=0.0, playout=0.0, backup=0.0)
        alg = dict(select=0, expand=0, playout=0, backup=0, total=0)
        t0 = time.perf_counter()
        for _ in range(steps):
            e.reseed()
            e.run(board, None, ex["turn"])
            playouts += e.performance_info["playouts"]
            mcts_steps += e.steps
            plies += e.performance_info["playout_plies"]
            dev += e.time_device_loop
            for k in stage:
                stage[k] += getattr(e, "time_" + k)
            ab = algorithmic_bytes(e._result, e.steps * p["n_trees"], acp=True, mn_e=225 + 1, A=225, P=p["n_playouts"])
            for key in alg:
                alg[key] += ab[key]
        wall = time.perf_counter() - t0
    cpu = None
    if not args.no_cpu_baseline:
        from oracle.oracle import Oracle
        cores = min(16, os.cpu_count() or 1)
        o = Oracle("gomoku", (15, 15), 0, 225, p["n_trees"], p["n_playouts"], p["variant"], ucb_c=p["ucb_c"], seed=p["seed"],
                   device_memory=p["device_memory"], threads=cores)
        t1 = time.perf_counter()
        o.run(board, None, ex["turn"], 40)
        dt = time.perf_counter() - t1
        cpu = {"value": int(o.result("root_ns").max()) / dt, "unit": "playouts/s", "cores": cores, "kind": "port",
               "mcts_steps_per_s": 40 / dt, "sample": "the same position, 40 MCTS steps, CPU oracle with OpenMP over playouts"}
    out = {"metric": "playouts/s + steps/s, Gomoku 15x15 ACP-prodigal 8x128 (the reference's README showcase) on 1 MI355X",
           "value": playouts / wall, "unit": "playouts/s", "n_gpus": 1, "steps": steps, "warmup": max(args.warmup, 1),
           "ms_per_step": wall / steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": "bit boards + int32 counters (UCB in f64 rounded to f32)", "data": "synthetic",
           "config": {"workload": "Gomoku 15x15, the 15-stone position of the reference's README, acp_prodigal n_trees=8 n_playouts=128 "
                                  "ucb_c=2.0 device_memory=2GiB seed=0, 442 steps (what the reference's 5 s run reached: 88 steps/s, "
                                  "18.8 M playouts/s there)"},
           "mcts_steps_per_s": mcts_steps / wall, "playout_plies_per_s": plies / dev, "device_loop_share": dev / wall,
           "stage_ms_per_mcts_step": {k: v / mcts_steps * 1e3 for k, v in stage.items()},
           "stage_achieved_gbs": {k: alg[k] / stage[k] / 1e9 for k in stage if stage[k]},
           "roofline_valu": valu_roofline((prof or {}).get("sq_insts_valu_per_launch"), dev / steps, prof or {},
                                          "one search, gomoku::search_kernel_for<Gomoku, true, 8> on 512 workgroups of 128 threads"),
           "roofline": {"bound": "hbm", "achieved": alg["total"] / dev / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": alg["total"] / dev / 1e9 / HBM_PEAK_GBS, "traffic": (prof or {}).get("traffic_bytes_per_launch"),
                        "traffic_source": {"file": prof["file"], "commit": prof.get("commit"), "stale": prof.get("stale")} if prof else None,
                        "kernel": "mctsnc::gomoku::search_kernel_for<Gomoku, true, 8>", "algorithmic_bytes_per_launch": alg["total"] / steps,
                        "avg_launch_ms": dev / steps * 1e3,
                        "stage_bytes_per_launch": {k: v / steps for k, v in alg.items() if k != "total"},
                        "note": "1.7 M playouts per step whose generators stay on chip: bound by the instruction stream of the "
                                "playouts (LDS-resident boards, two workgroups per CU), not by memory"},
           "cpu_baseline": cpu}
    e._release()
    print(json.dumps(out))


def puct_gomoku_search(board, steps, search_steps, warmup, **kw):
    """`steps` timed searches of `search_steps` steps each; returns totals and the algorithmic bytes by phase."""
    from mcts_numba_cuda_amd.puct_gomoku import PUCTGomoku
    e = PUCTGomoku(**kw)
    for _ in range(max(warmup, 1)):
        e.run(board, 1, 200)
    # legal cells of the nodes a search creates (a 16-byte record and a cell byte are written for each): the trees are the
    # same in every search, so one look at one search's arrays serves all
    e.run(board, 1, search_steps)
    counts, legal_arr, expanded_arr = e.read_array("node_count"), e.read_array("node_legal"), e.read_array("node_expanded")
    created = sum(int(c) - 1 for c in counts)
    legal_per_created = sum(int(legal_arr[t, 1:c][expanded_arr[t, 1:c] != -1].sum()) for t, c in enumerate(counts)) / max(created, 1)
    tot = dict(selections=0, leaves=0, busy=0, nodes=0, dev=0.0, select=0.0, expand=0.0, backup=0.0)
    alg = dict(select=0, expand=0, backup=0, total=0)
    t0 = time.perf_counter()
    for _ in range(steps):
        e.run(board, 1, search_steps)
        p, r = e.performance_info, e.result
        tot["selections"] += p["selections"]
        tot["leaves"] += p["leaves"]
        tot["busy"] += e.selections["busy"]
        tot["nodes"] += p["nodes_total"]
        tot["dev"] += r.time_device
        for k in ("select", "expand", "backup"):
            tot[k] += getattr(r, "time_" + k)
        # Algorithmic bytes of the loop's own layout.  Selection: a node that a group of traversals stands on is read once
        # (16-byte node word + one 16-byte record per expanded edge), a claim rewrites the edge's 4-byte link word and
        # adds a 4-byte path entry, every traversal leaves 12 bytes (selection word, length, claims).  Expansion: parent
        # position and node word in (64 + 16), the slot's cell in (1), child position, node word and link out (64 + 16 +
        # 12), one 16-byte record and one cell byte per legal cell of the child.  Backup: three 4-byte words of every
        # path edge in and out (24).
        legal_cells = legal_per_created * r.expansions_committed
        b_sel = 16 * r.nodes_read + 16 * r.edges_scored + 12 * p["selections"]
        b_exp = r.expansions_committed * (64 + 16 + 1 + 64 + 16 + 12) + 17 * legal_cells
        alg["select"] += b_sel
        alg["expand"] += b_exp
    wall = time.perf_counter() - t0
    # path edges: every visit of an edge was a path entry of a traversal that reached a node; visits = sum over all
    # edges of n minus the visit each child got at its creation.  Claims of busy traversals are not counted (few bytes).
    edge_n = e.read_array("edge_n")
    visits = 0
    for t, c in enumerate(counts):
        rows = edge_n[t, :c]
        ne = np.maximum(expanded_arr[t, :c], 0)
        visits += int(rows[np.arange(256)[None, :] < ne[:, None]].sum()) - (int(c) - 1)
    del edge_n
    alg["select"] += 8 * visits * steps
    alg["backup"] = 24 * visits * steps
    alg["total"] = alg["select"] + alg["expand"] + alg["backup"]
    e.close()
    return tot, alg, wall


def bench_puct_gomoku(args):
    """PUCT on Gomoku 15x15 with virtual loss, 16 trees x 16 traversals = 256 leaves per step, Dirichlet(0.3) priors and
    hashed values, c_puct = 1.5, 4000 steps; one bench step = one whole search.  c_pw = 16: a node without children
    admits a ticket per traversal, so every selection reaches a leaf; the reference's default c_pw = 1 is timed beside it
    (most traversals of a step then end busy behind the first to reach a new node: that follows from the widening rule,
    the host oracle shows the same share)."""
    steps = args.steps if args.steps != N_ROOTS else 5
    search_steps = 4000
    prof = profile_json("search_kernel_puct_gomoku_16_trees_x16.md")
    board = np.zeros((15, 15), np.int8)
    kw = dict(trees=16, traversals=16, path_depth=64, cpuct=1.5, alpha_pw=0.5, dirichlet_alpha=0.3, seed=0)
    tot, alg, wall = puct_gomoku_search(board, steps, search_steps, args.warmup, c_pw=16.0, max_nodes=65536, **kw)
    ref, _, ref_wall = puct_gomoku_search(board, max(steps // 2, 1), search_steps, 1, c_pw=1.0, max_nodes=16384, **kw)
    dev, n_steps = tot["dev"], steps * search_steps
    cpu = None
    if not args.no_cpu_baseline:
        from oracle import puct_oracle as po
        t1 = time.perf_counter()
        h = po.gomoku_search(board, 1, 1000, c_pw=16.0, max_nodes=16384, threads=1, **kw)
        dt = time.perf_counter() - t1
        cpu = {"value": int(h["tally"][:, 1:4].sum()) / dt, "unit": "leaves/s", "cores": 1, "kind": "port",
               "sample": "the same search for 1000 steps (256000 selections, all of them leaves), host oracle on one core"}
    out = {"metric": "PUCT leaves/s (selections that reach a node and are evaluated and backed up), Gomoku 15x15 search loop "
                     "with virtual loss (16 trees x 16 traversals)",
           "value": tot["leaves"] / wall, "unit": "leaves/s", "n_gpus": 1, "steps": steps, "warmup": max(args.warmup, 1),
           "ms_per_step": wall / steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": "f32 scores, int32 counters, claims in a fixed order (no atomics)", "data": "synthetic",
           "config": {"workload": "Gomoku 15x15 empty board, 16 trees x 16 traversals per step, Dirichlet(0.3) priors and hashed "
                                  "values, c_puct=1.5, c_pw=16, alpha_pw=0.5, 4000 steps per search, room for 65536 nodes per "
                                  "tree (64001 used), 4 evaluator workgroups per tree"},
           "selections_per_s": tot["selections"] / wall, "busy_share": tot["busy"] / tot["selections"],
           "leaves_per_step": tot["leaves"] / n_steps, "search_steps_per_s": n_steps / wall,
           "nodes_created_per_search": tot["nodes"] / steps, "device_share": dev / wall,
           "us_per_search_step": {"total": dev / n_steps * 1e6, "select": tot["select"] / n_steps * 1e6,
                                  "expand": tot["expand"] / n_steps * 1e6, "backup": tot["backup"] / n_steps * 1e6},
           "stage_achieved_gbs": {k: alg[k] / max(tot[k], 1e-12) / 1e9 for k in ("select", "expand", "backup")},
           "reference_default_widening": {
               "config": "c_pw=1 (src/puct/puct_gpu_v3_cpp.py:121), room for 16384 nodes per tree, otherwise the same",
               "leaves_per_s": ref["leaves"] / ref_wall, "selections_per_s": ref["selections"] / ref_wall,
               "busy_share": ref["busy"] / ref["selections"], "leaves_per_step": ref["leaves"] / (max(steps // 2, 1) * search_steps),
               "search_steps_per_s": max(steps // 2, 1) * search_steps / ref_wall},
           "roofline": {"bound": "hbm", "achieved": alg["total"] / dev / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": alg["total"] / dev / 1e9 / HBM_PEAK_GBS, "traffic": (prof or {}).get("traffic_bytes_per_launch"),
                        "traffic_source": {"file": prof["file"], "commit": prof.get("commit"), "stale": prof.get("stale")} if prof else None,
                        "kernel": "puct::search_kernel (select, expand, backup of all 4000 steps in one launch)",
                        "algorithmic_bytes_per_launch": alg["total"] / steps, "avg_launch_ms": dev / steps * 1e3,
                        "stage_bytes_per_launch": {k: v / steps for k, v in alg.items() if k != "total"},
                        "note": "16 tree workgroups of 16 wavefronts and 64 evaluator workgroups of 8: a step is a chain of dependent "
                                "decisions (the traversals on one node decide in turn) and one round trip per tree level, "
                                "not a stream"},
           "roofline_valu": valu_roofline((prof or {}).get("sq_insts_valu_per_launch"), dev / steps, prof or {}, "one search of 4000 steps"),
           "cpu_baseline": cpu}
    print(json.dumps(out))


def bench_c4_many(args):
    """Many searches of the headline configuration (C4 6x7 acp_prodigal 4x256, 5000 steps each) in one run_batch pass: the
    64 seeded roots repeated, every search with its own engine and pools (60 MiB each); one bench step = one pass."""
    import contextlib
    import io
    from mcts_numba_cuda_amd import MCTSNC, run_batch
    roots = make_roots(N_ROOTS)
    n = args.searches
    prof = profile_json("search_kernel_solo_c4_768_searches.md")
    steps = args.steps if args.steps != N_ROOTS else 3
    with contextlib.redirect_stdout(io.StringIO()):
        engines = []
        for _ in range(n):
            e = MCTSNC((M, N), A, A, search_time_limit=np.inf, search_steps_limit=STEPS, n_trees=T, n_playouts=P,
                       variant="acp_prodigal", device_memory=0.06, ucb_c=2.0, seed=0, verbose_info=False)
            e.init_device_side_arrays()
            apply_launch_options(e)
            engines.append(e)
        chunk = [roots[i % len(roots)] for i in range(n)]
        times = []
        for k in range(max(args.warmup, 1) + steps):
            for e in engines:
                e.reseed()
            t0 = time.perf_counter()
            run_batch(engines, [c[0] for c in chunk], [c[1] for c in chunk], [c[2] for c in chunk])
            if k >= max(args.warmup, 1):
                times.append(time.perf_counter() - t0)
        playouts = sum(e.performance_info["playouts"] for e in engines)
        abytes = sum(algorithmic_bytes(e._result, e.steps * T)["total"] for e in engines)
        dev = engines[0].time_device_loop
        for e in engines:
            e._release()
    dt = sum(times) / len(times)
    out = {"metric": "playouts/s, many concurrent C4 6x7 ACP-prodigal 4x256 searches in one pass on 1 MI355X", "value": playouts / dt,
           "unit": "playouts/s", "n_gpus": 1, "steps": steps, "warmup": max(args.warmup, 1), "ms_per_step": dt * 1e3,
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": "int64 bitboards + int32 counters (UCB in f64 rounded to f32)", "data": "synthetic",
           "config": {"workload": f"C4 6x7, {n} searches (the 64 seeded roots repeated) x acp_prodigal n_trees=4 n_playouts=256 "
                                  "search_steps_limit=5000 device_memory=60MiB each, all in one run_batch pass"},
           "searches_per_s": n / dt, "trees_in_flight": n * T, "mcts_steps_per_s_all_searches": n * STEPS / dt,
           "roofline": {"bound": "hbm", "achieved": abytes / dev / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": abytes / dev / 1e9 / HBM_PEAK_GBS,
                        "traffic": (prof or {}).get("traffic_bytes_per_launch") if n == (prof or {}).get("searches") else None,
                        "kernel": "mctsnc::c4::search_kernel_solo (batches of 896 trees or more), mctsnc::c4::search_kernel<true> below",
                        "algorithmic_bytes_per_launch": abytes, "avg_launch_ms": dev * 1e3},
           "roofline_valu": valu_roofline((prof or {}).get("sq_insts_valu_per_pass") if n == (prof or {}).get("searches") else None, dev, prof or {},
                                          f"one pass over {n} searches"),
           "cpu_baseline": None if args.no_cpu_baseline else cpu_oracle_baseline(roots)}
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=N_ROOTS, help="number of timed searches (roots)")
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-batched", action="store_true")
    ap.add_argument("--plain-launch", action="store_true",
                    help="launch the kernels whose workgroups wait for each other as ordinary kernels (for profilers)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run a plain 1 GiB device-to-device copy (the known-size kernel that FETCH_SIZE / "
                         "WRITE_SIZE readings are scaled by) and exit")
    ap.add_argument("--workload", default="c4", choices=("c4", "c4_many", "gomoku", "gomoku_acp", "puct_select", "puct_gomoku"),
                    help="c4: the headline MCTS-NC search (default); puct_select: the reference's deep-wide PUCT selection "
                         "benchmark through puct_select_winner_recalc_launch; puct_gomoku: the Gomoku PUCT search loop")
    ap.add_argument("--puct-shape", default="eq64_d512", choices=sorted(PUCT_SHAPES))
    ap.add_argument("--select-variant", default="edge_winner_recalc", choices=("edge_winner_recalc", "node_preclaim", "node_winner_recalc"),
                    help="puct_select: the C-ABI kernel with edge-level virtual loss (default) or one of the reference's two kernels "
                         "with node-level virtual loss")
    ap.add_argument("--searches", type=int, default=768, help="c4_many: concurrent searches in the pass")
    args = ap.parse_args()
    global PLAIN_LAUNCH
    PLAIN_LAUNCH = args.plain_launch
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (trees are independent and would shard over GPUs with one "
                 "final all-reduce of the root table, but no multi-GPU path is part of it); run with --gpus 1")

    if args.copy_calibration:
        import torch
        src = torch.arange(1 << 28, dtype=torch.int32, device="cuda")   # 1 GiB
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration_bytes_read": src.numel() * 4, "bytes_written": dst.numel() * 4, "copies": 4}))
        return

    if args.workload == "gomoku":
        return bench_gomoku(args)
    if args.workload == "gomoku_acp":
        return bench_gomoku_acp(args)
    if args.workload == "c4_many":
        return bench_c4_many(args)
    if args.workload == "puct_select":
        return bench_puct_select(args) if args.select_variant == "edge_winner_recalc" else bench_puct_node_select(args)
    if args.workload == "puct_gomoku":
        return bench_puct_gomoku(args)

    import contextlib
    import io
    from mcts_numba_cuda_amd import MCTSNC, run_batch

    roots = make_roots(max(N_ROOTS, 1))
    quiet = io.StringIO()
    prof = profile_json("search_kernel_c4_acp_prodigal_4x256_counters.md")

    def new_engine():
        e = MCTSNC((M, N), A, A, search_time_limit=np.inf, search_steps_limit=STEPS, n_trees=T, n_playouts=P,
                   variant="acp_prodigal", device_memory=DEVICE_MEMORY, ucb_c=2.0, seed=0, verbose_info=False)
        e.init_device_side_arrays()
        apply_launch_options(e)
        return e

    with contextlib.redirect_stdout(quiet):
        eng = new_engine()
        for w in range(args.warmup):
            b, f, t = roots[w % len(roots)]
            eng.reseed()
            eng.run(b, f, t)

        device_synchronize()
        playouts = mcts_steps = 0
        dev_time = 0.0
        alg = dict(select=0, expand=0, playout=0, backup=0, total=0)
        stage = dict(select=0.0, expand=0.0, playout=0.0, backup=0.0)
        plies = 0
        t0 = time.perf_counter()
        for k in range(args.steps):
            b, f, t = roots[k % len(roots)]
            eng.reseed()
            eng.run(b, f, t)
            playouts += eng.performance_info["playouts"]
            mcts_steps += eng.steps
            dev_time += eng.time_device_loop
            plies += eng.performance_info["playout_plies"]
            ab = algorithmic_bytes(eng._result, eng.steps * T)
            for key in alg:
                alg[key] += ab[key]
            stage["select"] += eng.time_select
            stage["expand"] += eng.time_expand
            stage["playout"] += eng.time_playout
            stage["backup"] += eng.time_backup
        device_synchronize()
        elapsed = time.perf_counter() - t0

        batched = trees_512 = None
        if not args.no_batched:
            # the same 64 searches, all handed to the device at once (one launch: the resident sets of workgroups take
            # further trees from a queue as they finish theirs); results are identical to the sequential runs
            nb = min(len(roots), max(args.steps, 1))
            engines = [eng] + [new_engine() for _ in range(nb - 1)]
            chunk = roots[:nb]
            for rep in range(2):    # first pass warms the pools up
                for e in engines:
                    e.reseed()
                t1 = time.perf_counter()
                run_batch(engines, [c[0] for c in chunk], [c[1] for c in chunk], [c[2] for c in chunk])
                bt = time.perf_counter() - t1
            bp = sum(e.performance_info["playouts"] for e in engines)
            bbytes = sum(algorithmic_bytes(e._result, e.steps * T)["total"] for e in engines)
            batched = {"roots_per_pass": nb, "playouts_per_s": bp / bt, "searches_per_s": nb / bt,
                       "mcts_steps_per_s_all_roots": nb * STEPS / bt, "ms_per_pass": bt * 1e3, "kernel_ms": engines[0].time_device_loop * 1e3,
                       "playout_plies_per_s": sum(e.performance_info["playout_plies"] for e in engines) / engines[0].time_device_loop,
                       "algorithmic_GB_per_s": bbytes / bt / 1e9, "hbm_frac": bbytes / bt / 1e9 / HBM_PEAK_GBS,
                       "valu": valu_roofline((prof or {}).get("batched_64_roots", {}).get("sq_insts_valu_per_pass") if nb == N_ROOTS else None,
                                             engines[0].time_device_loop, prof or {}, "one pass over the 64 roots, search_kernel<true>")}
            for e in engines[1:]:
                e._release()
            del engines
            # the widest search the reference's interface allows (n_trees=512, its MAX_N_TREES): the tree traffic of
            # one search is large enough here for the HBM fraction to mean something
            wide = MCTSNC((M, N), A, A, search_time_limit=np.inf, search_steps_limit=STEPS, n_trees=512, n_playouts=P,
                          variant="acp_prodigal", device_memory=16.0, ucb_c=2.0, seed=0, verbose_info=False)
            wide.init_device_side_arrays()
            apply_launch_options(wide)
            b, f, t = np.zeros((M, N), np.int8), np.zeros(N, np.int8), 1     # empty board
            for rep in range(2):
                wide.reseed()
                t1 = time.perf_counter()
                wide.run(b, f, t)
                wt = time.perf_counter() - t1
            wbytes = algorithmic_bytes(wide._result, wide.steps * 512)["total"]
            trees_512 = {"n_trees": 512, "root": "empty board", "playouts_per_s": wide.performance_info["playouts"] / wt, "ms_per_search": wt * 1e3,
                         "mcts_steps_per_s": wide.steps / wt, "tree_steps_per_s": wide.steps * 512 / wt,
                         "kernel_ms": wide.time_device_loop * 1e3, "playout_plies_per_s": wide.performance_info["playout_plies"] / wide.time_device_loop,
                         "algorithmic_GB_per_s": wbytes / wt / 1e9, "hbm_frac": wbytes / wt / 1e9 / HBM_PEAK_GBS,
                         "valu": valu_roofline((prof or {}).get("trees_512", {}).get("sq_insts_valu_per_search"), wide.time_device_loop, prof or {},
                                               "one search with 512 trees, search_kernel_solo")}
            wide._release()
        eng._release()      # free the pools now rather than at interpreter exit, after the HIP runtime has shut down

    value = playouts / elapsed
    launches = args.steps  # one search kernel launch per search at a fixed step budget
    roofline = {"bound": "hbm", "achieved": alg["total"] / dev_time / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": alg["total"] / dev_time / 1e9 / HBM_PEAK_GBS,
                # HBM bytes per launch from the rocprofv3 FETCH_SIZE / WRITE_SIZE runs summarised in the named file
                "traffic": (prof or {}).get("traffic_bytes_per_launch"),
                "traffic_source": {"file": prof["file"], "commit": prof.get("commit"), "launches": prof.get("traffic_launches")} if prof else None,
                "kernel": "mctsnc::c4::search_kernel<true>", "algorithmic_bytes_per_launch": alg["total"] / launches,
                "avg_launch_ms": dev_time / launches * 1e3,
                "stage_bytes_per_launch": {k: v / launches for k, v in alg.items() if k != "total"},
                "playout_plies_per_s": plies / dev_time,
                "note": "latency-bound pointer chasing plus integer playouts on 28 workgroups: a few KB of tree data per step"}

    # vector-ALU side: the counted instructions of the timed roots over their kernel time
    per_root = (prof or {}).get("sq_insts_valu_per_root")
    roofline_valu = None
    if per_root and len(per_root) == len(roots):
        roofline_valu = valu_roofline(sum(per_root[k % len(roots)] for k in range(args.steps)), dev_time, prof,
                                      "the timed single searches, search_kernel<true> on 28 of 256 CUs")

    cpu_baseline = None
    if not args.no_cpu_baseline:
        cpu_baseline = cpu_oracle_baseline(roots)

    cpu_mcts = None
    if not args.no_cpu_baseline:
        # the reference's own CPU player (src/mcts.py, mirrored in mcts_numba_cuda_amd/mcts.py): one playout per step,
        # single-threaded, on the first four roots of the workload for half a second each
        from mcts_numba_cuda_amd.c4 import C4
        from mcts_numba_cuda_amd.mcts import MCTS
        cpu_steps, cpu_time = 0, 0.0
        with contextlib.redirect_stdout(quiet):
            cpu_ai = MCTS(search_time_limit=0.5, search_steps_limit=np.inf, vanilla=True, ucb_c=2.0, seed=0)
            for b0, f0, t0_ in roots[:4]:
                state = C4()
                state.board[:], state.column_fills[:], state.turn = b0, f0, t0_
                cpu_ai.run(state)
                cpu_steps += cpu_ai.steps
                cpu_time += cpu_ai.time_total
        cpu_mcts = {"playouts_per_s": cpu_steps / cpu_time, "steps_per_s": cpu_steps / cpu_time, "cores": 1,
                    "kind": "host mirror of the reference's CPU MCTS (pure Python, no numba)",
                    "sample": "first four roots of the workload, 0.5 s time limit each"}

    out = {"metric": "playouts/s + steps/s, C4 6x7 ACP-prodigal 4x256 on 1 MI355X; % of roofline",
           "value": value, "unit": "playouts/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": elapsed / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": "int64 bitboards + int32 counters (UCB in f64 rounded to f32)", "data": "synthetic",
           "config": {"workload": "C4 6x7, 64 seeded roots (10-20 random plies), acp_prodigal n_trees=4 n_playouts=256 ucb_c=2.0 "
                                  "search_steps_limit=5000 device_memory=2GiB seed=0; one MCTSNC.run() per root, sequential",
                      "bench_step": "one search of 5000 MCTS steps"},
           "mcts_steps_per_s": mcts_steps / elapsed,
           "device_loop_share": dev_time / elapsed,
           "stage_ms_per_mcts_step": {k: v / mcts_steps * 1e3 for k, v in stage.items()},
           # algorithmic bytes of a stage over the device time of that stage (the stage clock of one workgroup of tree 0)
           "stage_achieved_gbs": {k: alg[k] / stage[k] / 1e9 for k in ("select", "expand", "playout", "backup") if stage.get(k)},
           "stage_hbm_frac": {k: alg[k] / stage[k] / 1e9 / HBM_PEAK_GBS for k in ("select", "expand", "playout", "backup") if stage.get(k)},
           "batched": batched, "trees_512": trees_512,
           "roofline": roofline, "roofline_valu": roofline_valu, "cpu_baseline": cpu_baseline, "cpu_mcts": cpu_mcts}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
