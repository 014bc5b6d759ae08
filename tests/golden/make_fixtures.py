"""Condenses the reference's recorded artefacts into the small fixtures kept in this folder.

Inputs (data files of the reference, read as data, never executed):
  * extras/mctsnc_{ocp,acp}_thrifty_c4_1000steps.json  -- complete tree dumps written by the
    reference's MCTSNC._json_dump (src/mctsnc.py:2377-2462) after 1000 steps, T=4, P=128, seed 0.
  * experiments/*.zip -- tournament archives (src/utils.py:168-185): the stdout log holds, for every
    search, all root actions' n / n_wins / win_flag, the step count and the tree statistics.

Outputs:
  * dump_<variant>_c4_1000steps.npz   per tree: trees (children rows of leaves masked to -1, because
                                      the reference leaves them uninitialised), depths, turns, ns,
                                      ns_wins; plus the last step's scratch arrays.
  * archive_games.json                for every archive: engine parameters and, for the first games,
                                      the ordered list of moves and MCTSNC / MCTS searches.

Usage: python tests/golden/make_fixtures.py [/root/reference]
"""
import ast
import glob
import json
import os
import re
import sys
import zipfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
N_GAMES_DEFAULT = 1
N_GAMES = {"mcts_5_inf_vanilla;mctsnc_5_inf_4_256_acp_prodigal": 3,
           "mcts_5_inf_vanilla;mctsnc_1_inf_1_32_ocp_thrifty": 4,
           "mcts_5_inf_vanilla;mctsnc_1_inf_2_64_acp_thrifty": 3,
           "mcts_5_inf_vanilla;mctsnc_1_inf_2_32_ocp_prodigal": 3,
           "mcts_5_inf_vanilla;mctsnc_1_inf_1_64_acp_prodigal": 3}


def condense_dump(path, out):
    d = json.load(open(path))
    sizes = np.array(d["trees_sizes"], dtype=np.int32)
    T = len(sizes)
    arrays = {"trees_sizes": sizes}
    meta = {k: d[k] for k in ["n_trees", "n_playouts", "variant", "search_steps_limit", "ucb_c", "seed", "device_memory"]}
    arrays["meta_json"] = np.frombuffer(json.dumps(meta).encode(), dtype=np.uint8)
    for ti in range(T):
        sz = int(sizes[ti])
        trees = np.array(d["trees"][ti], dtype=np.int32)[:sz]
        ns = np.array(d["trees_ns"][ti], dtype=np.int32)[:sz]
        # a node is expanded iff some other node names it as parent
        expanded = np.zeros(sz, dtype=bool)
        expanded[trees[1:, 0]] = True
        trees[~expanded, 1:] = -1
        arrays[f"trees_{ti}"] = trees
        arrays[f"depths_{ti}"] = np.array(d["trees_depths"][ti], dtype=np.int16)[:sz]
        arrays[f"turns_{ti}"] = np.array(d["trees_turns"][ti], dtype=np.int8)[:sz]
        arrays[f"ns_{ti}"] = ns
        arrays[f"ns_wins_{ti}"] = np.array(d["trees_ns_wins"][ti], dtype=np.int32)[:sz]
    arrays["nodes_selected"] = np.array(d["trees_nodes_selected"], dtype=np.int32)
    paths = np.array(d["trees_selected_paths"], dtype=np.int32)
    arrays["selected_paths"] = paths  # per tree: entries [0, len) valid, last entry = len
    arrays["actions_expanded"] = np.array(d["trees_actions_expanded"], dtype=np.int16)
    arrays["playout_outcomes"] = np.array(d["trees_playout_outcomes"], dtype=np.int32)
    if "trees_playout_outcomes_children" in d:
        arrays["playout_outcomes_children"] = np.array(d["trees_playout_outcomes_children"], dtype=np.int32)
    np.savez_compressed(out, **arrays)


_INSTANCE_RE = re.compile(r"MCTSNC\(search_time_limit=([^,]+), search_steps_limit=([^,]+), n_trees=(\d+), n_playouts=(\d+), "
                          r"variant='(\w+)', device_memory=([^,]+), ucb_c=([^,]+), seed: (\d+)\)")


def parse_instance(s):
    m = _INSTANCE_RE.search(s)
    if not m:
        return None
    return dict(n_trees=int(m.group(3)), n_playouts=int(m.group(4)), variant=m.group(5), device_memory=float(m.group(6)),
                ucb_c=float(m.group(7)), seed=int(m.group(8)))


def parse_block(lines, i):
    """Parses a '{' ... '}]' block printed by utils.dict_to_str starting at lines[i] == '{'; returns (dict, next_i)."""
    assert lines[i].strip() == "{", lines[i]
    out = {}
    i += 1
    while not lines[i].startswith("}"):
        line = lines[i].strip().rstrip(",")
        key, _, val = line.partition(": ")
        val = re.sub(r"np\.(?:float|int)\d+\(([^()]*)\)", r"\1", val)  # newer numpy reprs in some logs
        val = re.sub(r"\b(nan|inf)\b", r"None", val)
        try:
            out[key] = ast.literal_eval(val)
        except (ValueError, SyntaxError):
            out[key] = val
        i += 1
    return out, i + 1


def parse_log(log, n_games):
    lines = log.split("\n")
    games = []
    i = 0
    cur = None
    while i < len(lines):
        ln = lines[i]
        if ln.startswith("MCTS-NC EXPERIMENT..."):  # an interrupted experiment restarted in the same log
            games, cur = [], None
        m = re.match(r"GAME (\d+)/(\d+):", ln)
        if m:
            if int(m.group(1)) > n_games:
                break
            cur = {"black": lines[i + 1][len("BLACK: "):], "white": lines[i + 2][len("WHITE: "):], "events": []}
            games.append(cur)
            ply = 0
            i += 3
            continue
        if cur is not None and (ln.startswith("MCTSNC RUN...") or ln.startswith("MCTS RUN...")):
            kind = "mctsnc" if ln.startswith("MCTSNC") else "mcts"
            if not lines[i + 1].startswith("[actions info:"):  # search cut off by an interruption
                i += 1
                continue
            actions, j = parse_block(lines, i + 2)
            assert lines[j].startswith("[performance info:"), lines[j]
            perf, j = parse_block(lines, j + 1)
            ev = {"type": kind, "side": "black" if ply % 2 == 0 else "white", "steps": perf["steps"], "playouts": perf["playouts"]}
            best = actions.pop("best")
            ev["best"] = best["index"]
            ev["actions"] = {str(k): [v["n"], v["n_wins"], int(v["win_flag"])] for k, v in actions.items()}
            ev["n_root"] = best["n_root"]
            tr = perf.get("trees") or perf.get("tree")
            if kind == "mctsnc":
                ev["trees"] = {k: tr[k] for k in ["mean_depth", "max_depth", "mean_size", "max_size"]}
            else:
                ev["tree"] = {k: tr[k] for k in ["n_root", "mean_depth", "max_depth", "size"]}
            cur["events"].append(ev)
            i = j
            continue
        m = re.match(r"MOVE PLAYED: (\d+)", ln)
        if m and cur is not None:
            cur["events"].append({"type": "move", "action": int(m.group(1))})
            ply += 1
        m = re.match(r"GAME OUTCOME: (.*)", ln)
        if m and cur is not None:
            cur["outcome"] = m.group(1)
        i += 1
    return games


def condense_archives(ref_root, out):
    res = {}
    for path in sorted(glob.glob(os.path.join(ref_root, "experiments", "*.zip"))):
        name = os.path.basename(path)
        key = name[name.index("[") + 1:name.rindex("]")]
        if "C4_6x7" not in key:
            continue
        short = ";".join(key.split(";")[:2])
        z = zipfile.ZipFile(path)
        log = z.read([n for n in z.namelist() if n.endswith(".log")][0]).decode()
        games = parse_log(log, N_GAMES.get(short, N_GAMES_DEFAULT))
        engines = {}
        for g in games:
            for side in ("black", "white"):
                inst = parse_instance(g[side])
                if inst:
                    engines[g[side]] = inst
        sizes = [int(x) for x in re.findall(r"calculated max_tree_size: (\d+)", log)]
        res[key] = {"archive": name, "engines": engines, "max_tree_sizes_logged": sizes, "games": games}
    json.dump(res, open(out, "w"), separators=(",", ":"))


if __name__ == "__main__":
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    for variant in ("ocp_thrifty", "acp_thrifty"):
        condense_dump(os.path.join(ref, "extras", f"mctsnc_{variant}_c4_1000steps.json"),
                      os.path.join(HERE, f"dump_{variant}_c4_1000steps.npz"))
    condense_archives(ref, os.path.join(HERE, "archive_games.json"))
    print("fixtures written to", HERE)
