"""Condenses the reference's recorded artefacts into the small fixtures kept in this folder.

Inputs (data files of the reference, read as data, never executed):
  * README.md -- two example runs with their full printouts (the only recorded Gomoku search there is).
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
  * north_star_experiment.json.gz     all 100 games of the experiment with acp_prodigal 4x256 against the CPU
                                      player (moves and MCTSNC searches only), in the same format.
  * readme_examples.json              the two complete MCTSNC runs printed in the reference's README.md ("Example
                                      usage 1 (Connect 4)" and "Example usage 2 (Gomoku)"): the drawn root position,
                                      the constructor parameters of the printed instance, the step count, every root
                                      action row the printout shows (the Gomoku one elides most of its 210 rows), the
                                      best action and the tree statistics.

Usage: python tests/golden/make_fixtures.py [/root/reference]
"""
import ast
import glob
import gzip
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


sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from mcts_numba_cuda_amd.archive import parse_instance, parse_log  # noqa: E402  (the log parser lives with the replay tool)


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


NORTH_STAR = "mcts_5_inf_vanilla;mctsnc_5_inf_4_256_acp_prodigal;C4_6x7"


def condense_whole_experiment(ref_root, out):
    path = [p for p in glob.glob(os.path.join(ref_root, "experiments", "*.zip")) if NORTH_STAR in p][0]
    name = os.path.basename(path)
    z = zipfile.ZipFile(path)
    log = z.read([n for n in z.namelist() if n.endswith(".log")][0]).decode()
    games = parse_log(log, 10 ** 6)
    engines = {}
    for g in games:
        g["events"] = [e for e in g["events"] if e["type"] in ("move", "mctsnc")]
        for side in ("black", "white"):
            inst = parse_instance(g[side])
            if inst:
                engines[g[side]] = inst
    with gzip.GzipFile(out, "wb", mtime=0) as f:
        f.write(json.dumps({"archive": name, "engines": engines, "games": games}, separators=(",", ":")).encode())


def condense_readme(ref_root, out):
    """The two example runs of README.md.  Boards are drawn with the symbols of C4.SYMBOLS / Gomoku.SYMBOLS
    (src/c4.py:24, src/gomoku.py:25: index = cell value + 1, so the hollow disc is -1 and the full disc +1); a C4
    drawing lists row 0 first (src/c4.py:52-69), a Gomoku drawing lists row M-1 first and labels rows from 1
    (src/gomoku.py:44-64).  Stored as rows of 'X' (+1), 'O' (-1), '.' (empty) in board index order."""
    text = open(os.path.join(ref_root, "README.md"), encoding="utf-8").read()
    sym = {"\u25CF": "X", "\u25CB": "O", ".": ".", "+": "."}
    examples = {}
    for name, title in (("c4", "## Example usage 1 (Connect 4)"), ("gomoku", "## Example usage 2 (Gomoku)")):
        part = text[text.index(title):]
        part = part[:part.index("\n## ", 5)]
        blocks = re.findall(r"```bash\n(.*?)```", part, flags=re.S)
        drawing, printout = blocks[0], blocks[1]
        rows = []
        if name == "c4":
            for line in drawing.splitlines():
                if line.startswith("|"):
                    rows.append("".join(sym[ch] for ch in line.strip().strip("|").split("|")))
        else:
            labelled = {}
            for line in drawing.splitlines():
                mt = re.match(r"\s*(\d+)(\S+?)(\d+)\s*$", line)
                if mt and mt.group(1) == mt.group(3):
                    labelled[int(mt.group(1))] = "".join(sym[ch] for ch in mt.group(2))
            rows = [labelled[i + 1] for i in range(len(labelled))]
        n_pos = sum(r.count("X") for r in rows)
        n_neg = sum(r.count("O") for r in rows)
        turn = 1 if n_pos == n_neg else -1   # +1 moves first (src/mcts.py State.__init__: turn = 1)
        assert n_pos - n_neg in (0, 1)
        inst = re.search(r"MCTSNC RUN\.\.\. \[MCTSNC\((.*?)\)\]", printout).group(1)
        params = parse_instance_fields(inst)
        actions = {}
        for mt in re.finditer(r"^\s+(\d+): (\{.*?\}),?$", printout, flags=re.M):
            row = ast.literal_eval(mt.group(2))
            actions[int(mt.group(1))] = {k: row[k] for k in ("name", "n_root", "win_flag", "n", "n_wins", "q", "ucb")}
        best = ast.literal_eval(re.search(r"^\s+best: (\{.*?\})$", printout, flags=re.M).group(1))
        trees = ast.literal_eval(re.search(r"^\s+trees: (\{.*?\})$", printout, flags=re.M).group(1))
        examples[name] = {
            "source": "README.md, " + title[3:],
            "board_rows": rows, "turn": turn, "params": params,
            "per_state_memory": int(re.search(r"per_state_memory: (\d+) B", printout).group(1)),
            "max_tree_size": int(re.search(r"calculated max_tree_size: (\d+)", printout).group(1)),
            "steps": int(re.search(r"^\s+steps: (\d+),", printout, flags=re.M).group(1)),
            "playouts": int(re.search(r"^\s+playouts: (\d+),", printout, flags=re.M).group(1)),
            "rows_elided": re.search(r"^\s+\.\.\.$", printout, flags=re.M) is not None,
            "actions": actions, "best": best, "trees": trees,
        }
    json.dump(examples, open(out, "w"), indent=1)


def parse_instance_fields(inst):
    """'search_time_limit=5.0, ..., variant='acp_prodigal', ..., seed: 0' (MCTSNC.__str__, src/mctsnc.py:305) -> dict."""
    out = {}
    for item in inst.split(", "):
        key, value = re.split(r"=|: ", item, maxsplit=1)
        out[key] = value.strip("'") if value.startswith("'") else ("inf" if value == "inf" else float(value) if "." in value else int(value))
    return out


if __name__ == "__main__":
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    for variant in ("ocp_thrifty", "acp_thrifty"):
        condense_dump(os.path.join(ref, "extras", f"mctsnc_{variant}_c4_1000steps.json"),
                      os.path.join(HERE, f"dump_{variant}_c4_1000steps.npz"))
    condense_archives(ref, os.path.join(HERE, "archive_games.json"))
    condense_whole_experiment(ref, os.path.join(HERE, "north_star_experiment.json.gz"))
    condense_readme(ref, os.path.join(HERE, "readme_examples.json"))
    print("fixtures written to", HERE)
