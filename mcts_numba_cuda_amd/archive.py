"""Reads the experiment archives the reference's runner writes (src/utils.py:168-185: a zip with the stdout log of a
tournament) and replays their searches on this package's engines.

The log holds, for every search, the root table (`n`, `n_wins`, `win_flag` of every action), the step count and the
tree statistics (src/mctsnc.py:448-563, src/mcts.py:381-443), and the moves played, so every position can be
rebuilt.  The reference keeps one AI instance per side for a whole experiment and never reseeds it; replaying the
searches in their recorded order with the recorded step counts (`forced_search_steps_limit`,
src/game_runner.py:87-92) must therefore reproduce every logged number.  Connect 4 archives only.

Command line:  python -m mcts_numba_cuda_amd.archive EXPERIMENT.zip [--games N] [--cpu]
"""
import argparse
import ast
import contextlib
import io
import re
import sys
import zipfile

import numpy as np

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




def read_archive(path, n_games=None):
    """{"engines": {instance string: MCTSNC parameters}, "games": [...]} of an experiment zip."""
    z = zipfile.ZipFile(path)
    log = z.read([n for n in z.namelist() if n.endswith(".log")][0]).decode()
    games = parse_log(log, n_games if n_games is not None else 10 ** 9)
    engines = {}
    for g in games:
        for side in ("black", "white"):
            inst = parse_instance(g[side])
            if inst:
                engines[g[side]] = inst
    return {"engines": engines, "games": games}


def _mctsnc_result(ai):
    info = ai.actions_info
    actions = {int(k): (int(v["n"]), int(v["n_wins"]), int(v["win_flag"])) for k, v in info.items() if k != "best"}
    trees = ai.performance_info["trees"]
    return {"best": int(info["best"]["index"]), "n_root": int(info["best"]["n_root"]), "actions": actions,
            "tree": {k: trees[k] for k in ("mean_depth", "max_depth", "mean_size", "max_size")}}


def _mcts_result(ai):
    info = ai.root_actions_info
    actions = {int(k): (int(v["n"]), int(v["n_wins"]), int(v["win_flag"])) for k, v in info.items() if k != "best"}
    tree = ai.performance_info["tree"]
    return {"best": int(info["best"]["index"]), "n_root": int(info["best"]["n_root"]), "actions": actions,
            "tree": {k: tree[k] for k in ("n_root", "mean_depth", "max_depth", "size")}}


def _differences(ev, got):
    want_actions = {int(k): tuple(v) for k, v in ev["actions"].items()}
    out = []
    if got["actions"] != want_actions:
        out.append(f"root table {got['actions']} != {want_actions}")
    if got["best"] != ev["best"]:
        out.append(f"best action {got['best']} != {ev['best']}")
    if got["n_root"] != ev["n_root"]:
        out.append(f"n_root {got['n_root']} != {ev['n_root']}")
    want_tree = ev.get("trees") or ev.get("tree")
    for k, v in want_tree.items():
        g = got["tree"][k]
        if abs(g - v) > 1e-12 * max(1.0, abs(v)):
            out.append(f"{k} {g} != {v}")
    return out


def replay(archive, max_games=None, cpu=False, device=0, report=None):
    """Replays the MCTSNC searches of `archive` (a path or the result of read_archive) on the GPU engine, and with
    cpu=True also the searches of the CPU player on the host MCTS.  Returns (searches checked, list of mismatches);
    `report(text)` is called per search when given."""
    from . import MCTS, MCTSNC
    from .c4 import C4
    entry = read_archive(archive, max_games) if isinstance(archive, str) else archive
    ais, checked, failures = {}, 0, []
    quiet = io.StringIO()
    for gi, game in enumerate(entry["games"]):
        if max_games is not None and gi >= max_games:
            break
        state = C4()
        for ev in game["events"]:
            if ev["type"] == "move":
                state = state.take_action(ev["action"])
                continue
            inst = game[ev["side"]]
            if ev["type"] == "mctsnc":
                if inst not in ais:
                    p = entry["engines"][inst]
                    with contextlib.redirect_stdout(quiet):
                        ais[inst] = MCTSNC(C4.get_board_shape(), C4.get_extra_info_memory(), C4.get_max_actions(),
                                           n_trees=p["n_trees"], n_playouts=p["n_playouts"], variant=p["variant"],
                                           device_memory=p["device_memory"], ucb_c=p["ucb_c"], seed=p["seed"],
                                           action_index_to_name_function=C4.action_index_to_name, device=device)
                        ais[inst].init_device_side_arrays()
                with contextlib.redirect_stdout(quiet):
                    ais[inst].run(state.get_board(), state.get_extra_info(), state.get_turn(),
                                  forced_search_steps_limit=ev["steps"])
                got = _mctsnc_result(ais[inst])
            elif cpu:
                if inst not in ais:
                    m = re.search(r"vanilla=(\w+), ucb_c=([^,]+), seed: (\d+)", inst)
                    ais[inst] = MCTS(vanilla=m.group(1) == "True", ucb_c=float(m.group(2)), seed=int(m.group(3)))
                root = C4()
                root.board[:], root.column_fills[:], root.turn = state.board, state.column_fills, state.turn
                with contextlib.redirect_stdout(quiet):
                    ais[inst].run(root, forced_search_steps_limit=ev["steps"])
                got = _mcts_result(ais[inst])
            else:
                continue
            checked += 1
            diffs = _differences(ev, got)
            label = f"game {gi + 1}, search {checked} ({ev['type']}, {ev['steps']} steps)"
            if diffs:
                failures.append((label, diffs))
            if report:
                report(f"{label}: {'MISMATCH ' + '; '.join(diffs) if diffs else 'ok'}")
    return checked, failures


def main(argv=None):
    ap = argparse.ArgumentParser(description="Replay a reference experiment archive on the MI355X engine.")
    ap.add_argument("archive")
    ap.add_argument("--games", type=int, default=None, help="number of games to replay (default: all)")
    ap.add_argument("--cpu", action="store_true", help="also replay the searches of the CPU MCTS player (slow)")
    ap.add_argument("--device", type=int, default=0)
    args = ap.parse_args(argv)
    checked, failures = replay(args.archive, args.games, args.cpu, args.device, report=print)
    print(f"{checked} searches replayed, {len(failures)} mismatches")
    return 1 if failures else 0


if __name__ == "__main__":
    sys.exit(main())
