"""Replays recorded reference games (tests/golden/archive_games.json) through a search engine.

The reference keeps one MCTSNC instance per AI for a whole experiment and never reseeds it, so the
searches of an archive must be replayed in their recorded order with the recorded step counts
(reference: src/main.py:181-186, src/game_runner.py:87-92 forced_search_steps_limit).
"""
import json
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
M, N = 6, 7


def load_archives():
    with open(os.path.join(GOLDEN, "archive_games.json")) as f:
        return json.load(f)


def load_whole_experiment():
    """All 100 games of the reference's experiment with acp_prodigal 4x256 against its CPU player (moves and MCTSNC
    searches), shaped like one entry of load_archives()."""
    import gzip
    with gzip.open(os.path.join(GOLDEN, "north_star_experiment.json.gz"), "rt") as f:
        return json.load(f)


def find_archive(archives, a, b=None):
    """Key of the archive whose two AI short names are (a, b) in either order; b=None matches any."""
    for key in archives:
        names = key.split(";")[:2]
        if a in names and (b is None or b in names) and (b is not None or True):
            if b is None or set(names) == {a, b}:
                return key
    raise KeyError((a, b))


class C4Position:
    """Connect 4 position in the reference's state layout (src/c4.py:24-47): board int8[6,7] with +1 for the
    first player, column fills as extra info, turn of the player to move."""

    def __init__(self):
        self.board = np.zeros((M, N), dtype=np.int8)
        self.fills = np.zeros(N, dtype=np.int8)
        self.turn = 1

    def play(self, j):
        assert self.fills[j] < M
        self.board[M - 1 - self.fills[j], j] = self.turn
        self.fills[j] += 1
        self.turn = -self.turn


def check_search(ev, engine_result, label=""):
    """engine_result: dict with best, actions {a: (n, n_wins, win_flag)}, n_root, trees stats."""
    exp_actions = {int(k): tuple(v) for k, v in ev["actions"].items()}
    got_actions = {int(k): tuple(int(x) for x in v) for k, v in engine_result["actions"].items()}
    assert got_actions == exp_actions, f"{label}: root table differs\n got {got_actions}\n exp {exp_actions}"
    assert int(engine_result["best"]) == ev["best"], f"{label}: best action {engine_result['best']} != {ev['best']}"
    assert int(engine_result["n_root"]) == ev["n_root"], label
    tr = ev["trees"]
    got = engine_result["trees"]
    assert got["max_depth"] == tr["max_depth"] and got["max_size"] == tr["max_size"], f"{label}: {got} vs {tr}"
    assert got["mean_size"] == tr["mean_size"], f"{label}: {got} vs {tr}"
    assert abs(got["mean_depth"] - tr["mean_depth"]) <= 1e-12 * max(1.0, abs(tr["mean_depth"])), f"{label}: {got} vs {tr}"


def replay_archive(entry, make_engine, run_search, max_games=None, max_searches=None, on_search=None):
    """make_engine(params) -> engine; run_search(engine, board, fills, turn, steps) -> engine_result dict.
    Returns the number of MCTSNC searches checked."""
    engines = {}
    checked = 0
    for gi, game in enumerate(entry["games"]):
        if max_games is not None and gi >= max_games:
            break
        pos = C4Position()
        for ev in game["events"]:
            if ev["type"] == "move":
                pos.play(ev["action"])
            elif ev["type"] == "mctsnc":
                inst = game[ev["side"]]
                if inst not in engines:
                    engines[inst] = make_engine(entry["engines"][inst])
                res = run_search(engines[inst], pos.board.copy(), pos.fills.copy(), pos.turn, ev["steps"])
                check_search(ev, res, label=f"game {gi + 1} search {checked + 1} ({inst})")
                checked += 1
                if on_search:
                    on_search(checked, ev)
                if max_searches is not None and checked >= max_searches:
                    return checked
    return checked


def oracle_run_search(o, board, fills, turn, steps):
    """Runs one search on an oracle engine and shapes its output like MCTSNC._make_actions_info_* (src/mctsnc.py:496-563)."""
    o.run(board, fills, turn, steps)
    thrifty = o.variant.endswith("thrifty")
    rae = o.result("root_actions_expanded")
    root_ns, ns, ws, wf = o.result("root_ns"), o.result("actions_ns"), o.result("actions_ns_wins"), o.result("actions_win_flags")
    actions = {}
    n_root = 0
    if thrifty:
        for i in range(int(rae[-1])):
            actions[int(rae[i])] = (int(ns[i]), int(ws[i]), int(wf[i]))
            n_root = int(root_ns[i])
    else:
        for a in range(o.A):
            if root_ns[a] == 0:
                continue
            actions[a] = (int(ns[a]), int(ws[a]), int(wf[a]))
            n_root = int(root_ns[a])
    return dict(best=o.best["action"], actions=actions, n_root=n_root, trees=o.tree_stats())
