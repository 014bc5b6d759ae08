"""Seeded random configurations, engine against oracle: board sizes, variants, tree and playout counts, exploration
constants, pool sizes (down to pools that fill up within the search), root positions and step counts drawn at random,
two consecutive searches each, everything observable compared (helpers.compare_with_oracle).  The fixed tests pin
the cases that matter by name; this one sweeps the space between them."""
import numpy as np
import pytest

from helpers import compare_with_oracle, make_engine, random_c4_root, random_gomoku_root
from oracle.oracle import Oracle

pytestmark = pytest.mark.gpu

VARIANTS = ["ocp_thrifty", "ocp_prodigal", "acp_thrifty", "acp_prodigal"]


def draw_case(rng):
    game = "gomoku" if rng.random() < 0.6 else "c4"
    variant = VARIANTS[int(rng.integers(4))]
    many = rng.random() < 0.15   # many trees: the regimes in which a workgroup searches a whole tree
    T = int(rng.choice([16, 40, 100, 210, 300, 400])) if many else int(rng.choice([1, 2, 3, 5, 8]))
    P = int(rng.choice([1, 4, 16, 32, 64, 128, 256, 512]))
    if many:
        P = min(P, 128)
    ucb_c = float(rng.choice([0.0, 0.5, 2.0, 3.5]))
    seed = int(rng.integers(1000))
    device_memory = 0.5 if many else float(rng.choice([0.002, 0.05, 0.5]))
    if game == "gomoku":
        m, n = int(rng.integers(5, 17)), int(rng.integers(5, 17))
        stones = int(rng.integers(0, max(1, m * n // 3)))
        steps = int(rng.integers(3, 40)) if variant.startswith("acp") else int(rng.integers(10, 200))
        if variant.startswith("acp") and m * n > 150:
            steps = min(steps, 6)
        if many:
            steps, T = min(steps, 4 if variant.startswith("acp") else 30), min(T, 40)
        return dict(game=game, shape=(m, n), variant=variant, T=T, P=P, ucb_c=ucb_c, seed=seed, device_memory=device_memory,
                    stones=stones, steps=steps)
    while True:
        m, n = int(rng.integers(4, 12)), int(rng.integers(4, 9))
        if (m + 1) * n <= 64:
            break
    steps = int(rng.integers(5, 60)) if many else int(rng.integers(20, 600))
    return dict(game=game, shape=(m, n), variant=variant, T=T, P=P, ucb_c=ucb_c, seed=seed, device_memory=device_memory,
                stones=int(rng.integers(0, m * n // 2)), steps=steps)


def widen(rng, c):
    """Moves a Gomoku case to a board beyond 16 x 16 (sides up to 32, up to 512 cells: the engine's two wide board formats)."""
    while True:
        m, n = int(rng.integers(5, 33)), int(rng.integers(5, 33))
        if m * n <= 512 and (m > 16 or n > 16):
            break
    acp = c["variant"].startswith("acp")
    c.update(shape=(m, n), stones=int(rng.integers(0, m * n // 3)), steps=int(rng.integers(2, 5)) if acp else int(rng.integers(10, 120)),
             P=min(c["P"], 64 if acp else 256), T=min(c["T"], 8), device_memory=max(c["device_memory"], 0.05))
    return c


@pytest.mark.parametrize("block", range(5))
def test_random_configurations(block):
    """(Block 4: Gomoku on wide boards only.)"""
    rng = np.random.default_rng(1000 + block)
    for _ in range(30):
        c = draw_case(rng)
        if block == 4:
            if c["game"] != "gomoku":
                continue
            c = widen(rng, c)
        m, n = c["shape"]
        params = dict(n_trees=c["T"], n_playouts=c["P"], variant=c["variant"], device_memory=c["device_memory"], ucb_c=c["ucb_c"], seed=c["seed"])
        if c["game"] == "gomoku":
            e = make_engine(params, board_shape=(m, n), extra=0, actions=m * n, game="gomoku")
            o = Oracle("gomoku", (m, n), 0, m * n, c["T"], c["P"], c["variant"], ucb_c=c["ucb_c"], seed=c["seed"],
                       device_memory=c["device_memory"], threads=8)
            for _ in range(2):
                board, turn = random_gomoku_root(rng, m, n, c["stones"])
                compare_with_oracle(e, o, board, None, turn, c["steps"])
        else:
            e = make_engine(params, board_shape=(m, n), extra=n, actions=n)
            o = Oracle("c4", (m, n), n, n, c["T"], c["P"], c["variant"], ucb_c=c["ucb_c"], seed=c["seed"],
                       device_memory=c["device_memory"], threads=8)
            for _ in range(2):
                board, fills, turn = random_c4_root(rng, c["stones"], m, n)
                compare_with_oracle(e, o, board, fills, turn, c["steps"])
