"""MCTS-NC search engine for AMD MI355X (gfx950): hand-written HIP kernels behind the reference's MCTSNC interface,
PUCT selection / backup with virtual loss behind the reference's C ABI, and the host-side game states and CPU MCTS the
reference's runners pair them with."""
from .c4 import C4  # noqa: F401
from .gomoku import Gomoku  # noqa: F401
from .mcts import MCTS, State  # noqa: F401
from .mctsnc import MCTSNC, run_batch  # noqa: F401

__all__ = ["MCTSNC", "run_batch", "MCTS", "State", "C4", "Gomoku"]
