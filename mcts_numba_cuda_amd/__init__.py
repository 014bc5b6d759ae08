"""MCTS-NC search engine for AMD MI355X (gfx950): hand-written HIP kernels behind the reference's MCTSNC interface."""
from .mctsnc import MCTSNC, run_batch  # noqa: F401

__all__ = ["MCTSNC", "run_batch"]
