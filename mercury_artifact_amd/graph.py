"""Replay of one rank's step as a HIP graph.

A ring step is a fixed sequence of a few dozen short launches (block kernels, merges, casts); launched
one by one, the gaps between them cost a few per cent of the step.  :class:`GraphedStep` records the
sequence once on a capture stream and replays it with a single launch.  The reference has no counterpart:
its generated code is launched eagerly (mercury/search/bench.py:42-60).

Only the launch sequence is frozen: the step reads and writes the same tensors on every replay, so new
inputs are copied into them in place before ``replay()``.
"""
from __future__ import annotations

from typing import Callable

import torch

__all__ = ["GraphedStep"]


class GraphedStep:
    """``GraphedStep(fn)`` runs ``fn()`` twice eagerly on a side stream (so that every lazy initialisation
    and allocator warm-up has happened), then captures a third run.  ``fn`` must launch on torch's current
    stream only, as all operators of this package do, and must not synchronise."""

    def __init__(self, fn: Callable[[], None], warmup: int = 2):
        if not torch.cuda.is_available():
            raise RuntimeError("GraphedStep needs a GPU")
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(warmup):
                fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            fn()

    def replay(self) -> None:
        self.graph.replay()
