"""Replay one step of an accelerated model as a HIP graph.

A model step is a few dozen small launches (the shallow-water Runge-Kutta step: 13 fused sub-modules,
three to four kernels each); issued one by one from Python the host side costs more than the kernels.
``capture_step`` records one call of the compiled model into a HIP graph through ``torch.cuda.CUDAGraph``
and returns a function that replays it.  The reference launches every kernel from Python on every step
(python_wrapper/dynamic_replace_submodule.py:145-199); this has no counterpart there.

What makes the capture valid: the model's tensors and the wrappers' index buffers live at fixed
addresses; outputs of the fused sub-modules are allocated from the graph's private pool during capture and
keep their addresses; every library has its own scratch buffer, whose tile table is written by the
warm-up steps and only read by the captured launches when tile reuse is on.  The libraries use no memset
and no event timing inside a captured launch.
"""
from __future__ import annotations

from typing import Callable

import torch


def capture_step(compiled, warmup: int = 2) -> Callable[[], None]:
    """Run ``warmup`` ordinary steps (they advance the model), capture one more step into a graph and
    return ``replay()``, which advances the model by one step per call."""
    if not torch.cuda.is_available():
        raise RuntimeError("capture_step needs a GPU")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(max(warmup, 1)):
            compiled()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    # captured on the stream the warm-up ran on: every library keeps one scratch buffer per stream and
    # must not allocate a new one inside the capture
    with torch.cuda.graph(graph, stream=side):
        compiled()
    # the capture itself does not execute: the model is where the warm-up left it

    def replay() -> None:
        graph.replay()

    replay.graph = graph          # keeps the graph and its memory pool alive with the function
    return replay
