"""One greedy step captured as a HIP graph (``gpu/decodev2/graph.py:16-55``).

Position and KV length are device buffers, not capture-time scalars, so a single
capture replays for every position.  The capture is bound to one state and one
set of weights."""

from __future__ import annotations

import gc

import torch

from .linear import DeviceWeights
from .state import DecodeState
from .step import greedy_decode

__all__ = ["GreedyGraph", "capture_greedy"]


class GreedyGraph:
    def __init__(self, graph: torch.cuda.CUDAGraph, state: DecodeState, weights: DeviceWeights) -> None:
        self.graph = graph
        self.state = state
        self.weights = weights

    def replay(self) -> None:
        self.graph.replay()

    def __call__(self, state: DecodeState, weights: DeviceWeights) -> None:
        if state is not self.state or weights is not self.weights:
            raise RuntimeError("replay is bound to the captured state/weights")
        self.replay()


def capture_greedy(state: DecodeState, weights: DeviceWeights, *, warmup: int = 3,
                   schedule: str | None = None) -> GreedyGraph:
    """Warm up on a side stream (so one-time work such as kernel attribute calls
    stays out of the capture), then capture one ``greedy_decode``.

    The warm-up and the capture advance the state like any other step; callers
    that need a clean start save and restore the scalars (``snapshot``/``restore``)."""
    if state.device.type != "cuda":
        raise RuntimeError("the greedy graph needs the GPU")
    stream = torch.cuda.current_stream()
    side = torch.cuda.Stream()
    side.wait_stream(stream)
    with torch.cuda.stream(side):
        for _ in range(max(1, warmup)):
            greedy_decode(state, weights, schedule=schedule)
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        graph.capture_begin()
        try:
            greedy_decode(state, weights, schedule=schedule)
        finally:
            graph.capture_end()
    stream.wait_stream(side)
    gc.collect()
    return GreedyGraph(graph, state, weights)
