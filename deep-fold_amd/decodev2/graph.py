"""One greedy step as a HIP graph (operator surface of ``gpu/decodev2/graph.py:16-55``).

Token, position, KV length, next id and the finished flag are device scalars that the
step's kernels read and update themselves, so a single recording serves every position:
replaying it *is* taking a step.  Recording does not take one.  The dry runs that precede
the capture (first-launch attribute calls and allocator growth must not land inside it)
and the capture pass itself all start from the caller's scalars, which are put back after
each of them; the only trace left is a K/V row at ``position``, past ``valid_len``, which
the next real step overwrites.
"""

from __future__ import annotations

from typing import Iterable

import torch

from .linear import DeviceWeights
from .state import DecodeState
from .step import greedy_decode

__all__ = ["GreedyGraph", "capture_greedy"]

#: the device scalars a step advances
_REGISTERS = ("token", "position", "valid_len", "next_token", "finished")


def _registers(state: DecodeState) -> Iterable[torch.Tensor]:
    return (getattr(state, name) for name in _REGISTERS)


class _Registers:
    """A copy of the step's device scalars and the way back to it (device-to-device
    copies on the current stream, no host read)."""

    def __init__(self, state: DecodeState) -> None:
        self._state = state
        self._saved = [t.clone() for t in _registers(state)]

    def put_back(self) -> None:
        for live, kept in zip(_registers(self._state), self._saved):
            live.copy_(kept)


class GreedyGraph:
    """A recorded greedy step, tied to the state and weights whose buffers it recorded."""

    def __init__(self, graph: torch.cuda.CUDAGraph, state: DecodeState, weights: DeviceWeights) -> None:
        self.graph = graph
        self.state = state
        self.weights = weights
        self.replays = 0

    def replay(self) -> None:
        self.replays += 1
        self.graph.replay()

    def __call__(self, state: DecodeState, weights: DeviceWeights) -> None:
        """Same call shape as ``greedy_decode(state, weights)``, so a runner can take either;
        any other state or weights than the recorded ones is an error, not a silent replay
        on the wrong buffers."""
        if state is not self.state:
            raise RuntimeError("this graph recorded another DecodeState's buffers")
        if weights is not self.weights:
            raise RuntimeError("this graph recorded another DeviceWeights' buffers")
        self.replay()


def capture_greedy(state: DecodeState, weights: DeviceWeights, *, warmup: int = 3,
                   schedule: str | None = None) -> GreedyGraph:
    """Record one ``greedy_decode(state, weights)``; ``warmup`` dry runs come first.

    The caller's token, position, KV length, next id and finished flag read the same
    after this returns as before."""
    if state.device.type != "cuda":
        raise RuntimeError("a greedy step can only be recorded on the GPU")
    dry_runs = max(1, int(warmup))
    graph = torch.cuda.CUDAGraph()
    ahead = torch.cuda.current_stream()
    side = torch.cuda.Stream()          # default priority; capture needs a non-default stream
    side.wait_stream(ahead)
    with torch.cuda.stream(side):
        kept = _Registers(state)
        for _ in range(dry_runs):
            greedy_decode(state, weights, schedule=schedule)
            kept.put_back()
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            greedy_decode(state, weights, schedule=schedule)
        kept.put_back()                 # capture runs nothing, but keep the contract explicit
    ahead.wait_stream(side)
    return GreedyGraph(graph, state, weights)
