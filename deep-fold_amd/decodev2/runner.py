"""Greedy runner (operator surface of ``gpu/decodev2/runner.py:17-81``): the prompt goes
through chunked prefill, decode steps feed themselves on the GPU and the host only reads
the ids it returns.

A prompt is cut into windows of at most the chunk width; every window writes its K/V rows
at its own slots, and only the last one computes logits (the next id comes from them).
Two prefill paths take the same windows: the feature-major launches of ``ChunkPrefill``
when the caller passes one, otherwise the token-major sequence of ``forward_prefill``.
"""

from __future__ import annotations

from collections.abc import Callable, Iterator, Sequence

import torch

from .linear import DeviceWeights
from .prefill import ChunkPrefill, forward_prefill, prefill_chunk_width
from .state import DecodeState
from .step import greedy_decode

__all__ = ["consume_prompt", "generate"]


def _windows(n_tokens: int, width: int) -> Iterator[tuple[int, int, bool]]:
    """(first, past-the-last, is-final) of each prefill window over ``n_tokens`` ids."""
    first = 0
    while first < n_tokens:
        past = min(n_tokens, first + width)
        yield first, past, past == n_tokens
        first = past


def _window_width(state: DecodeState, chunk: int | None, prefill: ChunkPrefill | None) -> int:
    if prefill is None:
        return prefill_chunk_width(state, chunk)
    if chunk is None:
        return prefill.width            # the launches' own, wider windows
    return max(1, min(int(chunk), prefill.MAX_WIDTH))


def consume_prompt(state: DecodeState, weights: DeviceWeights, token_ids: Sequence[int], *,
                   chunk: int | None = None, start: int = 0,
                   prefill: ChunkPrefill | None = None) -> None:
    """Write K/V for ``token_ids`` into slots ``start ..`` and leave the id that follows
    them in ``state.next_token``.  ``start == 0`` is a cold prompt (after ``reset``); a
    positive ``start`` appends a suffix behind a prefix that is already in the cache."""
    ids = [int(t) for t in token_ids]
    if len(ids) == 0:
        raise ValueError("prompt must be non-empty")
    slot0 = int(start)
    if slot0 < 0:
        raise ValueError(f"start {slot0} is negative")
    if slot0 + len(ids) > state.spec.max_seq:
        raise ValueError(f"prompt {slot0}+{len(ids)} exceeds max_seq={state.spec.max_seq}")
    on_device = torch.as_tensor(ids, dtype=torch.long).to(state.device)
    for first, past, final in _windows(len(ids), _window_width(state, chunk, prefill)):
        window = on_device[first:past]
        if prefill is None:
            forward_prefill(state, weights, window, start=slot0 + first, logits=final)
        else:
            prefill.run(window, slot0 + first, logits=final)


def generate(state: DecodeState, weights: DeviceWeights, prompt_ids: Sequence[int], n_new: int, *,
             step: Callable[[DecodeState, DeviceWeights], None] | None = None,
             ignore_eos: bool = False, chunk: int | None = None,
             prefill: ChunkPrefill | None = None) -> list[int]:
    """Up to ``n_new`` new ids as a host list.  ``step`` takes one decode step: the default
    is ``greedy_decode``; a recorded ``GreedyGraph`` has the same call shape.

    The first id comes out of the prefill's logits.  Each later id is the token a step has
    just committed on the device; the step itself raises ``finished`` when that id is the
    end-of-sequence id, and the host only looks at the flag."""
    consume_prompt(state, weights, prompt_ids, chunk=chunk, prefill=prefill)
    take_step = greedy_decode if step is None else step
    wanted = int(n_new)
    produced = [int(state.next_token.item())]
    stop_on_eos = not ignore_eos
    if stop_on_eos and produced[0] == int(state.spec.eos_id):
        state.finished.fill_(1)
        return produced
    state.token.copy_(state.next_token)     # the prefill does not commit; the steps do
    while len(produced) < wanted:
        take_step(state, weights)
        produced.append(int(state.token.item()))
        if stop_on_eos and bool(state.finished.item()):
            break
    return produced
