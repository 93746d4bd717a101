"""Greedy runner (``gpu/decodev2/runner.py:17-81``): the prompt goes through the
chunked prefill, decode tokens stay on the GPU."""

from __future__ import annotations

from collections.abc import Sequence

import torch

from .linear import DeviceWeights
from .prefill import ChunkPrefill, forward_prefill, prefill_chunk_width
from .state import DecodeState
from .step import greedy_decode

__all__ = ["consume_prompt", "generate"]


def consume_prompt(state: DecodeState, weights: DeviceWeights, token_ids: Sequence[int], *,
                   chunk: int | None = None, start: int = 0,
                   prefill: ChunkPrefill | None = None) -> None:
    """Fill KV for ``token_ids`` starting at slot ``start`` (0 = a cold prompt after
    ``reset``; a positive value appends a suffix to an existing prefix).  With
    ``prefill`` the chunks go through its feature-major launches (and graphs)
    instead of the token-major torch glue."""
    if not len(token_ids):
        raise ValueError("prompt must be non-empty")
    ids = [int(t) for t in token_ids]
    n = len(ids)
    pos = int(start)
    if pos < 0:
        raise ValueError(f"start {pos} is negative")
    if pos + n > state.spec.max_seq:
        raise ValueError(f"prompt {pos}+{n} exceeds max_seq={state.spec.max_seq}")
    width = prefill_chunk_width(state, chunk)
    if prefill is not None:  # its own, wider chunks unless the caller asked for a width
        width = prefill.width if chunk is None else max(1, min(int(chunk), prefill.MAX_WIDTH))
    buf = torch.tensor(ids, dtype=torch.long, device=state.device)
    for lo in range(0, n, width):
        hi = min(lo + width, n)
        if prefill is not None:
            prefill.run(buf[lo:hi], pos + lo, logits=(hi == n))
        else:
            forward_prefill(state, weights, buf[lo:hi], start=pos + lo, logits=(hi == n))


def generate(state: DecodeState, weights: DeviceWeights, prompt_ids: Sequence[int], n_new: int, *,
             step=None, ignore_eos: bool = False, chunk: int | None = None,
             prefill: ChunkPrefill | None = None) -> list[int]:
    """Host list of new ids.  ``step`` is ``greedy_decode`` or a captured graph."""
    consume_prompt(state, weights, prompt_ids, chunk=chunk, prefill=prefill)
    decode = greedy_decode if step is None else step
    out = [int(state.next_token.item())]
    if not ignore_eos:
        if out[0] == state.spec.eos_id:
            state.finished.fill_(1)
            return out
    state.token.copy_(state.next_token)
    for _ in range(max(0, int(n_new) - 1)):
        decode(state, weights)
        out.append(int(state.token.item()))
        if not ignore_eos and int(state.finished.item()) == 1:
            break
    return out
