"""Chunked prompt prefill (``gpu/decodev2/prefill.py:26-141``): at most 32 prompt
positions per pass, linears on the MFMA GEMM, never captured into the graph."""

from __future__ import annotations

import torch

from ..nf4 import LIVE_MAX_N
from .embed import gather_embed
from .linear import DeviceWeights, nf4_linear
from .ops import causal_attend, rms, split_qkv, swiglu
from .rope import apply_rope_torch
from .state import DecodeState

__all__ = ["forward_prefill", "prefill_chunk_width"]


def prefill_chunk_width(state: DecodeState, chunk: int | None = None) -> int:
    cap = min(int(LIVE_MAX_N), int(state.spec.max_seq))
    return cap if chunk is None else max(1, min(int(chunk), cap))


def forward_prefill(state: DecodeState, weights: DeviceWeights, token_ids: torch.Tensor, start: int,
                    *, logits: bool = True) -> None:
    """Teacher-force ``token_ids`` into KV slots ``start..start+n-1``.  ``lm_head``
    runs only when ``logits`` (the last chunk), on the last row."""
    ids = token_ids.reshape(-1).to(device=state.device, dtype=torch.long)
    n = int(ids.numel())
    if n < 1:
        raise ValueError("prefill chunk must be non-empty")
    start = int(start)
    seq = start + n
    spec = state.spec
    if seq > spec.max_seq:
        raise ValueError(f"prefill {start}..{seq} exceeds max_seq={spec.max_seq}")
    x = gather_embed(weights.embed, ids)
    cos, sin = state.cos[start:seq], state.sin[start:seq]
    for li, layer in enumerate(weights.layers):
        h = rms(x, layer.norm1, spec.rms_eps)
        q, k, v = split_qkv(layer, h, spec)
        q = apply_rope_torch(q, cos, sin)
        k = apply_rope_torch(k, cos, sin)
        state.kv.write_range(li, start, k, v)
        k_all, v_all = state.kv.view(li, seq)
        attn = causal_attend(q, k_all, v_all, spec, start)
        x = x + nf4_linear(layer.o, attn)
        h = rms(x, layer.norm2, spec.rms_eps)
        x = x + nf4_linear(layer.down, swiglu(nf4_linear(layer.gate, h), nf4_linear(layer.up, h)))
    state.position.fill_(seq)
    state.valid_len.fill_(seq)
    if not logits:
        return
    hidden = rms(x[-1:], weights.final_norm, spec.rms_eps)
    state.arena.logits.copy_(nf4_linear(weights.lm_head, hidden).reshape(1, -1))
    state.pick_next(commit=False)
