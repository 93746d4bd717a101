"""One resident decode token (``gpu/decodev2/step.py:162-193``).

No host read, no allocation, no Python-visible sequence length: the token id,
the position and the KV length are device scalars, so the same launches serve
every position and can be captured once as a graph.

Per layer: rms -> q/k/v GEMV -> attention (RoPE and the cache write fused) ->
o GEMV accumulating into the residual -> rms -> fused SwiGLU GEMV -> down GEMV
accumulating into the residual.  Then the final norm, lm_head and a device-side
argmax that also feeds the id back.
"""

from __future__ import annotations

import torch

from ..nf4 import ATTN_SPLIT, nf4_attn, nf4_gemv, nf4_qkv, nf4_rms, nf4_swiglu
from .embed import gather_embed
from .linear import DeviceLayer, DeviceLinear, DeviceWeights
from .state import DecodeState

__all__ = ["forward_decode", "greedy_decode", "teacher_force_token"]


def _gemv_accum(mat: DeviceLinear, src: torch.Tensor, dest: torch.Tensor) -> None:
    """``dest += W @ src`` in one launch (residual added in fp32 before rounding)."""
    d = dest.view(-1)
    nf4_gemv(mat.packed, mat.scale, src.view(-1), mat.M, mat.K, mat.K_pad, d, d)
    if mat.bias is not None:
        d.add_(mat.bias)


def _qkv(state: DecodeState, layer: DeviceLayer, h: torch.Tensor):
    """q, k, v of the current token as contiguous ``[heads*hd]`` views."""
    ar = state.arena
    spec = state.spec
    if layer.wqkv is not None:
        m = layer.wqkv
        nf4_gemv(m.packed, m.scale, h.view(-1), m.M, m.K, m.K_pad, ar.qkv.view(-1),
                 None if m.bias is None else m.bias)
        flat = ar.qkv.view(-1)
        return (flat[: spec.q_dim], flat[spec.q_dim: spec.q_dim + spec.kv_dim],
                flat[spec.q_dim + spec.kv_dim:])
    q, k, v = layer.q, layer.k, layer.v
    nf4_qkv(q.packed, q.scale, k.packed, k.scale, v.packed, v.scale, h.view(-1), q.M, k.M, v.M, q.K,
            q.K_pad, ar.q.view(-1), ar.k.view(-1), ar.v.view(-1), q.bias, k.bias, v.bias)
    return ar.q.view(-1), ar.k.view(-1), ar.v.view(-1)


def forward_decode(state: DecodeState, weights: DeviceWeights, *, commit: bool = False) -> None:
    """Logits of ``state.token`` at ``state.position`` into the arena, its argmax
    into ``state.next_token``; with ``commit`` the id is fed back on the device."""
    spec = state.spec
    ar = state.arena
    n_q, n_kv, hd = spec.n_q, spec.n_kv, spec.head_dim
    gather_embed(weights.embed, state.token.reshape(1), out=ar.x)
    state.kv.mark_written(state.position)
    for li, layer in enumerate(weights.layers):
        nf4_rms(ar.x, layer.norm1, ar.h, spec.rms_eps)
        q, k, v = _qkv(state, layer, ar.h)
        kc, vc = state.kv.layer(li)
        nf4_attn(q.view(n_q, hd), kc, vc, ar.attn, state.valid_len, spec.attn_scale, ar.attn_ws,
                 ATTN_SPLIT, k.view(n_kv, hd), v.view(n_kv, hd), state.cos, state.sin,
                 state.position)
        _gemv_accum(layer.o, ar.attn, ar.x)
        nf4_rms(ar.x, layer.norm2, ar.h, spec.rms_eps)
        g, u = layer.gate, layer.up
        nf4_swiglu(g.packed, g.scale, u.packed, u.scale, ar.h.view(-1), g.M, g.K, g.K_pad,
                   ar.down_in.view(-1))
        _gemv_accum(layer.down, ar.down_in, ar.x)
    nf4_rms(ar.x, weights.final_norm, ar.h, spec.rms_eps)
    head = weights.lm_head
    nf4_gemv(head.packed, head.scale, ar.h.view(-1), head.M, head.K, head.K_pad, ar.logits.view(-1),
             None if head.bias is None else head.bias)
    state.pick_next(commit)


def greedy_decode(state: DecodeState, weights: DeviceWeights) -> None:
    forward_decode(state, weights, commit=True)


def teacher_force_token(state: DecodeState, weights: DeviceWeights, token_id: int) -> None:
    state.load_token(token_id)
    forward_decode(state, weights, commit=False)
    state.position.add_(1)
