"""One resident decode token (``gpu/decodev2/step.py:162-193``).

No host read, no allocation, no Python-visible sequence length: the token id,
the position and the KV length are device scalars, so the same launches serve
every position and can be captured once as a graph.

Per layer: rms -> q/k/v GEMV -> attention (RoPE and the cache write fused) ->
o GEMV accumulating into the residual -> rms -> fused SwiGLU GEMV -> down GEMV
accumulating into the residual.  Then the final norm, lm_head and a device-side
argmax that also feeds the id back.

Two launch schedules compute that sequence:

``plain``     the reference's call sequence, eight launches per layer;
``fold_rms``  every RMSNorm runs inside the GEMV that consumes it, the merge of the
              attention splits runs inside the o projection, and the embedding
              gather also sets the KV length: five launches per layer.  A
              dependent launch costs about 5 us on an MI355X whatever it does, so
              the launch count is what this buys.  Where every launch that writes the
              residual stream can do so, it also leaves the sum of squares of what it
              wrote for the launch that normalises it (``_sumsq_handover``).
"""

from __future__ import annotations

import os

import torch

from ..nf4 import (ATTN_SPLIT, dv2_attn_parts, dv2_begin_step, dv2_gemv_attn, dv2_sumsq_ok, nf4_attn,
                   nf4_gemv, nf4_qkv, nf4_rms, nf4_swiglu)
from .embed import PackedEmbed, gather_embed
from .linear import DeviceLayer, DeviceLinear, DeviceWeights
from .state import DecodeState

__all__ = ["forward_decode", "greedy_decode", "teacher_force_token", "SCHEDULES"]


def _gemv_accum(mat: DeviceLinear, src: torch.Tensor, dest: torch.Tensor,
                sumsq_out: torch.Tensor | None = None) -> None:
    """``dest += W @ src`` in one launch (residual added in fp32 before rounding); with
    ``sumsq_out`` the launch leaves the sum of squares of the new ``dest`` (no bias then)."""
    d = dest.view(-1)
    nf4_gemv(mat.packed, mat.scale, src.view(-1), mat.M, mat.K, mat.K_pad, d, d, sumsq_out=sumsq_out)
    if mat.bias is not None:
        d.add_(mat.bias)


def _sumsq_handover(weights: DeviceWeights) -> bool:
    """Whether the folded step hands the sum of squares of the residual stream from the launch
    that writes it (prologue, o projection, down projection) to the launch that normalises it
    (q/k/v, gate/up, lm_head), which then skips its own sum over the workgroup (two barriers
    ahead of its first product: 0.7 us of a 7 us launch).  Every writer must be the last to
    touch the stream (no separate bias add) and run on a kernel that leaves the sum.
    ``CHR_DV2_SUMSQ=0`` keeps every launch summing for itself."""
    if os.environ.get("CHR_DV2_SUMSQ", "1") == "0":
        return False
    shapes = getattr(weights, "_sumsq_writers", None)
    if shapes is None:
        shapes = set()
        for layer in weights.layers:
            for mat, merges in ((layer.o, True), (layer.down, False)):
                shapes.add((mat.M, mat.K, mat.K_pad, merges, mat.bias is None))
        weights._sumsq_writers = shapes
    return all(no_bias and dv2_sumsq_ok(m, k, k_pad, merges) for m, k, k_pad, merges, no_bias in shapes)


def _qkv(state: DecodeState, layer: DeviceLayer, h: torch.Tensor, rms_w: torch.Tensor | None = None,
         sumsq_in: torch.Tensor | None = None):
    """q, k, v of the current token as contiguous ``[heads*hd]`` views; with ``rms_w``
    the GEMV normalises ``h`` itself (from the sum of squares in ``sumsq_in`` when given)."""
    ar = state.arena
    spec = state.spec
    eps = spec.rms_eps
    if layer.wqkv is not None:
        m = layer.wqkv
        nf4_gemv(m.packed, m.scale, h.view(-1), m.M, m.K, m.K_pad, ar.qkv.view(-1),
                 None if m.bias is None else m.bias, rms_w, eps, sumsq_in=sumsq_in)
        flat = ar.qkv.view(-1)
        return (flat[: spec.q_dim], flat[spec.q_dim: spec.q_dim + spec.kv_dim],
                flat[spec.q_dim + spec.kv_dim:])
    q, k, v = layer.q, layer.k, layer.v
    nf4_qkv(q.packed, q.scale, k.packed, k.scale, v.packed, v.scale, h.view(-1), q.M, k.M, v.M, q.K,
            q.K_pad, ar.q.view(-1), ar.k.view(-1), ar.v.view(-1), q.bias, k.bias, v.bias, rms_w, eps,
            sumsq_in=sumsq_in)
    return ar.q.view(-1), ar.k.view(-1), ar.v.view(-1)


SCHEDULES = ("plain", "fold_rms")
#: schedule used when the caller does not name one
DEFAULT_SCHEDULE = "fold_rms"


def _attend_into_o(state: DecodeState, li: int, layer: DeviceLayer, q, k, v,
                   sumsq_out: torch.Tensor | None = None) -> None:
    """Attention + o projection + residual as two launches: the attention workgroups (several
    per head, so a head's cache rows stream through several compute units) leave their
    softmax states, and the o GEMV merges them while it stages its activations."""
    spec = state.spec
    ar = state.arena
    n_q, n_kv, hd = spec.n_q, spec.n_kv, spec.head_dim
    kc, vc = state.kv.layer(li)
    dv2_attn_parts(q.view(n_q, hd), kc, vc, state.valid_len, spec.attn_scale, ar.attn_state,
                   k_act=k.view(n_kv, hd), v_act=v.view(n_kv, hd), cos=state.cos, sin=state.sin,
                   position=state.position)
    o = layer.o
    d = ar.x.view(-1)
    dv2_gemv_attn(o.packed, o.scale, ar.attn_state, n_q, hd, o.M, o.K, o.K_pad, d, d, sumsq_out=sumsq_out)
    if o.bias is not None:
        d.add_(o.bias)


def _attend(state: DecodeState, li: int, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> None:
    spec = state.spec
    ar = state.arena
    n_q, n_kv, hd = spec.n_q, spec.n_kv, spec.head_dim
    kc, vc = state.kv.layer(li)
    nf4_attn(q.view(n_q, hd), kc, vc, ar.attn, state.valid_len, spec.attn_scale, ar.attn_ws,
             ATTN_SPLIT, k.view(n_kv, hd), v.view(n_kv, hd), state.cos, state.sin, state.position)


def _forward_calls(state: DecodeState, weights: DeviceWeights, commit: bool, fold: bool) -> None:
    """``fold`` == False: the reference's call sequence.  ``fold`` == True: RMSNorm inside
    the consuming GEMV (the ``rms_w`` argument of the GEMV entry points,
    ``gpu/nf4/nf4_gemv.cu:264-289``), one-launch attention, one-launch step prologue."""
    spec = state.spec
    ar = state.arena
    eps = spec.rms_eps
    emb = weights.embed
    merge_in_o = fold and spec.head_dim % 8 == 0
    # sq: the parts buffer when every writer of ar.x leaves its sum of squares for the next reader
    sq = ar.sumsq if (merge_in_o and isinstance(emb, PackedEmbed) and _sumsq_handover(weights)) else None
    if fold and isinstance(emb, PackedEmbed):
        dv2_begin_step(emb.packed, emb.scale, emb.hidden, state.token, state.position,
                       state.valid_len, ar.x.view(-1), sumsq_out=sq)
    else:
        gather_embed(emb, state.token.reshape(1), out=ar.x)
        state.kv.mark_written(state.position)
    for li, layer in enumerate(weights.layers):
        if fold:
            q, k, v = _qkv(state, layer, ar.x, layer.norm1, sq)
        else:
            nf4_rms(ar.x, layer.norm1, ar.h, eps)
            q, k, v = _qkv(state, layer, ar.h)
        if merge_in_o:
            _attend_into_o(state, li, layer, q, k, v, sq)
        else:
            _attend(state, li, q, k, v)
            _gemv_accum(layer.o, ar.attn, ar.x)
        g, u = layer.gate, layer.up
        if fold:
            nf4_swiglu(g.packed, g.scale, u.packed, u.scale, ar.x.view(-1), g.M, g.K, g.K_pad,
                       ar.down_in.view(-1), layer.norm2, eps, sumsq_in=sq)
        else:
            nf4_rms(ar.x, layer.norm2, ar.h, eps)
            nf4_swiglu(g.packed, g.scale, u.packed, u.scale, ar.h.view(-1), g.M, g.K, g.K_pad,
                       ar.down_in.view(-1))
        _gemv_accum(layer.down, ar.down_in, ar.x, sq)
    head = weights.lm_head
    bias = None if head.bias is None else head.bias
    if fold:
        nf4_gemv(head.packed, head.scale, ar.x.view(-1), head.M, head.K, head.K_pad,
                 ar.logits.view(-1), bias, weights.final_norm, eps, sumsq_in=sq)
    else:
        nf4_rms(ar.x, weights.final_norm, ar.h, eps)
        nf4_gemv(head.packed, head.scale, ar.h.view(-1), head.M, head.K, head.K_pad,
                 ar.logits.view(-1), bias)
    state.pick_next(commit)


def forward_decode(state: DecodeState, weights: DeviceWeights, *, commit: bool = False,
                   schedule: str | None = None) -> None:
    """Logits of ``state.token`` at ``state.position`` into the arena, its argmax
    into ``state.next_token``; with ``commit`` the id is fed back on the device.
    ``schedule`` names the launch schedule (``SCHEDULES``; default ``DEFAULT_SCHEDULE``)."""
    if schedule is None:
        schedule = DEFAULT_SCHEDULE
    if schedule not in SCHEDULES:
        raise ValueError(f"schedule must be one of {SCHEDULES}, got {schedule!r}")
    _forward_calls(state, weights, commit, schedule == "fold_rms")


def greedy_decode(state: DecodeState, weights: DeviceWeights, *, schedule: str | None = None) -> None:
    forward_decode(state, weights, commit=True, schedule=schedule)


def teacher_force_token(state: DecodeState, weights: DeviceWeights, token_id: int) -> None:
    state.load_token(token_id)
    forward_decode(state, weights, commit=False)
    state.position.add_(1)
