"""Preallocated activations for one decode token (``gpu/decodev2/arena.py:18-59``):
nothing on the step path allocates."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ..nf4 import ATTN_SPLIT, dv2_argmax_ws_bytes, dv2_attn_state_floats, dv2_sumsq_parts
from .plan import ArchSpec

__all__ = ["Arena"]


@dataclass
class Arena:
    spec: ArchSpec
    x: torch.Tensor
    h: torch.Tensor
    q: torch.Tensor
    k: torch.Tensor
    v: torch.Tensor
    qkv: torch.Tensor
    attn: torch.Tensor
    down_in: torch.Tensor
    logits: torch.Tensor
    attn_ws: torch.Tensor
    attn_state: torch.Tensor     # softmax states of the attention whose merge the o projection does
    argmax_ws: torch.Tensor      # per-slice candidates of the two-launch argmax
    sumsq: torch.Tensor          # sum of squares of x, in parts, from the launch that wrote x to the one that normalises it

    @classmethod
    def allocate(cls, spec: ArchSpec, *, device, dtype: torch.dtype = torch.bfloat16) -> "Arena":
        def z(*shape):
            return torch.zeros(shape, dtype=dtype, device=device)

        return cls(
            spec=spec,
            x=z(1, spec.hidden),
            h=z(1, spec.hidden),
            q=z(1, spec.n_q, spec.head_dim),
            k=z(1, spec.n_kv, spec.head_dim),
            v=z(1, spec.n_kv, spec.head_dim),
            qkv=z(1, spec.wqkv_out),
            attn=z(1, spec.q_dim),
            down_in=z(1, spec.intermediate),
            logits=z(1, spec.vocab),
            attn_ws=torch.zeros(spec.n_q * ATTN_SPLIT * (spec.head_dim + 2), dtype=torch.float32,
                                device=device),
            attn_state=torch.zeros(dv2_attn_state_floats(spec.n_q, spec.head_dim), dtype=torch.float32,
                                   device=device),
            argmax_ws=torch.zeros(dv2_argmax_ws_bytes() // 8, dtype=torch.int64, device=device),
            sumsq=torch.zeros(dv2_sumsq_parts(), dtype=torch.float32, device=device),
        )
