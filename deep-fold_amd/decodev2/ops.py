"""Token-parallel glue of the chunked prefill, in stock torch ops as in the
reference (``gpu/decodev2/ops.py:18-44``, ``gpu/decodev2/prefill.py:58-92``): only
the linears are custom kernels there, and here."""

from __future__ import annotations

import torch
import torch.nn.functional as F

from .linear import DeviceLayer, nf4_linear
from .plan import ArchSpec

__all__ = ["rms", "swiglu", "split_qkv", "causal_attend"]


def rms(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return F.rms_norm(x, w.shape, w, eps)


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    return F.silu(gate) * up


def split_qkv(layer: DeviceLayer, h: torch.Tensor, spec: ArchSpec):
    n = int(h.shape[0])
    if layer.wqkv is not None:
        y = nf4_linear(layer.wqkv, h)  # rows are already [Q | K | V]
        q, k, v = torch.split(y, [spec.q_dim, spec.kv_dim, spec.kv_dim], dim=-1)
    else:
        q, k, v = nf4_linear(layer.q, h), nf4_linear(layer.k, h), nf4_linear(layer.v, h)
    return (q.reshape(n, spec.n_q, spec.head_dim), k.reshape(n, spec.n_kv, spec.head_dim),
            v.reshape(n, spec.n_kv, spec.head_dim))


def causal_attend(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, spec: ArchSpec, start: int) -> torch.Tensor:
    """``q`` is ``[n, n_q, hd]`` at positions ``start..start+n-1``; ``k``/``v`` are
    ``[1, n_kv, seq, hd]`` with ``seq = start + n``.  Query i sees keys 0..start+i."""
    n = int(q.shape[0])
    seq = int(k.shape[2])
    q_pos = torch.arange(start, start + n, device=q.device).unsqueeze(1)
    k_pos = torch.arange(seq, device=q.device).unsqueeze(0)
    mask = (k_pos <= q_pos)[None, None]
    qs = q.permute(1, 0, 2).unsqueeze(0)
    if spec.n_q != spec.n_kv:
        k = k.repeat_interleave(spec.n_rep, dim=1)
        v = v.repeat_interleave(spec.n_rep, dim=1)
    a = F.scaled_dot_product_attention(qs, k, v, attn_mask=mask, scale=spec.attn_scale)
    return a.squeeze(0).permute(1, 0, 2).reshape(n, spec.q_dim)
