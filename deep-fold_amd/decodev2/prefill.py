"""Chunked prompt prefill (``gpu/decodev2/prefill.py:26-141``): at most 32 prompt
positions per pass, linears on the MFMA GEMM.

Two forms.  ``forward_prefill`` is the reference's sequence: token-major torch glue
around the GEMMs, never captured.  ``ChunkPrefill`` keeps every activation in the
GEMM's own feature-major ``[features, N]`` layout, runs the glue (RMSNorm, RoPE + cache
write, causal attention, SwiGLU, bias/residual) as library launches, and replays each
chunk width as a captured graph, so a layer costs its kernels and not the host's
dispatch."""

from __future__ import annotations

import torch

from ..nf4 import (LIVE_MAX_N, PLAN_MAX_N, dv2_add_cols, dv2_attn_chunk, dv2_gemm_qkv, dv2_gemm_swiglu,
                   dv2_rms_cols, dv2_rope_kv_cols, dv2_sq_blocks, dv2_swiglu_elems, nf4_gemm)
from .embed import gather_embed
from .linear import DeviceLinear, DeviceWeights, nf4_linear
from .ops import causal_attend, rms, split_qkv, swiglu
from .rope import apply_rope_torch
from .state import DecodeState

__all__ = ["forward_prefill", "prefill_chunk_width", "ChunkPrefill"]


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


def _gemm_cols(mat: DeviceLinear, x: torch.Tensor, residual: torch.Tensor | None = None,
               colsq: torch.Tensor | None = None):
    """``[K, N] -> [M, N]`` with the bias, if any, added per row; with ``residual`` the
    result is added to it in place.  One column (a one-token chunk) goes to the GEMV and
    takes its bias and residual from separate launches.  With ``colsq`` the return value is
    whether the launch left the result's column sums of squares there."""
    if x.size(1) >= 2:
        if colsq is not None:
            return nf4_gemm(mat.packed, mat.scale, x, mat.M, mat.K, mat.K_pad, int(PLAN_MAX_N),
                            bias=mat.bias, residual=residual, colsq=colsq)[1]
        return nf4_gemm(mat.packed, mat.scale, x, mat.M, mat.K, mat.K_pad, int(PLAN_MAX_N),
                        bias=mat.bias, residual=residual)
    y = nf4_gemm(mat.packed, mat.scale, x, mat.M, mat.K, mat.K_pad)
    if mat.bias is not None:
        dv2_add_cols(y, bias=mat.bias)
    if residual is not None:
        dv2_add_cols(residual, y)
        return False if colsq is not None else residual
    return False if colsq is not None else y


class ChunkPrefill:
    """Feature-major prefill of one request's prompt chunks.

    ``run(ids, start, logits)`` has ``forward_prefill``'s contract.  All launches of a
    chunk read the chunk's ids, its first cache slot and the prefix length of its first
    token from fixed device buffers, so one captured graph per chunk width serves every
    position (``use_graph``); without graphs the same launches are issued eagerly.

    ``width`` is the chunk ``consume_prompt`` cuts prompts into: up to 64 tokens, twice the
    reference's 32, so the weights are streamed half as often (the 33..64-column GEMM tile
    dequantises each weight once for both 32-column blocks)."""

    MAX_WIDTH = int(PLAN_MAX_N)

    def __init__(self, state: DecodeState, weights: DeviceWeights, *, use_graph: bool = True,
                 width: int | None = None) -> None:
        self.state = state
        self.weights = weights
        self.use_graph = bool(use_graph)
        dev = state.device
        spec = state.spec
        cap = min(self.MAX_WIDTH, int(spec.max_seq))
        self.width = cap if width is None else max(1, min(int(width), cap))
        self.ids = torch.zeros(self.MAX_WIDTH, dtype=torch.long, device=dev)
        self.start = torch.zeros((), dtype=torch.int64, device=dev)
        self.first_len = torch.zeros((), dtype=torch.int32, device=dev)
        self.last_hidden = torch.zeros(spec.hidden, dtype=torch.bfloat16, device=dev)
        # column sums of squares of the residual stream, left by the launch that last wrote it
        self._colsq = torch.zeros(dv2_sq_blocks(spec.hidden, self.MAX_WIDTH) * self.MAX_WIDTH,
                                  dtype=torch.float32, device=dev)
        self._graphs: dict[int, torch.cuda.CUDAGraph] = {}
        # stacked q/k/v biases for the one-launch q/k/v GEMM (zeros where a matrix has none)
        self._qkv_bias: list[torch.Tensor | None] = []
        for layer in weights.layers:
            mats = (layer.q, layer.k, layer.v)
            if layer.wqkv is not None or all(m.bias is None for m in mats):
                self._qkv_bias.append(None)
            else:
                self._qkv_bias.append(torch.cat([
                    m.bias if m.bias is not None else torch.zeros(m.M, dtype=torch.bfloat16, device=dev)
                    for m in mats]).contiguous())

    def _chunk(self, n: int) -> None:
        state, weights, spec = self.state, self.weights, self.state.spec
        x = gather_embed(weights.embed, self.ids[:n]).t().contiguous()  # [hidden, n]
        q_rows = torch.empty((n, spec.q_dim), dtype=torch.bfloat16, device=x.device)
        attn = torch.empty((spec.q_dim, n), dtype=torch.bfloat16, device=x.device)
        sq = None  # self._colsq while it holds x's sums (the embedding gather leaves none)
        for li, layer in enumerate(weights.layers):
            h = dv2_rms_cols(x, layer.norm1, spec.rms_eps, colsq=sq)
            if layer.wqkv is not None:
                y = _gemm_cols(layer.wqkv, h)  # rows are [Q | K | V]
                q, k, v = y[:spec.q_dim], y[spec.q_dim:spec.q_dim + spec.kv_dim], y[spec.q_dim + spec.kv_dim:]
            elif n >= 2:
                y = dv2_gemm_qkv(*((m.packed, m.scale, m.M) for m in (layer.q, layer.k, layer.v)), h,
                                 bias=self._qkv_bias[li])
                q, k, v = y[:spec.q_dim], y[spec.q_dim:spec.q_dim + spec.kv_dim], y[spec.q_dim + spec.kv_dim:]
            else:
                q, k, v = _gemm_cols(layer.q, h), _gemm_cols(layer.k, h), _gemm_cols(layer.v, h)
            k_cache, v_cache = state.kv.layer(li)
            dv2_rope_kv_cols(q, k, v, q_rows, k_cache, v_cache, state.cos, state.sin, self.start)
            dv2_attn_chunk(q_rows, k_cache, v_cache, attn, self.first_len, spec.attn_scale)
            sq = self._colsq if _gemm_cols(layer.o, attn, residual=x, colsq=self._colsq) else None
            h = dv2_rms_cols(x, layer.norm2, spec.rms_eps, colsq=sq)
            if n >= 2 and layer.gate.bias is None and layer.up.bias is None:
                act = dv2_gemm_swiglu((layer.gate.packed, layer.gate.scale, layer.gate.M),
                                      (layer.up.packed, layer.up.scale, layer.up.M), h)
            else:
                act = dv2_swiglu_elems(_gemm_cols(layer.gate, h), _gemm_cols(layer.up, h))
            sq = self._colsq if _gemm_cols(layer.down, act, residual=x, colsq=self._colsq) else None
        self.last_hidden.copy_(x[:, n - 1])

    def _replay(self, n: int) -> None:
        if not self.use_graph:
            self._chunk(n)
            return
        g = self._graphs.get(n)
        if g is None:
            # one eager pass first: it sizes the GEMM's dynamic LDS and warms the allocator
            self._chunk(n)
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                self._chunk(n)
            self._graphs[n] = g
            return  # the capture pass does not run; the eager pass above already did the work
        g.replay()

    def run(self, token_ids: torch.Tensor, start: int, *, logits: bool = True) -> None:
        state, spec = self.state, self.state.spec
        ids = token_ids.reshape(-1).to(device=state.device, dtype=torch.long)
        n = int(ids.numel())
        if n < 1:
            raise ValueError("prefill chunk must be non-empty")
        if n > self.MAX_WIDTH:
            raise ValueError(f"prefill chunk of {n} tokens exceeds {self.MAX_WIDTH}")
        start = int(start)
        seq = start + n
        if start < 0 or seq > spec.max_seq:
            raise ValueError(f"prefill {start}..{seq} exceeds max_seq={spec.max_seq}")
        self.ids[:n].copy_(ids)
        self.start.fill_(start)
        self.first_len.fill_(start + 1)
        self._replay(n)
        state.position.fill_(seq)
        state.valid_len.fill_(seq)
        if not logits:
            return
        hidden = rms(self.last_hidden.view(1, -1), self.weights.final_norm, spec.rms_eps)
        state.arena.logits.copy_(nf4_linear(self.weights.lm_head, hidden).reshape(1, -1))
        state.pick_next(commit=False)
