"""NF4 linears on the device and the uploaded weights of a model
(``gpu/decodev2/linear.py:46-235``).

``nf4_linear`` takes HF-style rows ``[N, K]`` and returns ``[N, M]``: one row goes
to the GEMV, more rows go to the MFMA GEMM in chunks of at most 32 columns.
There is no CPU path."""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from ..nf4 import LIVE_MAX_N, nf4_gemm, nf4_gemv, nf4_quantize
from ..nf4.plan import k_pad
from .embed import PackedEmbed
from .plan import ArchSpec
from .synth import Nf4Matrix, SynthLayer, SynthModel

__all__ = ["DeviceLinear", "DeviceLayer", "DeviceWeights", "nf4_linear", "internlm_row_order"]


@dataclass
class DeviceLinear:
    packed: torch.Tensor
    scale: torch.Tensor
    M: int
    K: int
    K_pad: int
    bias: torch.Tensor | None = None

    @classmethod
    def from_nf4(cls, mat: Nf4Matrix, device, dtype: torch.dtype = torch.bfloat16,
                 row_order: np.ndarray | None = None) -> "DeviceLinear":
        packed = np.ascontiguousarray(mat.packed)
        scale = np.ascontiguousarray(mat.scale)
        bias = mat.bias
        if row_order is not None:
            packed, scale = packed[row_order], scale[row_order]
            bias = None if bias is None else bias[row_order]
        return cls(
            packed=torch.from_numpy(np.ascontiguousarray(packed)).to(device=device, dtype=torch.uint8),
            scale=torch.from_numpy(np.ascontiguousarray(scale).view(np.float16)).to(device=device),
            M=mat.M, K=mat.K, K_pad=mat.K_pad,
            bias=None if bias is None else torch.from_numpy(np.ascontiguousarray(bias)).to(
                device=device, dtype=dtype),
        )

    @classmethod
    def random(cls, m: int, k: int, *, generator: torch.Generator, sigma: float = 0.02,
               bias: bool = False) -> "DeviceLinear":
        """W ~ N(0, sigma) drawn and quantised on the GPU (weights at model scale)."""
        dev = generator.device
        w = torch.randn((m, k), generator=generator, device=dev, dtype=torch.float32) * sigma
        packed, scale = nf4_quantize(w)
        b = None
        if bias:
            b = (torch.randn(m, generator=generator, device=dev, dtype=torch.float32) * sigma).to(
                torch.bfloat16)
        return cls(packed, scale, m, k, k_pad(k), b)

    @property
    def nbytes(self) -> int:
        return self.packed.numel() + 2 * self.scale.numel()


def internlm_row_order(spec: ArchSpec) -> np.ndarray:
    """Row permutation that turns InternLM2's fused wqkv (per KV head: its query
    heads, then K, then V; ``gpu/loop/generate.py:73-89``) into ``[Q | K | V]``
    blocks, so one GEMV leaves q, k and v contiguous and no copy is needed."""
    hd, rep = spec.head_dim, spec.n_rep
    rows = np.arange(spec.wqkv_out).reshape(spec.n_kv, rep + 2, hd)
    q = rows[:, :rep, :].reshape(-1)
    k = rows[:, rep, :].reshape(-1)
    v = rows[:, rep + 1, :].reshape(-1)
    return np.concatenate([q, k, v])


def nf4_linear(mat: DeviceLinear, x: torch.Tensor) -> torch.Tensor:
    """``x`` is ``[N, K]`` bf16 on the GPU -> ``[N, M]``."""
    if x.shape[-1] != mat.K:
        raise ValueError(f"x K={x.shape[-1]} != {mat.K}")
    if x.device.type != "cuda":
        raise RuntimeError("nf4_linear: x must be on the GPU (there is no CPU path)")
    row = x.reshape(-1, mat.K)
    n = int(row.size(0))
    if n == 1:
        y = nf4_gemv(mat.packed, mat.scale, row.reshape(mat.K), mat.M, mat.K, mat.K_pad).view(1, mat.M)
    else:
        outs = []
        for lo in range(0, n, LIVE_MAX_N):
            xk = row[lo:lo + LIVE_MAX_N].t().contiguous()  # [K, n] token index fastest
            col = nf4_gemm(mat.packed, mat.scale, xk, mat.M, mat.K, mat.K_pad)
            outs.append(col.t())
        y = outs[0].contiguous() if len(outs) == 1 else torch.cat(outs, dim=0)
    if y.dtype != x.dtype:
        y = y.to(dtype=x.dtype)
    if mat.bias is not None:
        y = y + mat.bias.to(dtype=y.dtype)
    return y


@dataclass
class DeviceLayer:
    norm1: torch.Tensor
    norm2: torch.Tensor
    q: DeviceLinear | None
    k: DeviceLinear | None
    v: DeviceLinear | None
    wqkv: DeviceLinear | None  # rows already in [Q | K | V] order
    o: DeviceLinear
    gate: DeviceLinear
    up: DeviceLinear
    down: DeviceLinear


@dataclass
class DeviceWeights:
    spec: ArchSpec
    embed: torch.Tensor | PackedEmbed
    final_norm: torch.Tensor
    lm_head: DeviceLinear
    layers: list[DeviceLayer]

    @property
    def nbytes(self) -> int:
        n = self.lm_head.nbytes
        for ly in self.layers:
            for m in (ly.q, ly.k, ly.v, ly.wqkv, ly.o, ly.gate, ly.up, ly.down):
                if m is not None:
                    n += m.nbytes
        return n

    @classmethod
    def from_synth(cls, model: SynthModel, device="cuda",
                   dtype: torch.dtype = torch.bfloat16) -> "DeviceWeights":
        device = torch.device(device)
        spec = model.spec
        order = internlm_row_order(spec) if spec.family == "internlm_gqa" else None

        def up(m: Nf4Matrix | None, row_order=None):
            return None if m is None else DeviceLinear.from_nf4(m, device, dtype, row_order)

        def vec(a: np.ndarray) -> torch.Tensor:
            return torch.from_numpy(np.ascontiguousarray(a)).to(device=device, dtype=dtype)

        def layer(ly: SynthLayer) -> DeviceLayer:
            return DeviceLayer(vec(ly.norm1), vec(ly.norm2), up(ly.q), up(ly.k), up(ly.v),
                               up(ly.wqkv, order), up(ly.o), up(ly.gate), up(ly.up), up(ly.down))

        embed: torch.Tensor | PackedEmbed
        if model.embed_nf4 is not None:
            e = DeviceLinear.from_nf4(model.embed_nf4, device, dtype)
            embed = PackedEmbed(e.packed, e.scale, spec.vocab, spec.hidden)
        else:
            embed = vec(model.embed)
        return cls(spec, embed, vec(model.final_norm), up(model.lm_head),
                   [layer(ly) for ly in model.layers])

    @classmethod
    def random(cls, spec: ArchSpec, seed: int, device="cuda", *, sigma: float = 0.02,
               packed_embed: bool = True) -> "DeviceWeights":
        """Random-init weights of ``spec`` created on the GPU: every linear and the
        embedding rows NF4 group-64, norms 1 + small noise."""
        g = torch.Generator(device=device)
        g.manual_seed(int(seed))
        h, kv, f = spec.hidden, spec.kv_dim, spec.intermediate

        def lin(m, k, bias=False):
            return DeviceLinear.random(m, k, generator=g, sigma=sigma, bias=bias)

        def norm():
            return (1.0 + 0.05 * torch.randn(h, generator=g, device=device)).to(torch.bfloat16)

        layers = []
        for _ in range(spec.n_layers):
            if spec.family == "llama_swiglu":
                q, k, v, wqkv = lin(h, h, spec.qkv_bias), lin(kv, h, spec.qkv_bias), lin(kv, h, spec.qkv_bias), None
            else:
                q = k = v = None
                wqkv = lin(spec.wqkv_out, h)
            layers.append(DeviceLayer(norm(), norm(), q, k, v, wqkv, lin(h, h), lin(f, h), lin(f, h),
                                      lin(h, f)))
        if packed_embed:
            e = DeviceLinear.random(spec.vocab, h, generator=g, sigma=0.5)
            embed = PackedEmbed(e.packed, e.scale, spec.vocab, h)
        else:
            embed = (torch.randn((spec.vocab, h), generator=g, device=device) * 0.5).to(torch.bfloat16)
        return cls(spec, embed, norm(), lin(spec.vocab, h), layers)
