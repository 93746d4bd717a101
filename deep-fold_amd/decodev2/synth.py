"""Seeded synthetic NF4 transformers: no checkpoints, no files.

``build`` draws every tensor from one ``numpy.random.default_rng(seed)`` stream in
the reference's order (``gpu/decodev2/synth.py:60-99``): per layer q, k, v (or
wqkv), norm1, norm2, o, gate, up, down; then embed, final_norm, lm_head.  The
quantiser is injectable: by default the library's GPU encoder (bit-exact against
the CPU codec), so that building a model is itself a product path.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Callable

import numpy as np

from ..nf4.plan import k_pad
from .plan import ArchSpec

__all__ = ["Nf4Matrix", "SynthLayer", "SynthModel", "build", "gpu_encode"]

Encoder = Callable[[np.ndarray], "tuple[np.ndarray, np.ndarray]"]


@dataclass
class Nf4Matrix:
    packed: np.ndarray
    scale: np.ndarray
    M: int
    K: int
    K_pad: int
    bias: np.ndarray | None = None


@dataclass
class SynthLayer:
    norm1: np.ndarray
    norm2: np.ndarray
    q: Nf4Matrix | None
    k: Nf4Matrix | None
    v: Nf4Matrix | None
    wqkv: Nf4Matrix | None
    o: Nf4Matrix
    gate: Nf4Matrix
    up: Nf4Matrix
    down: Nf4Matrix


@dataclass
class SynthModel:
    spec: ArchSpec
    seed: int
    embed: np.ndarray
    final_norm: np.ndarray
    lm_head: Nf4Matrix
    layers: list[SynthLayer]
    #: packed form of ``embed`` when the model keeps its embedding rows in NF4;
    #: ``embed`` then holds exactly the values those rows decode to (as bf16)
    embed_nf4: Nf4Matrix | None = None


def gpu_encode(w: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """Quantise on the GPU with the library's encoder and bring the blobs back."""
    import torch

    from ..nf4 import nf4_quantize

    if not torch.cuda.is_available():
        raise RuntimeError("synthetic models are quantised on the GPU; no GPU is visible "
                           "(pass encode= to use another bit-exact encoder)")
    packed, scale = nf4_quantize(torch.from_numpy(np.ascontiguousarray(w, dtype=np.float32)).cuda())
    return packed.cpu().numpy(), scale.cpu().numpy()


def gpu_decode_bf16(mat: Nf4Matrix) -> np.ndarray:
    """The bf16 values (as float32) the library's row decoder gives for ``mat``."""
    import torch

    from ..nf4 import nf4_embed_rows

    packed = torch.from_numpy(np.ascontiguousarray(mat.packed)).cuda()
    scale = torch.from_numpy(np.ascontiguousarray(mat.scale).view(np.float16)).cuda()
    ids = torch.arange(mat.M, device="cuda", dtype=torch.int64)
    return nf4_embed_rows(packed, scale, ids, mat.K).float().cpu().numpy()


def build(spec: ArchSpec, seed: int, *, encode: Encoder | None = None,
          packed_embed: bool = False) -> SynthModel:
    """``packed_embed`` keeps the embedding rows in NF4 as the large checkpoints do
    (``gpu/decodev2/embed.py:17-94``); the draws are the same either way."""
    enc = gpu_encode if encode is None else encode
    rng = np.random.default_rng(int(seed))

    def matrix(m: int, k: int, sigma: float = 0.05) -> Nf4Matrix:
        w = rng.standard_normal((m, k), dtype=np.float32) * np.float32(sigma)
        packed, scale = enc(w)
        return Nf4Matrix(np.asarray(packed), np.asarray(scale), m, k, k_pad(k))

    def vector(n: int, sigma: float = 0.5) -> np.ndarray:
        return rng.standard_normal(n, dtype=np.float32) * np.float32(sigma)

    h, kv, inter = spec.hidden, spec.kv_dim, spec.intermediate
    layers: list[SynthLayer] = []
    for _ in range(spec.n_layers):
        if spec.family == "llama_swiglu":
            q, k, v, wqkv = matrix(h, h), matrix(kv, h), matrix(kv, h), None
        else:
            q = k = v = None
            wqkv = matrix(spec.wqkv_out, h)
        norm1 = vector(h)
        norm2 = vector(h)
        o = matrix(h, h)
        gate = matrix(inter, h)
        up = matrix(inter, h)
        down = matrix(h, inter)
        layers.append(SynthLayer(norm1, norm2, q, k, v, wqkv, o, gate, up, down))
    embed = vector(spec.vocab * h).reshape(spec.vocab, h)
    final_norm = vector(h)
    lm_head = matrix(spec.vocab, h)
    embed_nf4 = None
    if packed_embed:
        packed, scale = enc(embed)
        embed_nf4 = Nf4Matrix(np.asarray(packed), np.asarray(scale), spec.vocab, h, k_pad(h))
        embed = gpu_decode_bf16(embed_nf4)
    return SynthModel(spec, int(seed), embed, final_norm, lm_head, layers, embed_nf4)
