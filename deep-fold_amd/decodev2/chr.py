"""A decoder's weights to and from a CHR0 ``.chr`` file.

``weights_from_chr`` fills the same ``DeviceLinear`` seats ``DeviceWeights.from_synth`` fills,
straight from the file's byte ranges (no dequantisation, no HF modules); the reference
reaches those seats through its HF loader (``gpu/decodev2/linear.py:190-235``).  Tensors are
found by the header's ``kind`` and ``layer`` fields, not by a family's naming, so Llama/Qwen
(``q_proj`` ..) and InternLM2 (``wqkv``, ``wo``, ``w1/w3/w2``) files both load.
``write_synth_chr`` puts a synthetic model on disk in Llama/Qwen names."""

from __future__ import annotations

import os

import numpy as np
import torch

from .. import chr0
from .embed import PackedEmbed
from .linear import DeviceLayer, DeviceLinear, DeviceWeights, internlm_row_order
from .plan import ArchSpec
from .synth import Nf4Matrix, SynthModel

__all__ = ["weights_from_chr", "write_synth_chr"]

_NORM1 = ("input_layernorm", "attention_norm", "ln_1")
_NORM2 = ("post_attention_layernorm", "ffn_norm", "ln_2")


def _bf16_bytes(a: np.ndarray) -> bytes:
    t = torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16)
    return t.view(torch.int16).numpy().tobytes()


def _nf4_entry(name: str, m: Nf4Matrix) -> list[chr0.TensorEntry]:
    out = [chr0.TensorEntry(name, "nf4", (m.M, m.K), {
        "data": np.ascontiguousarray(m.packed, dtype=np.uint8).tobytes(),
        "scale": np.ascontiguousarray(m.scale).view(np.uint16).astype("<u2").tobytes()})]
    if m.bias is not None:
        out.append(chr0.TensorEntry(name + ".bias", "bf16", (m.M,), {"data": _bf16_bytes(m.bias)}))
    return out


def write_synth_chr(model: SynthModel, path: str | os.PathLike) -> int:
    """Write ``model`` as CHR0 v1 (codec nf4) and return the file size.  The embedding must
    be kept in NF4 rows: a file has one codec for its linear, embedding and lm_head tensors."""
    spec = model.spec
    if model.embed_nf4 is None:
        raise ValueError("build the model with packed_embed=True: a .chr file has no dense embedding")
    entries = _nf4_entry("model.embed_tokens", model.embed_nf4)
    for i, ly in enumerate(model.layers):
        pre = f"model.layers.{i}."
        entries.append(chr0.TensorEntry(pre + "input_layernorm", "bf16", (spec.hidden,),
                                        {"data": _bf16_bytes(ly.norm1)}))
        if ly.wqkv is not None:
            entries += _nf4_entry(pre + "attention.wqkv", ly.wqkv)
        else:
            entries += _nf4_entry(pre + "self_attn.q_proj", ly.q)
            entries += _nf4_entry(pre + "self_attn.k_proj", ly.k)
            entries += _nf4_entry(pre + "self_attn.v_proj", ly.v)
        entries += _nf4_entry(pre + "self_attn.o_proj", ly.o)
        entries.append(chr0.TensorEntry(pre + "post_attention_layernorm", "bf16", (spec.hidden,),
                                        {"data": _bf16_bytes(ly.norm2)}))
        entries += _nf4_entry(pre + "mlp.gate_proj", ly.gate)
        entries += _nf4_entry(pre + "mlp.up_proj", ly.up)
        entries += _nf4_entry(pre + "mlp.down_proj", ly.down)
    entries.append(chr0.TensorEntry("model.norm", "bf16", (spec.hidden,), {"data": _bf16_bytes(model.final_norm)}))
    entries += _nf4_entry("lm_head", model.lm_head)
    return chr0.write_chr(path, entries, arch=spec.family, hidden_size=spec.hidden,
                          intermediate_size=spec.intermediate, num_layers=spec.n_layers,
                          vocab_size=spec.vocab)


def weights_from_chr(path: str | os.PathLike, spec: ArchSpec, device="cuda") -> DeviceWeights:
    """Load every seat of ``spec`` from ``path``; the file's shapes must be ``spec``'s."""
    hdr = chr0.load_header(path)
    codec = chr0.quantized_codec(hdr)
    if codec != "nf4":
        raise chr0.CodecError(f"{hdr.path}: codec {codec!r}, the decoder runs nf4 files only")
    if (hdr.hidden_size, hdr.num_layers) != (spec.hidden, spec.n_layers):
        raise ValueError(f"{hdr.path}: hidden {hdr.hidden_size} x {hdr.num_layers} layers, "
                         f"spec {spec.name} has {spec.hidden} x {spec.n_layers}")
    dev = torch.device(device)
    by_seat: dict[tuple[int | None, str], list[chr0.TensorInfo]] = {}
    for t in hdr.tensors.values():
        if not t.is_bias:
            by_seat.setdefault((t.layer, t.kind), []).append(t)

    def one(layer: int | None, kind: str, shape: tuple[int, int], optional: bool = False):
        found = by_seat.get((layer, kind), [])
        if not found and optional:
            return None
        if len(found) != 1:
            raise chr0.TensorNotFoundError(f"{hdr.path}: layer {layer} has {len(found)} tensors of kind {kind}")
        if tuple(found[0].shape) != shape:
            raise ValueError(f"{found[0].name}: shape {list(found[0].shape)}, spec wants {list(shape)}")
        return found[0]

    def linear(info: chr0.TensorInfo, row_order: np.ndarray | None = None) -> DeviceLinear:
        m = chr0.materialize_nf4(hdr.path, info.name, dev, header=hdr)
        packed, scale = m.packed, m.scale
        bias = None
        if info.name + ".bias" in hdr:
            bias = chr0.read_bf16(hdr.path, info.name + ".bias", dev, header=hdr)
        if row_order is not None:
            idx = torch.from_numpy(row_order).to(dev)
            packed, scale = packed.index_select(0, idx).contiguous(), scale.index_select(0, idx).contiguous()
            bias = None if bias is None else bias.index_select(0, idx).contiguous()
        return DeviceLinear(packed, scale, m.M, m.K, m.K_pad, bias)

    def norm(layer: int | None, names: tuple[str, ...]) -> torch.Tensor:
        for t in by_seat.get((layer, "norm"), []):
            if t.name.rsplit(".", 1)[-1] in names:
                if tuple(t.shape) != (spec.hidden,):
                    raise ValueError(f"{t.name}: shape {list(t.shape)}, spec wants [{spec.hidden}]")
                return chr0.read_bf16(hdr.path, t.name, dev, header=hdr)
        raise chr0.TensorNotFoundError(f"{hdr.path}: layer {layer} has no norm named any of {names}")

    h, kv, f = spec.hidden, spec.kv_dim, spec.intermediate
    fused = spec.family == "internlm_gqa"
    order = internlm_row_order(spec) if fused else None
    layers = []
    for i in range(spec.n_layers):
        layers.append(DeviceLayer(
            norm1=norm(i, _NORM1), norm2=norm(i, _NORM2),
            q=None if fused else linear(one(i, "q", (spec.q_dim, h))),
            k=None if fused else linear(one(i, "k", (kv, h))),
            v=None if fused else linear(one(i, "v", (kv, h))),
            wqkv=linear(one(i, "qkv", (spec.wqkv_out, h)), order) if fused else None,
            o=linear(one(i, "o", (h, spec.q_dim))),
            gate=linear(one(i, "gate", (f, h))), up=linear(one(i, "up", (f, h))),
            down=linear(one(i, "down", (h, f)))))
    e = linear(one(None, "embed", (spec.vocab, h)))
    head = one(None, "lm_head", (spec.vocab, h), optional=spec.tied_embed)
    lm_head = linear(head) if head is not None else DeviceLinear(e.packed, e.scale, e.M, e.K, e.K_pad)
    return DeviceWeights(spec, PackedEmbed(e.packed, e.scale, spec.vocab, h), norm(None, ("norm",)),
                         lm_head, layers)
