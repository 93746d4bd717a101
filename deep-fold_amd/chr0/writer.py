"""CHR0 v1 writer for already-encoded tensors (``docs/spec/chr0.md`` sections 2.1-2.3, 3.3,
3.4, 6.1).  The reference writes ``.chr`` files from its Go compressor (``internal/chr0``);
this one exists so that synthetic models and test fixtures can be put on disk in the same
bytes, and it is checked against the specification's byte-level header example."""

from __future__ import annotations

import json
import os
import struct
from collections.abc import Mapping, Sequence
from dataclasses import dataclass

from .errors import Chr0Error, CodecError, HeaderError
from .header import (KINDS, LINEAR_KINDS, MAX_HEADER_BYTES, NF4_GROUP_SIZE, VQ_GROUP_SIZE, align64,
                     blob_sizes, layer_of)

__all__ = ["TensorEntry", "kind_of", "chr_name", "plan_layout", "write_chr"]

_NORM_LAST = frozenset((
    "norm", "input_layernorm", "post_attention_layernorm", "post_feedforward_layernorm",
    "pre_feedforward_layernorm", "final_layernorm", "final_norm", "attention_norm", "ffn_norm",
    "rms_norm", "q_norm", "k_norm", "ln_f", "ln_1", "ln_2", "ln_3"))
_KIND_BY_LAST = {
    "q_proj": "q", "k_proj": "k", "v_proj": "v", "o_proj": "o", "wo": "o", "wqkv": "qkv",
    "gate_proj": "gate", "up_proj": "up", "down_proj": "down", "w1": "gate", "w3": "up",
    "w2": "down", "embed_tokens": "embed", "wte": "embed", "lm_head": "lm_head"}
_BLOB_ORDER = {"bf16": ("data",), "nf4": ("data", "scale"), "int4": ("data", "scale", "zero"),
               "vq": ("codebook", "index")}


def chr_name(hf_name: str) -> str:
    """HF parameter name -> CHR0 name: one trailing ``.weight`` is dropped."""
    return hf_name[:-len(".weight")] if hf_name.endswith(".weight") else hf_name


def kind_of(name: str) -> str:
    """Seat of a CHR0 name, decided by its last dotted component (a ``.bias`` suffix
    is looked through)."""
    base = name[:-len(".bias")] if name.endswith(".bias") else name
    last = base.rsplit(".", 1)[-1]
    if last in _KIND_BY_LAST:
        return _KIND_BY_LAST[last]
    if last in _NORM_LAST or any(s in last for s in ("layernorm", "layer_norm", "rmsnorm")):
        return "norm"
    return "other"


@dataclass(frozen=True)
class TensorEntry:
    """One tensor to write: its blobs are final bytes (NF4 nibbles, fp16/bf16 little-endian)."""

    name: str
    codec: str
    shape: tuple[int, ...]
    blobs: Mapping[str, bytes | bytearray | memoryview]
    kind: str | None = None  # default: kind_of(name)


def _tensor_json(e: TensorEntry, kind: str, ranges: Mapping[str, tuple[int, int]]) -> dict:
    out: dict = {}
    layer = layer_of(e.name)
    if layer is not None:
        out["layer"] = layer
    out["kind"] = kind
    out["codec"] = e.codec
    out["shape"] = list(e.shape)
    if e.codec in ("nf4", "int4"):
        out["group_size"] = NF4_GROUP_SIZE
    elif e.codec == "vq":
        out["group_size"] = VQ_GROUP_SIZE
        out["n_codebooks"] = 2
        out["codebook_bits"] = 8
    for key in ("data", "scale", "zero", "codebook", "index"):
        if key in ranges:
            out[key] = list(ranges[key])
    return out


def plan_layout(entries: Sequence[TensorEntry], root: Mapping[str, object]) -> tuple[bytes, dict]:
    """Header JSON and ``{name: {key: (start, end)}}``.  Offsets sit inside the JSON whose
    length moves the offsets, so the pair is iterated until the length stops changing."""
    sizes = {}
    kinds = {}
    for e in entries:
        if e.name in sizes:
            raise HeaderError(f"tensor {e.name!r} given twice")
        kind = e.kind or kind_of(e.name)
        if kind not in KINDS:
            raise HeaderError(f"{e.name}: unknown kind {kind!r}")
        if e.codec not in _BLOB_ORDER:
            raise CodecError(f"{e.name}: unknown codec {e.codec!r}")
        if e.codec != "bf16" and (kind not in LINEAR_KINDS or e.name.endswith(".bias")):
            raise CodecError(f"{e.name}: kind {kind} / bias tensors are bf16 only")
        want = blob_sizes(e.codec, tuple(e.shape))
        keys = [k for k in _BLOB_ORDER[e.codec] if k in e.blobs]
        if set(keys) != set(e.blobs) or any(k not in e.blobs for k in want if k != "zero"):
            raise CodecError(f"{e.name}: codec {e.codec} wants blobs {sorted(want)}, got {sorted(e.blobs)}")
        for k in keys:
            if len(e.blobs[k]) != want[k]:
                raise Chr0Error(f"{e.name}.{k}: {len(e.blobs[k])} bytes, shape and codec give {want[k]}")
        sizes[e.name] = [(k, want[k]) for k in keys]
        kinds[e.name] = kind
    if not entries:
        raise HeaderError("no tensors")
    n = 0
    for _ in range(8):
        pos = align64(8 + n)
        ranges: dict[str, dict[str, tuple[int, int]]] = {}
        for e in entries:
            ranges[e.name] = {}
            for key, nbytes in sizes[e.name]:
                ranges[e.name][key] = (pos, pos + nbytes)
                pos = align64(pos + nbytes)
        doc = dict(root)
        by_name = {e.name: e for e in entries}
        doc["tensors"] = {name: _tensor_json(by_name[name], kinds[name], ranges[name])
                          for name in sorted(by_name, key=lambda s: s.encode("utf-8"))}
        text = json.dumps(doc, separators=(",", ":"), ensure_ascii=False).encode("utf-8")
        if len(text) == n:
            return text, ranges
        n = len(text)
        if n > MAX_HEADER_BYTES:
            raise HeaderError(f"header_too_large: {n} bytes")
    raise HeaderError("header_not_stable")


def write_chr(path: str | os.PathLike, entries: Sequence[TensorEntry], *, arch: str,
              hidden_size: int, intermediate_size: int, num_layers: int, vocab_size: int) -> int:
    """Write ``entries`` (blobs land in the order given) and return the file size.  The
    file appears under its name only when complete."""
    path = os.fspath(path)
    root = {"magic": "CHR0", "version": 1, "arch": str(arch), "hidden_size": int(hidden_size),
            "intermediate_size": int(intermediate_size), "num_layers": int(num_layers),
            "vocab_size": int(vocab_size), "tile": {"row": 64, "col_group": 8}}
    text, ranges = plan_layout(entries, root)
    part = path + ".part"
    try:
        with open(part, "wb") as f:
            f.write(struct.pack("<Q", len(text)))
            f.write(text)
            pos = 8 + len(text)
            for e in entries:
                for key, (start, end) in ranges[e.name].items():
                    f.write(b"\0" * (start - pos))
                    f.write(e.blobs[key])
                    pos = end
            f.write(b"\0" * (align64(pos) - pos))
            size = align64(pos)
        os.replace(part, path)
    except BaseException:
        if os.path.exists(part):
            os.remove(part)
        raise
    return size
