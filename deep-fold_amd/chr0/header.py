"""CHR0 v1 header: parse, validate, describe (``docs/spec/chr0.md`` sections 1, 2, 4.1, 7.2;
the reference reader is ``gpu/chr0/header.py:399-532``).

A ``.chr`` file is ``uint64le N``, ``N`` bytes of one compact JSON object, zero padding to a
64-byte boundary, then byte ranges ("blobs") that each start on a 64-byte boundary; every
offset counts from the start of the file.  Nothing here reads a blob or needs torch."""

from __future__ import annotations

import json
import os
import struct
from collections.abc import Iterator, Mapping
from dataclasses import dataclass
from typing import Any

from .errors import (AlignmentError, CodecError, GroupSizeError, HeaderError, OverlapError,
                     SizeMismatchError, TensorNotFoundError, TruncatedError)

__all__ = ["NF4_GROUP_SIZE", "VQ_GROUP_SIZE", "MAX_HEADER_BYTES", "KINDS", "LINEAR_KINDS", "Blob",
           "TensorInfo", "Header", "align64", "blob_sizes", "parse_header", "load_header",
           "iter_linears", "quantized_codec"]

NF4_GROUP_SIZE = 64
VQ_GROUP_SIZE = 8
MAX_HEADER_BYTES = 100_000_000
KINDS = ("q", "k", "v", "o", "qkv", "gate", "up", "down", "embed", "lm_head", "norm", "other")
#: kinds whose (non-bias) tensors carry the file's one quantised codec
LINEAR_KINDS = frozenset(KINDS[:10])

_ROOT_KEYS = ("magic", "version", "arch", "hidden_size", "intermediate_size", "num_layers",
              "vocab_size", "tile", "tensors")
_RANGE_KEYS = ("data", "scale", "zero", "codebook", "index")
_PARAM_KEYS = ("group_size", "n_codebooks", "codebook_bits")
# codec -> keys it must have, keys it may have (besides layer/kind/codec/shape)
_CODEC_FIELDS = {
    "bf16": (("data",), ()),
    "nf4": (("group_size", "data", "scale"), ()),
    "int4": (("group_size", "data", "scale"), ("zero",)),
    "vq": (("group_size", "n_codebooks", "codebook_bits", "codebook", "index"), ()),
}
_INT63 = (1 << 63) - 1


def align64(x: int) -> int:
    """Smallest multiple of 64 that is >= ``x``."""
    return (int(x) + 63) // 64 * 64


@dataclass(frozen=True)
class Blob:
    """Bytes ``[start, end)`` of the file."""

    start: int
    end: int

    @property
    def nbytes(self) -> int:
        return self.end - self.start


@dataclass(frozen=True)
class TensorInfo:
    name: str
    kind: str
    codec: str
    shape: tuple[int, ...]
    layer: int | None
    group_size: int | None
    n_codebooks: int | None
    codebook_bits: int | None
    blobs: Mapping[str, Blob]

    @property
    def M(self) -> int:  # noqa: N802
        return self.shape[0]

    @property
    def K(self) -> int:  # noqa: N802
        if len(self.shape) != 2:
            raise SizeMismatchError(f"{self.name}: a rank-{len(self.shape)} tensor has no K")
        return self.shape[1]

    @property
    def K_pad(self) -> int:  # noqa: N802
        g = self.group_size or NF4_GROUP_SIZE
        return (self.K + g - 1) // g * g

    @property
    def n_groups(self) -> int:
        return self.K_pad // (self.group_size or NF4_GROUP_SIZE)

    @property
    def is_bias(self) -> bool:
        return self.name.endswith(".bias")


@dataclass(frozen=True)
class Header:
    """A validated header; holds neither payload bytes nor an open file."""

    path: str
    header_nbytes: int
    payload_start: int
    file_size: int
    magic: str
    version: int
    arch: str
    hidden_size: int
    intermediate_size: int
    num_layers: int
    vocab_size: int
    tile_row: int
    tile_col_group: int
    tensors: Mapping[str, TensorInfo]

    def tensor(self, name: str) -> TensorInfo:
        info = self.tensors.get(name)
        if info is None:
            raise TensorNotFoundError(f"not_found: no tensor {name!r} in {self.path}")
        return info

    def __contains__(self, name: object) -> bool:
        return name in self.tensors


# ---------------------------------------------------------------------------- JSON

def _no_float(text: str):
    raise HeaderError(f"json_invalid: {text!r} is not an integer")


def _no_constant(text: str):
    raise HeaderError(f"json_invalid: constant {text!r}")


def _unique(pairs):
    seen: dict[str, Any] = {}
    for key, value in pairs:
        if key in seen:
            raise HeaderError(f"json_invalid: key {key!r} appears twice")
        seen[key] = value
    return seen


def _decode_object(raw: bytes) -> dict[str, Any]:
    if raw[:1] != b"{":
        raise HeaderError("json_invalid: the header does not start with '{'")
    try:
        text = raw.decode("utf-8", errors="strict")
    except UnicodeDecodeError as exc:
        raise HeaderError(f"json_invalid: not UTF-8 ({exc})") from None
    dec = json.JSONDecoder(object_pairs_hook=_unique, parse_float=_no_float,
                           parse_constant=_no_constant)
    try:
        obj, stop = dec.raw_decode(text)
    except json.JSONDecodeError as exc:
        raise HeaderError(f"json_invalid: {exc}") from None
    if text[stop:].strip(" \t\n\r"):
        raise HeaderError("json_invalid: bytes after the header object")
    if not isinstance(obj, dict):
        raise HeaderError("json_invalid: the header is not an object")
    return obj


def _integer(value: Any, what: str) -> int:
    if type(value) is not int:  # bool is refused too
        raise HeaderError(f"{what}: want an integer, got {type(value).__name__}")
    return value


# ---------------------------------------------------------------------------- tensors

def blob_sizes(codec: str, shape: tuple[int, ...]) -> dict[str, int]:
    """Byte length of every range a tensor of ``codec`` and logical ``shape`` owns
    (``docs/spec/chr0.md`` section 7.2); ``zero`` of int4 is listed though optional."""
    count = 1
    for dim in shape:
        count *= dim
    if codec == "bf16":
        return {"data": 2 * count}
    if len(shape) != 2:
        raise SizeMismatchError(f"codec {codec} needs a rank-2 shape, got {list(shape)}")
    rows, cols = shape
    if codec in ("nf4", "int4"):
        padded = (cols + NF4_GROUP_SIZE - 1) // NF4_GROUP_SIZE * NF4_GROUP_SIZE
        sizes = {"data": rows * padded // 2, "scale": rows * (padded // NF4_GROUP_SIZE) * 2}
        if codec == "int4":
            sizes["zero"] = sizes["scale"]
        return sizes
    if codec == "vq":
        padded = (cols + VQ_GROUP_SIZE - 1) // VQ_GROUP_SIZE * VQ_GROUP_SIZE
        return {"codebook": 2 * 256 * 8 * 2, "index": rows * (padded // VQ_GROUP_SIZE) * 2}
    raise CodecError(f"unknown codec {codec!r}")


def layer_of(name: str) -> int | None:
    """``n`` of the first ``layers.<n>`` pair of dotted components, else None."""
    parts = name.split(".")
    for here, nxt in zip(parts, parts[1:]):
        if here == "layers" and nxt.isascii() and nxt.isdigit():
            return int(nxt)
    return None


def _check_name(name: str) -> None:
    size = len(name.encode("utf-8"))
    if size < 1 or size > 1024:
        raise HeaderError(f"tensor name of {size} bytes (1..1024 allowed)")
    if any(ord(ch) < 0x20 for ch in name):
        raise HeaderError(f"tensor name {name!r} holds a control character")


def _range(name: str, key: str, value: Any, want: int, file_size: int) -> Blob:
    what = f"{name}.{key}"
    if not isinstance(value, list) or len(value) != 2:
        raise HeaderError(f"{what}: want [start, end]")
    start, end = _integer(value[0], what), _integer(value[1], what)
    if not 0 <= start < end <= _INT63:
        raise HeaderError(f"{what}: need 0 <= start < end, got [{start}, {end}]")
    if start % 64:
        raise AlignmentError(f"{what}: start {start} is not a multiple of 64")
    if end - start != want:
        raise SizeMismatchError(f"{what}: {end - start} bytes, shape and codec give {want}")
    if end > file_size:
        raise TruncatedError(f"truncated: {what} ends at {end}, the file has {file_size} bytes")
    return Blob(start, end)


def _tensor(name: str, obj: Any, num_layers: int, file_size: int) -> TensorInfo:
    _check_name(name)
    if not isinstance(obj, dict):
        raise HeaderError(f"{name}: want an object")
    for key in ("kind", "codec", "shape"):
        if key not in obj:
            raise HeaderError(f"{name}: key {key!r} is missing")
    kind, codec = obj["kind"], obj["codec"]
    if kind not in KINDS:
        raise HeaderError(f"{name}: unknown kind {kind!r}")
    if not isinstance(codec, str) or codec not in _CODEC_FIELDS:
        raise CodecError(f"{name}: unknown codec {codec!r}")
    need, may = _CODEC_FIELDS[codec]
    allowed = {"layer", "kind", "codec", "shape", *need, *may}
    for key in obj:
        if key not in allowed:
            foreign = key in _RANGE_KEYS or key in _PARAM_KEYS
            raise (CodecError if foreign else HeaderError)(f"{name}: key {key!r} does not belong to codec {codec}")
    for key in need:
        if key not in obj:
            raise CodecError(f"{name}: codec {codec} needs key {key!r}")

    raw_shape = obj["shape"]
    if not isinstance(raw_shape, list) or not 1 <= len(raw_shape) <= 2:
        raise HeaderError(f"{name}: shape must have rank 1 or 2")
    shape = tuple(_integer(d, f"{name}.shape") for d in raw_shape)
    if any(d < 1 for d in shape):
        raise HeaderError(f"{name}: shape {list(shape)} has an element below 1")

    want_layer = layer_of(name)
    layer = None
    if want_layer is None:
        if "layer" in obj:
            raise HeaderError(f"{name}: has a layer key but no layers.<n> in its name")
    else:
        if "layer" not in obj:
            raise HeaderError(f"{name}: layer key is missing")
        layer = _integer(obj["layer"], f"{name}.layer")
        if layer != want_layer or not 0 <= layer < num_layers:
            raise HeaderError(f"{name}: layer {layer} (name says {want_layer}, file has {num_layers} layers)")

    if codec != "bf16" and (kind in ("norm", "other") or name.endswith(".bias")):
        raise CodecError(f"{name}: kind {kind} / bias tensors are bf16 only, got {codec}")

    params = {key: (_integer(obj[key], f"{name}.{key}") if key in obj else None) for key in _PARAM_KEYS}
    fixed = {"nf4": NF4_GROUP_SIZE, "int4": NF4_GROUP_SIZE, "vq": VQ_GROUP_SIZE}.get(codec)
    if fixed is not None and params["group_size"] != fixed:
        raise GroupSizeError(f"{name}: group_size {params['group_size']}, codec {codec} fixes {fixed}")
    if codec == "vq" and (params["n_codebooks"] != 2 or params["codebook_bits"] != 8):
        raise CodecError(f"{name}: vq is fixed at n_codebooks 2, codebook_bits 8")

    sizes = blob_sizes(codec, shape)
    blobs = {key: _range(name, key, obj[key], sizes[key], file_size)
             for key in _RANGE_KEYS if key in obj}
    return TensorInfo(name, kind, codec, shape, layer, params["group_size"], params["n_codebooks"],
                      params["codebook_bits"], blobs)


def _no_overlap(tensors: Mapping[str, TensorInfo], payload_start: int) -> None:
    spans = sorted((b.start, b.end, f"{t.name}.{key}") for t in tensors.values()
                   for key, b in t.blobs.items())
    if spans and spans[0][0] < payload_start:
        raise OverlapError(f"{spans[0][2]} starts at {spans[0][0]}, inside the header ({payload_start} bytes)")
    for (_, end_a, name_a), (start_b, _, name_b) in zip(spans, spans[1:]):
        if start_b < end_a:
            raise OverlapError(f"{name_a} and {name_b} overlap")


def quantized_codec(header: Header) -> str | None:
    """The one codec of the file's linear, embedding and lm_head tensors (None if it has
    none); a mix, or bf16 among them, is refused (``docs/spec/chr0.md`` section 2.3)."""
    seen = {t.codec for t in header.tensors.values() if t.kind in LINEAR_KINDS and not t.is_bias}
    if not seen:
        return None
    if len(seen) > 1 or "bf16" in seen:
        raise CodecError(f"one codec per file: linear tensors use {sorted(seen)}")
    return next(iter(seen))


def parse_header(raw: bytes, *, file_size: int, path: str = "<bytes>") -> Header:
    """Validate the first ``8 + N`` bytes of a file of ``file_size`` bytes."""
    if len(raw) < 8 or file_size < 8:
        raise TruncatedError(f"truncated: {min(len(raw), file_size)} bytes, the length word alone is 8")
    (n,) = struct.unpack_from("<Q", raw, 0)
    if n < 2:
        raise HeaderError(f"header_nbytes: {n} bytes cannot hold an object")
    if n > MAX_HEADER_BYTES:
        raise HeaderError(f"header_too_large: {n} bytes (limit {MAX_HEADER_BYTES})")
    if 8 + n > file_size or 8 + n > len(raw):
        raise HeaderError(f"header_nbytes: {n} bytes of JSON do not fit a file of {file_size}")
    root = _decode_object(raw[8:8 + n])
    for key in root:
        if key not in _ROOT_KEYS:
            raise HeaderError(f"unknown root key {key!r}")
    for key in _ROOT_KEYS:
        if key not in root:
            raise HeaderError(f"root key {key!r} is missing")
    if root["magic"] != "CHR0":
        raise HeaderError(f"magic {root['magic']!r}, want 'CHR0'")
    if _integer(root["version"], "version") != 1:
        raise HeaderError(f"unsupported version {root['version']}")
    arch = root["arch"]
    if not isinstance(arch, str) or not arch:
        raise HeaderError("arch must be a non-empty string")
    dims = {key: _integer(root[key], key)
            for key in ("hidden_size", "intermediate_size", "num_layers", "vocab_size")}
    if dims["hidden_size"] < 1 or min(dims.values()) < 0:
        raise HeaderError(f"model sizes out of range: {dims}")
    tile = root["tile"]
    if not isinstance(tile, dict) or set(tile) != {"row", "col_group"}:
        raise HeaderError("tile must be {row, col_group}")
    if _integer(tile["row"], "tile.row") != 64 or _integer(tile["col_group"], "tile.col_group") != 8:
        raise HeaderError(f"tile {tile}, v1 fixes row 64, col_group 8")
    entries = root["tensors"]
    if not isinstance(entries, dict) or not entries:
        raise HeaderError("tensors must be a non-empty object")
    tensors = {name: _tensor(name, obj, dims["num_layers"], file_size) for name, obj in entries.items()}
    payload_start = align64(8 + n)
    _no_overlap(tensors, payload_start)
    header = Header(path=path, header_nbytes=n, payload_start=payload_start, file_size=file_size,
                    magic="CHR0", version=1, arch=arch, tile_row=64, tile_col_group=8,
                    tensors=tensors, **dims)
    quantized_codec(header)
    return header


def load_header(path: str | os.PathLike) -> Header:
    """Read and validate the header of ``path``; the file is opened read-only and closed."""
    path = os.fspath(path)
    with open(path, "rb") as f:
        file_size = os.fstat(f.fileno()).st_size
        word = f.read(8)
        if len(word) < 8:
            raise TruncatedError(f"truncated: {path} has {len(word)} bytes")
        (n,) = struct.unpack("<Q", word)
        body = b""
        if 2 <= n <= MAX_HEADER_BYTES and 8 + n <= file_size:
            body = f.read(n)
    return parse_header(word + body, file_size=file_size, path=path)


def iter_linears(header: Header) -> Iterator[str]:
    """Names of the NF4 matrices (weights of linear, embedding and lm_head seats), in
    blob order on disk."""
    picked = [t for t in header.tensors.values()
              if t.codec == "nf4" and t.kind in LINEAR_KINDS and not t.is_bias]
    picked.sort(key=lambda t: t.blobs["data"].start)
    for t in picked:
        yield t.name
