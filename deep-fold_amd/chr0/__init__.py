"""CHR0 ``.chr`` checkpoints: header reader, NF4 materialiser, writer
(``docs/spec/chr0.md``; reference reader ``gpu/chr0/``).  Parsing a header needs no torch."""

from __future__ import annotations

from .errors import (AlignmentError, Chr0Error, CodecError, GroupSizeError, HeaderError,
                     OverlapError, SizeMismatchError, TensorNotFoundError, TruncatedError)
from .header import (NF4_GROUP_SIZE, Blob, Header, TensorInfo, align64, blob_sizes, iter_linears,
                     load_header, parse_header, quantized_codec)
from .writer import TensorEntry, chr_name, kind_of, plan_layout, write_chr

__all__ = [
    "load_header", "parse_header", "iter_linears", "quantized_codec", "materialize_nf4", "read_bf16",
    "ChrMatrix", "Header", "TensorInfo", "Blob", "align64", "blob_sizes", "NF4_GROUP_SIZE",
    "TensorEntry", "chr_name", "kind_of", "plan_layout", "write_chr",
    "Chr0Error", "TruncatedError", "HeaderError", "AlignmentError", "SizeMismatchError",
    "OverlapError", "CodecError", "GroupSizeError", "TensorNotFoundError",
]


def __getattr__(name: str):
    if name in ("materialize_nf4", "ChrMatrix", "read_bf16"):  # these need torch
        from . import loader
        return getattr(loader, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
