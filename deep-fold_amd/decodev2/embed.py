"""Packed NF4 embedding rows (``gpu/decodev2/embed.py:17-94``): the gather decodes
only the requested rows, in one kernel, and never densifies the table."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ..nf4 import nf4_embed_rows

__all__ = ["PackedEmbed", "gather_embed"]


@dataclass
class PackedEmbed:
    packed: torch.Tensor
    scale: torch.Tensor
    vocab: int
    hidden: int

    @property
    def device(self) -> torch.device:
        return self.packed.device

    @property
    def shape(self) -> tuple[int, int]:
        return (self.vocab, self.hidden)

    @property
    def nbytes(self) -> int:
        return (self.packed.numel() * self.packed.element_size()
                + self.scale.numel() * self.scale.element_size())

    def gather(self, ids: torch.Tensor, *, out: torch.Tensor | None = None) -> torch.Tensor:
        return nf4_embed_rows(self.packed, self.scale, ids.reshape(-1), self.hidden, out=out)


def gather_embed(embed, ids: torch.Tensor, *, dtype: torch.dtype = torch.bfloat16,
                 out: torch.Tensor | None = None) -> torch.Tensor:
    """``[n, hidden]`` rows of a packed table or of a dense one."""
    if isinstance(embed, PackedEmbed):
        if dtype != torch.bfloat16:
            raise ValueError("packed rows decode to bf16")
        return embed.gather(ids, out=out)
    flat = ids.reshape(-1).to(device=embed.device, dtype=torch.long)
    if out is not None:
        return torch.index_select(embed, 0, flat, out=out)
    return embed.index_select(0, flat).to(dtype=dtype)
