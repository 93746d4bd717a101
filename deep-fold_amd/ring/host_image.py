"""Host side of a streamed NF4 matrix: one pinned byte arena holding the packed codes
followed by the fp16 scales, so the whole matrix is a single host-to-device copy
(``gpu/host/host_image.py:31-137``).

The arena is allocated pinned from the start when a GPU is present (pinning memory
that already exists is not available on these hosts); without a GPU it is ordinary
memory, which is what the protocol tests use."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ..nf4.plan import k_pad

__all__ = ["GROUP", "HostImage", "arena_nbytes", "is_pinned", "pack_arena", "unpack_arena"]

GROUP = 64


def arena_nbytes(m: int, k: int) -> int:
    """Bytes of packed‖scale for an ``[M, K]`` matrix."""
    pad = k_pad(int(k))
    return int(m) * (pad // 2) + int(m) * (pad // GROUP) * 2


def is_pinned(t: torch.Tensor) -> bool:
    """``Tensor.is_pinned`` is a method; a bare truth test of it is always true."""
    return bool(t.is_cpu and t.is_pinned())


def _new_arena(n: int) -> torch.Tensor:
    pin = torch.cuda.is_available()
    return torch.empty(int(n), dtype=torch.uint8, pin_memory=pin)


def pack_arena(packed: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """``packed [M, K_pad/2]`` u8 and ``scale [M, K_pad/64]`` f16 -> one 1-d u8 arena."""
    if packed.dtype is not torch.uint8:
        raise TypeError(f"packed must be uint8, got {packed.dtype}")
    if scale.dtype is not torch.float16:
        raise TypeError(f"scale must be float16, got {scale.dtype}")
    if packed.dim() != 2 or scale.dim() != 2:
        raise ValueError(f"packed {tuple(packed.shape)} / scale {tuple(scale.shape)}: expected rank 2")
    m, width = int(packed.shape[0]), int(packed.shape[1])
    if int(scale.shape[0]) != m:
        raise ValueError(f"M mismatch: packed {m} vs scale {int(scale.shape[0])}")
    groups = (width * 2) // GROUP
    if int(scale.shape[1]) != groups:
        raise ValueError(f"scale n_groups {int(scale.shape[1])} != K_pad/64 ({groups})")
    code_bytes = packed.contiguous().reshape(-1).cpu()
    scale_bytes = scale.contiguous().cpu().view(torch.uint8).reshape(-1)
    arena = _new_arena(code_bytes.numel() + scale_bytes.numel())
    arena[: code_bytes.numel()].copy_(code_bytes)
    arena[code_bytes.numel():].copy_(scale_bytes)
    return arena


def unpack_arena(arena: torch.Tensor, m: int, k: int, *, k_pad_: int | None = None):
    """packed / scale views of ``arena`` (same storage, no copy)."""
    if arena.dtype is not torch.uint8 or arena.dim() != 1:
        raise TypeError(f"arena must be uint8 1d, got {arena.dtype} {tuple(arena.shape)}")
    m = int(m)
    pad = int(k_pad_) if k_pad_ is not None else k_pad(int(k))
    code_n = m * (pad // 2)
    groups = pad // GROUP
    if int(arena.numel()) != code_n + m * groups * 2:
        raise ValueError(f"arena {int(arena.numel())} bytes != packed {code_n} + scale {m * groups * 2}")
    return arena[:code_n].view(m, pad // 2), arena[code_n:].view(torch.float16).view(m, groups)


@dataclass(frozen=True)
class HostImage:
    """One NF4 matrix on the host as packed‖scale."""

    arena: torch.Tensor
    M: int
    K: int
    K_pad: int

    @property
    def packed(self) -> torch.Tensor:
        return unpack_arena(self.arena, self.M, self.K, k_pad_=self.K_pad)[0]

    @property
    def scale(self) -> torch.Tensor:
        return unpack_arena(self.arena, self.M, self.K, k_pad_=self.K_pad)[1]

    @property
    def nbytes(self) -> int:
        return int(self.arena.numel())

    @classmethod
    def from_blobs(cls, packed: torch.Tensor, scale: torch.Tensor, k: int) -> "HostImage":
        pad = int(packed.shape[1]) * 2
        if pad != k_pad(int(k)):
            raise ValueError(f"packed width {packed.shape[1]} != K_pad/2 ({k_pad(int(k)) // 2})")
        return cls(pack_arena(packed, scale), int(packed.shape[0]), int(k), pad)
