"""Host side of a streamed NF4 matrix (operator surface of
``gpu/host/host_image.py:31-137``): one byte arena holding the packed codes and, right
behind them, the fp16 scales, so that a matrix moves to the device as a single copy and a
slot can be viewed as (packed, scale) without touching a byte.

With a GPU present the arena is pinned memory from the moment it is allocated (these
hosts cannot pin memory that already exists); without one it is ordinary memory, which is
what the protocol tests use.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ..nf4.plan import k_pad

__all__ = ["GROUP", "HostImage", "arena_nbytes", "is_pinned", "pack_arena", "unpack_arena"]

GROUP = 64          # weights per fp16 scale
_SCALE_BYTES = 2


def _layout(m: int, pad: int) -> tuple[int, int, int]:
    """(bytes of codes, scale groups per row, bytes of scales) of an ``[m, pad]`` matrix."""
    groups = pad // GROUP
    return m * (pad // 2), groups, m * groups * _SCALE_BYTES


def arena_nbytes(m: int, k: int) -> int:
    """Bytes of codes plus scales for an ``[M, K]`` matrix."""
    codes, _, scales = _layout(int(m), k_pad(int(k)))
    return codes + scales


def is_pinned(t: torch.Tensor) -> bool:
    """Whether ``t`` is page-locked host memory (``Tensor.is_pinned`` is a method: testing
    the attribute itself is always true)."""
    return t.device.type == "cpu" and bool(t.is_pinned())


def pack_arena(packed: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """``packed [M, K_pad/2]`` u8 and ``scale [M, K_pad/64]`` f16 -> a new 1-d u8 arena,
    codes first."""
    if packed.dtype != torch.uint8:
        raise TypeError(f"packed must be uint8, got {packed.dtype}")
    if scale.dtype != torch.float16:
        raise TypeError(f"scale must be float16, got {scale.dtype}")
    if packed.ndim != 2 or scale.ndim != 2:
        raise ValueError(f"packed {tuple(packed.shape)} / scale {tuple(scale.shape)}: expected rank 2")
    m, row_bytes = packed.shape
    codes, groups, scales = _layout(m, 2 * row_bytes)
    if scale.shape[0] != m:
        raise ValueError(f"M mismatch: packed {m} vs scale {scale.shape[0]}")
    if scale.shape[1] != groups:
        raise ValueError(f"scale n_groups {scale.shape[1]} != K_pad/64 ({groups})")
    arena = torch.empty(codes + scales, dtype=torch.uint8, pin_memory=torch.cuda.is_available())
    # write through the two views the arena will later be read through
    into_codes, into_scales = unpack_arena(arena, m, 2 * row_bytes, k_pad_=2 * row_bytes)
    into_codes.copy_(packed)
    into_scales.copy_(scale)
    return arena


def unpack_arena(arena: torch.Tensor, m: int, k: int, *, k_pad_: int | None = None):
    """(packed, scale) views of ``arena``: the same storage, no copy."""
    if arena.dtype != torch.uint8 or arena.ndim != 1:
        raise TypeError(f"arena must be uint8 1d, got {arena.dtype} {tuple(arena.shape)}")
    rows = int(m)
    pad = k_pad(int(k)) if k_pad_ is None else int(k_pad_)
    codes, groups, scales = _layout(rows, pad)
    if arena.numel() != codes + scales:
        raise ValueError(f"arena {arena.numel()} bytes != packed {codes} + scale {scales}")
    packed, tail = arena.split([codes, scales])
    return packed.view(rows, pad // 2), tail.view(torch.float16).view(rows, groups)


@dataclass(frozen=True)
class HostImage:
    """One NF4 matrix on the host: codes then scales in one arena."""

    arena: torch.Tensor
    M: int
    K: int
    K_pad: int

    def _views(self):
        return unpack_arena(self.arena, self.M, self.K, k_pad_=self.K_pad)

    @property
    def packed(self) -> torch.Tensor:
        return self._views()[0]

    @property
    def scale(self) -> torch.Tensor:
        return self._views()[1]

    @property
    def nbytes(self) -> int:
        return self.arena.numel()

    @classmethod
    def from_blobs(cls, packed: torch.Tensor, scale: torch.Tensor, k: int) -> "HostImage":
        pad = 2 * int(packed.shape[1])
        if pad != k_pad(int(k)):
            raise ValueError(f"packed width {packed.shape[1]} != K_pad/2 ({k_pad(int(k)) // 2})")
        return cls(pack_arena(packed, scale), int(packed.shape[0]), int(k), pad)
