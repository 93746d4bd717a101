"""Device arenas a streamed matrix is copied into (``gpu/host/slots.py:28-69``).

Each arena is ``nbytes`` of uint8 sized for the largest streamed matrix; a view is the
packed‖scale prefix of one matrix, the rest of the arena is never read.  Allocate the
slots before the resident weights so their addresses stay put.  ``device`` may be the
CPU: the protocol tests run without a GPU."""

from __future__ import annotations

import torch

from .host_image import arena_nbytes, unpack_arena

__all__ = ["SLOT_ALIGN", "SLOT_COUNT", "SlotPair"]

SLOT_ALIGN = 16   # the GEMV/GEMM kernels read packed rows with 16-byte loads
SLOT_COUNT = 2    # ping-pong: one slot under the kernel, one under the copy


class SlotPair:
    def __init__(self, nbytes: int, device: str | torch.device, count: int = SLOT_COUNT) -> None:
        n = int(nbytes)
        if n < 0:
            raise ValueError(f"SlotPair nbytes must be >= 0, got {n}")
        c = int(count)
        if c < 2:
            raise ValueError(f"SlotPair count must be >= 2, got {c}")
        self.nbytes = n
        self.count = c
        self.device = torch.device(device)
        self.arena = tuple(torch.empty(n, dtype=torch.uint8, device=self.device) for _ in range(c))
        for i, buf in enumerate(self.arena):
            if n > 0 and int(buf.data_ptr()) % SLOT_ALIGN != 0:
                raise RuntimeError(f"SlotPair arena[{i}] data_ptr {int(buf.data_ptr()):#x} is not "
                                   f"{SLOT_ALIGN}-byte aligned")

    def view(self, i: int, M: int, K: int, K_pad: int):  # noqa: N803
        """packed / scale views into ``arena[i][:arena_nbytes(M, K)]``."""
        if i < 0 or i >= self.count:
            raise IndexError(f"SlotPair.view index must be 0..{self.count - 1}, got {i}")
        n = arena_nbytes(M, K)
        if n > self.nbytes:
            raise ValueError(f"view arena_nbytes({M},{K})={n} exceeds slot {self.nbytes} bytes")
        return unpack_arena(self.arena[i][:n], int(M), int(K), k_pad_=int(K_pad))

    def __repr__(self) -> str:
        return f"SlotPair(nbytes={self.nbytes}, count={self.count}, device={self.device})"
