"""Device slots that streamed matrices are copied into (operator surface of
``gpu/host/slots.py:28-69``).

All slots of a ring are carved out of ONE device allocation, at a stride rounded up to 256
bytes: one allocator call, addresses that stay put for the life of the ring (graphs and
kernels may keep them), and every slot start aligned for the kernels' 16-byte loads
whatever the matrix size is.  A matrix occupies the packed-then-scale prefix of its slot;
what lies behind that prefix is never read.  ``device`` may be the CPU: the ring's protocol
tests run without a GPU.  Allocate the slots before the resident weights so that a large
model cannot fragment them out of reach.
"""

from __future__ import annotations

import torch

from .host_image import arena_nbytes, unpack_arena

__all__ = ["SLOT_ALIGN", "SLOT_COUNT", "SlotPair"]

SLOT_ALIGN = 16    # what the GEMV/GEMM kernels need of a packed row's first byte
SLOT_COUNT = 2     # ping-pong: one slot under the kernel, one under the copy
_SLOT_STRIDE_ALIGN = 256


def _round_up(n: int, to: int) -> int:
    return (n + to - 1) // to * to


class SlotPair:
    """``count`` slots of ``nbytes`` each.  ``arena[i]`` is slot i as a uint8 tensor."""

    def __init__(self, nbytes: int, device: str | torch.device, count: int = SLOT_COUNT) -> None:
        self.nbytes = int(nbytes)
        self.count = int(count)
        if self.nbytes < 0:
            raise ValueError(f"SlotPair nbytes must be >= 0, got {self.nbytes}")
        if self.count < 2:
            raise ValueError(f"SlotPair count must be >= 2, got {self.count}")
        self.device = torch.device(device)
        stride = _round_up(self.nbytes, _SLOT_STRIDE_ALIGN)
        self._backing = torch.empty(max(1, stride * self.count), dtype=torch.uint8, device=self.device)
        lead = (-self._backing.data_ptr()) % SLOT_ALIGN   # CPU allocations may start anywhere
        if lead:
            self._backing = torch.empty(stride * self.count + SLOT_ALIGN, dtype=torch.uint8,
                                        device=self.device)
            lead = (-self._backing.data_ptr()) % SLOT_ALIGN
        self.arena = tuple(self._backing[lead + i * stride: lead + i * stride + self.nbytes]
                           for i in range(self.count))
        for i, slot in enumerate(self.arena):
            if self.nbytes and slot.data_ptr() % SLOT_ALIGN:
                raise RuntimeError(f"SlotPair arena[{i}] data_ptr {slot.data_ptr():#x} is not "
                                   f"{SLOT_ALIGN}-byte aligned")

    def view(self, i: int, M: int, K: int, K_pad: int):  # noqa: N803
        """(packed ``[M, K_pad/2]`` u8, scale ``[M, K_pad/64]`` f16) over the first
        ``arena_nbytes(M, K)`` bytes of slot ``i``: the same storage, no copy."""
        if not 0 <= i < self.count:
            raise IndexError(f"SlotPair.view index must be 0..{self.count - 1}, got {i}")
        need = arena_nbytes(M, K)
        if need > self.nbytes:
            raise ValueError(f"view arena_nbytes({M},{K})={need} exceeds slot {self.nbytes} bytes")
        return unpack_arena(self.arena[i][:need], int(M), int(K), k_pad_=int(K_pad))

    def __repr__(self) -> str:
        return f"SlotPair(nbytes={self.nbytes}, count={self.count}, device={self.device})"
