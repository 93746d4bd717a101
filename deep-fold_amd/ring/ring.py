"""Host-to-device ring for NF4 matrices that live in pinned host memory and are streamed
into a few static device slots just before the kernel that reads them
(``gpu/loop/ring.py:76-423``).

Per slot ``s`` there are two events:

    copy stream : wait(gemm_done[s]) -> one packed‖scale copy into slot s -> record(copied[s])
    compute     : wait(copied[s])    -> kernel on the slot views          -> record(gemm_done[s])

so a slot is never overwritten under a kernel and a kernel never starts on a half-copied
slot.  With ``n`` slots up to ``n - 1`` copies run ahead of the compute stream.  All copies
go through one extra stream at the default priority (the copy engine is shared whatever
the number of streams); compute stays on the caller's current stream.

``ops``, ``slot_order``, ``issue_count`` and ``ahead`` record the protocol on the host, so
its order can be asserted without a GPU: with a CPU ``SlotPair`` the copies are plain
tensor copies and no events exist."""

from __future__ import annotations

import os
from collections import deque
from dataclasses import dataclass
from typing import Sequence

import torch

from .host_image import HostImage
from .slots import SlotPair

__all__ = ["CopyRing", "StreamedMatrix", "default_join_copy"]


@dataclass
class StreamedMatrix:
    """What the ring needs to know of a linear (the reference's ``Gemm`` record,
    ``gpu/loop/graph.py:383``): ``home`` is ``"host"`` for a streamed matrix (then
    ``host_image`` is set) or ``"device"`` for a resident one (then ``packed``/``scale``)."""

    name: str
    M: int
    K: int
    K_pad: int
    home: str = "device"
    host_image: HostImage | None = None
    packed: torch.Tensor | None = None
    scale: torch.Tensor | None = None

    @classmethod
    def on_host(cls, name: str, image: HostImage) -> "StreamedMatrix":
        return cls(name, image.M, image.K, image.K_pad, "host", image)


def _same(a: StreamedMatrix, b: StreamedMatrix) -> bool:
    return a is b or a.name == b.name


def default_join_copy() -> bool:
    """Whether ``bind`` also blocks the host on the copy.  Linux does not need it (the
    compute stream waits on the event); ``DEEPFOLD_COPY_JOIN=1`` turns it on."""
    return os.environ.get("DEEPFOLD_COPY_JOIN", "").strip().lower() in ("1", "true", "yes", "on")


class CopyRing:
    def __init__(self, slots: SlotPair, *, timing: bool = False,
                 n_copy_streams: int | None = None) -> None:
        self.slots = slots
        self.timing = bool(timing)
        self.n_slots = int(slots.count)
        self.max_ahead = max(1, self.n_slots - 1)
        n_cs = 1 if n_copy_streams is None else int(n_copy_streams)
        if n_cs < 1:
            raise ValueError(f"n_copy_streams must be >= 1, got {n_cs}")
        self.n_copy_streams = n_cs
        # host-visible protocol record
        self.ops: list[tuple] = []
        self.slot_order: list[int] = []
        self.issue_count = 0
        self.forward_bytes = 0
        self.forward_copy_ms = 0.0
        self.total_copies = 0
        self.total_bytes = 0
        self.total_copy_ms = 0.0
        self.total_forwards = 0
        # ring state
        self._next_slot = 0
        self._ahead = 0
        self._inflight: deque[tuple[StreamedMatrix, int]] = deque()
        self._tape: tuple[StreamedMatrix, ...] = ()
        self._tape_pos = 0
        self._bound_slot: int | None = None
        self._bound: StreamedMatrix | None = None
        self._join_copy = default_join_copy()
        self._gpu = torch.cuda.is_available() and slots.device.type == "cuda"
        n = self.n_slots
        if self._gpu:
            self._streams = tuple(torch.cuda.Stream(device=slots.device) for _ in range(min(n_cs, n)))
            self.copy_stream = self._streams[0]
            self._copied = tuple(torch.cuda.Event(enable_timing=self.timing) for _ in range(n))
            self._gemm_done = tuple(torch.cuda.Event() for _ in range(n))
            self._copy_start = tuple(torch.cuda.Event(enable_timing=True) if self.timing else None
                                     for _ in range(n))
            for e in self._gemm_done:
                e.record()   # every slot starts free; never wait on an unrecorded event
        else:
            self._streams = ()
            self.copy_stream = None
            self._copied = self._gemm_done = self._copy_start = (None,) * n

    # ---- bookkeeping ---------------------------------------------------------------
    @property
    def ahead(self) -> int:
        """Copies issued and not yet consumed by a bind."""
        return self._ahead

    def _stream_of(self, slot: int):
        return self._streams[slot % len(self._streams)] if self._streams else None

    def arm(self, gemms: Sequence[StreamedMatrix]) -> None:
        """Start a forward: the HOST matrices of ``gemms``, in the order they will be
        consumed, become the tape.  Copies that ``prefetch_next`` already issued for the
        head of this tape are kept and not repeated."""
        tape = tuple(g for g in gemms if g.home == "host")
        carried = self._carried_prefix(tape)
        if carried is None:
            self._inflight.clear()
            self._ahead = 0
            self._next_slot = 0
            self._tape_pos = 0
        else:
            self._tape_pos = carried
        self._tape = tape
        self._bound_slot = None
        self._bound = None
        self.ops.clear()
        self.slot_order.clear()
        self.issue_count = 0
        self.forward_bytes = 0
        self.forward_copy_ms = 0.0
        self.total_forwards += 1

    def _carried_prefix(self, tape) -> int | None:
        if not tape or not self._inflight or self._bound_slot is not None:
            return None
        if self._ahead != len(self._inflight) or len(self._inflight) > len(tape):
            return None
        if any(not _same(g, tape[i]) for i, (g, _) in enumerate(self._inflight)):
            return None
        return len(self._inflight)

    # ---- copies ---------------------------------------------------------------------
    def prefetch(self) -> None:
        """Issue tape entries until ``max_ahead`` copies run ahead (or the tape ends)."""
        while self._ahead < self.max_ahead and self._tape_pos < len(self._tape):
            if self._bound_slot is not None and self._next_slot == self._bound_slot:
                break
            g = self._tape[self._tape_pos]
            self._tape_pos += 1
            self.issue(g)

    def prefetch_next(self) -> None:
        """After the last HOST matrix of a forward: start the head of the same tape for
        the next forward (it overlaps whatever resident work is left, e.g. lm_head)."""
        if not self._tape or self._tape_pos < len(self._tape) or self._bound_slot is not None:
            return
        i = 0
        while self._ahead < self.max_ahead and i < len(self._tape):
            self.issue(self._tape[i])
            i += 1

    def issue(self, gemm: StreamedMatrix) -> int:
        """Start the copy of one host image into the next slot; returns the slot."""
        if self._ahead >= self.max_ahead:
            raise RuntimeError(f"CopyRing prefetch depth is {self.max_ahead}; issue({gemm.name}) "
                               f"would make ahead={self._ahead + 1}")
        if gemm.home != "host" or gemm.host_image is None:
            raise RuntimeError(f"{gemm.name}: CopyRing.issue expects a HOST gemm")
        s = self._next_slot
        if self._bound_slot is not None and s == self._bound_slot:
            raise RuntimeError(f"CopyRing.issue({gemm.name}) would overwrite in-GEMM slot {s}")
        nbytes = int(gemm.host_image.nbytes)
        if nbytes > self.slots.nbytes:
            raise ValueError(f"{gemm.name}: host image {nbytes} bytes exceeds slot {self.slots.nbytes}")
        src = gemm.host_image.arena
        if int(src.numel()) != nbytes:
            raise ValueError(f"{gemm.name}: arena {int(src.numel())} != nbytes {nbytes}")
        dst = self.slots.arena[s][:nbytes]
        self.ops.append(("wait_gemm", s))
        if self._gpu:
            cs = self._stream_of(s)
            cs.wait_event(self._gemm_done[s])
            with torch.cuda.stream(cs):
                if self.timing:
                    self._copy_start[s].record(cs)
                dst.copy_(src, non_blocking=True)
            self._copied[s].record(cs)
        else:
            dst.copy_(src)
        self.ops.append(("h2d", s, nbytes))
        self.ops.append(("record_copy", s))
        self._inflight.append((gemm, s))
        self._next_slot = (s + 1) % self.n_slots
        self._ahead += 1
        self.issue_count += 1
        self.forward_bytes += nbytes
        self.total_copies += 1
        self.total_bytes += nbytes
        self.slot_order.append(s)
        return s

    def _issue_unprefetched(self, gemm: StreamedMatrix) -> None:
        if self._tape_pos < len(self._tape) and _same(self._tape[self._tape_pos], gemm):
            self._tape_pos += 1
        self.issue(gemm)

    # ---- consumption ------------------------------------------------------------------
    def _take(self, gemm: StreamedMatrix, who: str):
        if not self._inflight:
            self._issue_unprefetched(gemm)
        head, s = self._inflight[0]
        if not _same(head, gemm):
            raise RuntimeError(f"CopyRing.{who}({gemm.name}): queue head is {head.name}")
        self._inflight.popleft()
        self._ahead = max(0, self._ahead - 1)
        self.ops.append(("wait_copy", s))
        if self._gpu:
            torch.cuda.current_stream().wait_event(self._copied[s])
            if self._join_copy or self.timing:
                self._copied[s].synchronize()
            if self.timing:
                dt = float(self._copy_start[s].elapsed_time(self._copied[s]))
                self.forward_copy_ms += dt
                self.total_copy_ms += dt
        views = self.slots.view(s, gemm.M, gemm.K, gemm.K_pad)
        self._bound_slot = s
        self._bound = gemm
        return views

    def bind_for_gemm(self, gemm: StreamedMatrix):
        """packed / scale to launch the kernel on: the resident tensors of a DEVICE matrix,
        or — once its copy is ordered before the current stream — views of the **slot** a
        HOST matrix was copied into.  The next copies are issued before returning, so they
        run under the caller's kernel."""
        if gemm.home != "host":
            return gemm.packed, gemm.scale
        if self._bound_slot is not None:
            raise RuntimeError(f"CopyRing.bind_for_gemm({gemm.name}): previous GEMM not record_gemm'd")
        views = self._take(gemm, "bind_for_gemm")
        self.prefetch()
        return views

    def bind_hold(self, gemm: StreamedMatrix):
        """Like ``bind_for_gemm`` but the slot stays bound over several kernels (prefill:
        one copy, many column chunks) and nothing is prefetched until ``release_hold``."""
        if gemm.home != "host":
            raise RuntimeError(f"CopyRing.bind_hold({gemm.name}): expected HOST gemm")
        if self._bound_slot is not None:
            raise RuntimeError(f"CopyRing.bind_hold({gemm.name}): hold already active")
        return self._take(gemm, "bind_hold")

    def gemm_hold(self) -> None:
        if self._bound_slot is None:
            raise RuntimeError("CopyRing.gemm_hold: no active hold")

    def release_hold(self, gemm: StreamedMatrix) -> None:
        self.record_gemm(gemm)
        self.prefetch()

    def record_gemm(self, gemm: StreamedMatrix | None = None) -> None:
        """The kernel on the bound slot has been launched: the slot may be overwritten
        once the compute stream gets here."""
        s = self._bound_slot
        if s is None:
            raise RuntimeError("CopyRing.record_gemm: no active bind")
        if gemm is not None and self._bound is not None and not _same(gemm, self._bound):
            raise RuntimeError(f"CopyRing.record_gemm({gemm.name}): active is {self._bound.name}")
        self.ops.append(("record_gemm", s))
        if self._gpu:
            self._gemm_done[s].record()
        self._bound_slot = None
        self._bound = None

    # ---- reporting --------------------------------------------------------------------
    def snapshot(self) -> dict:
        return {
            "slot_nbytes": int(self.slots.nbytes),
            "n_slots": self.n_slots,
            "max_ahead": self.max_ahead,
            "n_copy_streams": self.n_copy_streams,
            "ahead": self._ahead,
            "issue_count": self.issue_count,
            "forward_bytes": self.forward_bytes,
            "forward_copy_ms": float(self.forward_copy_ms) if self.timing else None,
            "total_copies": self.total_copies,
            "total_bytes": self.total_bytes,
            "total_copy_ms": float(self.total_copy_ms) if self.timing else None,
            "total_forwards": self.total_forwards,
            "timing": self.timing,
            "cuda": self._gpu,
        }

    def __repr__(self) -> str:
        return (f"CopyRing(n_slots={self.n_slots}, max_ahead={self.max_ahead}, "
                f"slot_nbytes={self.slots.nbytes}, ahead={self._ahead}, issued={self.issue_count}, "
                f"total_bytes={self.total_bytes}, cuda={self._gpu}, timing={self.timing})")
