"""Streaming of NF4 matrices from pinned host memory through static device slots
(the overflow path of the reference's older executor: ``gpu/loop/ring.py``,
``gpu/host/slots.py``, ``gpu/host/host_image.py``)."""

from .host_image import GROUP, HostImage, arena_nbytes, is_pinned, pack_arena, unpack_arena
from .ring import CopyRing, StreamedMatrix, default_join_copy
from .slots import SLOT_ALIGN, SLOT_COUNT, SlotPair
from .stream import streamed_linear

__all__ = ["GROUP", "HostImage", "arena_nbytes", "is_pinned", "pack_arena", "unpack_arena", "CopyRing",
           "StreamedMatrix", "default_join_copy", "SLOT_ALIGN", "SLOT_COUNT", "SlotPair",
           "streamed_linear"]
