"""A linear whose weights may be streamed: bind, launch, record
(``gpu/loop/graph.py:433-457``)."""

from __future__ import annotations

import torch

from ..nf4 import LIVE_MAX_N, nf4_gemm, nf4_gemv
from .ring import CopyRing, StreamedMatrix

__all__ = ["streamed_linear"]


def streamed_linear(ring: CopyRing, gemm: StreamedMatrix, x: torch.Tensor) -> torch.Tensor:
    """``x`` is ``[K]`` (one token, GEMV) or ``[K, N]`` with N <= 32 (GEMM) on the GPU;
    returns ``[M]`` / ``[M, N]``.  A HOST matrix is waited for, used from its slot and
    released; the next copy of the tape runs under the kernel."""
    packed, scale = ring.bind_for_gemm(gemm)
    if x.dim() == 1:
        y = nf4_gemv(packed, scale, x, gemm.M, gemm.K, gemm.K_pad).view(-1)
    else:
        if int(x.size(1)) > LIVE_MAX_N:
            raise ValueError(f"streamed_linear takes at most {LIVE_MAX_N} columns, got {int(x.size(1))}")
        y = nf4_gemm(packed, scale, x, gemm.M, gemm.K, gemm.K_pad)
    if gemm.home == "host":
        ring.record_gemm(gemm)
    return y
