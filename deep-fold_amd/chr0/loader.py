"""NF4 matrices of a ``.chr`` file onto the GPU (``gpu/chr0/loader.py:28-130``): the bytes
on disk are the bytes in HBM, nothing is decoded.  One positioned read per matrix into a
pinned staging buffer, one copy into one device allocation, ``packed`` and ``scale`` are
views of it."""

from __future__ import annotations

import os
from dataclasses import dataclass

import torch

from .errors import CodecError, GroupSizeError, TruncatedError
from .header import NF4_GROUP_SIZE, Header, load_header

__all__ = ["ChrMatrix", "materialize_nf4", "read_bf16"]


@dataclass(frozen=True)
class ChrMatrix:
    """The fields of ``chr_nf4_dev_t`` (``gpu/include/chr_gpu.h:11-17``) plus the name."""

    name: str
    M: int
    K: int
    K_pad: int
    packed: torch.Tensor  # uint8 [M, K_pad // 2]
    scale: torch.Tensor   # float16 [M, K_pad // 64]

    @property
    def n_groups(self) -> int:
        return self.K_pad // NF4_GROUP_SIZE

    @property
    def device(self) -> torch.device:
        return self.packed.device

    @property
    def nbytes(self) -> int:
        return self.packed.numel() + 2 * self.scale.numel()


def _read_into(path: str, host: torch.Tensor, at: int, start: int, nbytes: int, what: str) -> None:
    view = memoryview(host.numpy())[at:at + nbytes]
    fd = os.open(path, os.O_RDONLY)
    try:
        got = 0
        while got < nbytes:
            step = os.preadv(fd, [view[got:]], start + got)
            if step <= 0:
                break
            got += step
    finally:
        os.close(fd)
    if got != nbytes:
        raise TruncatedError(f"truncated: {what} wanted {nbytes} bytes at {start}, got {got}")


def _host_buffer(nbytes: int, device: torch.device) -> torch.Tensor:
    return torch.empty(nbytes, dtype=torch.uint8, pin_memory=device.type == "cuda")


def materialize_nf4(path: str | os.PathLike, name: str, device: str | torch.device = "cuda", *,
                    header: Header | None = None) -> ChrMatrix:
    """Load tensor ``name`` (codec nf4).  Without ``header`` the file's header is read and
    validated first; either way every byte is in host memory before the device is touched."""
    path = os.fspath(path)
    hdr = header if header is not None else load_header(path)
    info = hdr.tensor(name)
    if info.codec != "nf4":
        raise CodecError(f"{name}: codec {info.codec!r}, only nf4 matrices are materialised")
    if info.group_size != NF4_GROUP_SIZE:
        raise GroupSizeError(f"{name}: group_size {info.group_size}, must be {NF4_GROUP_SIZE}")
    data, scale = info.blobs["data"], info.blobs["scale"]
    dev = torch.device(device)
    if dev.type == "cuda" and not torch.cuda.is_available():
        raise RuntimeError("device 'cuda' asked for, but no GPU is visible")
    host = _host_buffer(data.nbytes + scale.nbytes, dev)
    if scale.start == data.end:  # the writer's layout: one read covers both
        _read_into(path, host, 0, data.start, data.nbytes + scale.nbytes, name)
    else:
        _read_into(path, host, 0, data.start, data.nbytes, f"{name}.data")
        _read_into(path, host, data.nbytes, scale.start, scale.nbytes, f"{name}.scale")
    arena = host.to(dev) if dev.type == "cuda" else host.clone()
    m, kp = info.M, info.K_pad
    return ChrMatrix(name=name, M=m, K=info.K, K_pad=kp,
                     packed=arena[:data.nbytes].view(m, kp // 2),
                     scale=arena[data.nbytes:].view(torch.float16).view(m, info.n_groups))


def read_bf16(path: str | os.PathLike, name: str, device: str | torch.device = "cuda", *,
              header: Header | None = None) -> torch.Tensor:
    """A bf16 tensor (norm weight, bias) of the file, in its logical shape."""
    path = os.fspath(path)
    hdr = header if header is not None else load_header(path)
    info = hdr.tensor(name)
    if info.codec != "bf16":
        raise CodecError(f"{name}: codec {info.codec!r} is not bf16")
    blob = info.blobs["data"]
    dev = torch.device(device)
    host = _host_buffer(blob.nbytes, dev)
    _read_into(path, host, 0, blob.start, blob.nbytes, name)
    return host.view(torch.bfloat16).view(*info.shape).to(dev)
