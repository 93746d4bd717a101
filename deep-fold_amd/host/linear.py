"""``CompressedLinear``: the ``nn.Linear``-shaped seat of the NF4 kernels (operator surface
of ``gpu/host/linear.py:31-220``).

The module owns the file's bytes (``packed``, ``scale``) and never an ``[out, in]`` weight:
nothing registers one, ``weight`` is a read-only 0-element stand-in, so neither
``model.to("cuda")`` nor a generic utility can bring a dense copy into HBM.

Layout glue lives here: callers hand ``[..., K]`` activations, the kernels take ``[K, N]``
(token index fastest) and answer ``[M, N]``.  One token is a view (no copy) and goes to the
GEMV; more tokens go to the MFMA GEMM in windows of at most 32, each window's answer
written straight into its rows of the one output buffer.  The bias is added afterwards in
bf16, as the reference does (``linear.py:62-63,79-80``), so both seats round alike.
"""

from __future__ import annotations

import math

import torch
from torch import nn

from ..chr0.loader import ChrMatrix
from ..nf4 import LIVE_MAX_N, nf4_gemm
from ..nf4.plan import k_pad
from ..ring.host_image import HostImage

__all__ = ["CompressedLinear", "nf4_linear", "k_pad"]

GROUP_SIZE = 64


def nf4_linear(x: torch.Tensor, packed: torch.Tensor, scale: torch.Tensor, M: int, K: int,  # noqa: N803
               K_pad: int, bias: torch.Tensor | None = None) -> torch.Tensor:  # noqa: N803
    """``y[..., M] = x[..., K] @ dequant(packed, scale).T (+ bias)`` in bf16."""
    if x.shape[-1] != K:
        raise ValueError(f"the last dimension of x is {x.shape[-1]}, the matrix multiplies K={K}")
    lead = x.shape[:-1]
    n = math.prod(lead)
    if n < 1:
        raise ValueError(f"x{tuple(x.shape)} holds no token to multiply")
    rows = x.to(torch.bfloat16).reshape(n, K)
    if n == 1:
        out = nf4_gemm(packed, scale, rows.reshape(K, 1), M, K, K_pad).reshape(1, M)
    else:
        out = torch.empty((n, M), dtype=torch.bfloat16, device=rows.device)
        for lo in range(0, n, LIVE_MAX_N):
            window = rows[lo:lo + LIVE_MAX_N]
            feature_major = window.t().contiguous()                       # [K, window]
            out[lo:lo + window.shape[0]] = nf4_gemm(packed, scale, feature_major, M, K, K_pad).t()
    if bias is not None:
        out = out + bias
    return out.reshape(*lead, M)


class CompressedLinear(nn.Module):
    """Stands where an ``nn.Linear(in_features, out_features)`` stood; its weight is an NF4
    matrix attached later (``attach``), so swapping modules in costs nothing and a skeleton
    can be built before any file is read."""

    def __init__(self, in_features: int, out_features: int, bias: bool = False, *,
                 device: torch.device | str | None = None,
                 dtype: torch.dtype = torch.bfloat16) -> None:
        super().__init__()
        self.in_features, self.out_features = int(in_features), int(out_features)
        if min(self.in_features, self.out_features) < 1:
            raise ValueError(f"in_features={in_features} and out_features={out_features} must both be positive")
        self.K, self.M = self.in_features, self.out_features
        self.K_pad = k_pad(self.K)
        self.n_groups = self.K_pad // GROUP_SIZE
        self.compute_dtype = dtype
        where = torch.device("cpu" if device is None else device)
        # file bytes, not state of ours: kept out of state_dict
        self.register_buffer("packed", torch.empty(0, dtype=torch.uint8, device=where), persistent=False)
        self.register_buffer("scale", torch.empty(0, dtype=torch.float16, device=where), persistent=False)
        self.register_buffer("bias", torch.empty(0, dtype=dtype, device=where) if bias else None,
                             persistent=False)
        self.chr_name: str | None = None
        self.host_image: HostImage | None = None

    # ---- what stands in for nn.Linear.weight --------------------------------------------
    @property
    def weight(self) -> torch.Tensor:
        """0 elements of the compute dtype on the layer's device, for code that asks a
        linear for ``weight.dtype`` / ``weight.device``.  There is no setter: assigning a
        dense weight raises instead of allocating ``out x in``."""
        return self.packed.new_empty(0, dtype=self.compute_dtype)

    def _on_device(self) -> bool:
        return self.packed.numel() > 0

    @property
    def home(self) -> str:
        """``"device"``, ``"host"`` (pinned image waiting for a streaming ring) or ``"empty"``."""
        if self._on_device():
            return "device"
        return "host" if self.host_image is not None else "empty"

    @property
    def is_loaded(self) -> bool:
        return self.home != "empty"

    @property
    def nbytes(self) -> int:
        """Device bytes of the weight (0 for a host-resident one)."""
        return self.packed.numel() + self.scale.numel() * self.scale.element_size()

    # ---- attaching ----------------------------------------------------------------------
    def _check_shape(self, what: str, m: int, k: int, pad: int) -> None:
        if (int(m), int(k)) != (self.M, self.K):
            raise ValueError(f"{what} has {m} rows of {k}, this seat holds {self.M} rows of {self.K}")
        if int(pad) != self.K_pad:
            raise ValueError(f"{what} pads its rows to {pad} codes, this seat to {self.K_pad}")

    def attach(self, matrix: ChrMatrix) -> None:
        """Use ``matrix``'s tensors as they are (shared, not copied: tied layers can hold
        one matrix)."""
        self._check_shape(f"{matrix.name}: matrix", matrix.M, matrix.K, matrix.K_pad)
        if matrix.packed.dtype != torch.uint8 or matrix.scale.dtype != torch.float16:
            raise TypeError(f"{matrix.name}: codes must be uint8 and scales float16, not "
                            f"{matrix.packed.dtype} and {matrix.scale.dtype}")
        self.packed, self.scale = matrix.packed, matrix.scale
        self.chr_name, self.host_image = matrix.name, None

    def attach_host(self, image: HostImage) -> None:
        """Keep the matrix on the host (its arena is pinned from allocation when a GPU is
        present); ``forward`` refuses until a ring streams it: there is no silent copy."""
        self._check_shape("HostImage", image.M, image.K, image.K_pad)
        if self._on_device():
            self.packed, self.scale = self.packed.new_empty(0), self.scale.new_empty(0)
        self.host_image = image

    def set_bias(self, bias: torch.Tensor) -> None:
        if self.bias is None:
            raise ValueError(f"{self.chr_name or self} was built with bias=False: there is no bias to set")
        if tuple(bias.shape) != (self.M,):
            raise ValueError(f"a bias of shape {tuple(bias.shape)} does not fit {self.M} output features")
        self.bias = bias.to(self.compute_dtype)

    # ---- forward ------------------------------------------------------------------------
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        label = f"CompressedLinear[{self.M},{self.K}] ({self.chr_name or 'unnamed'})"
        where = self.home
        if where == "host":
            raise RuntimeError(f"{label} is host-resident; a CopyRing has to stream it, "
                               "forward does no silent host-to-device copy")
        if where == "empty":
            raise RuntimeError(f"{label} has no weights yet: attach() a ChrMatrix before calling it")
        bias = self.bias if self.bias is not None and self.bias.numel() else None
        return nf4_linear(x, self.packed, self.scale, self.M, self.K, self.K_pad, bias)

    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, "
                f"bias={self.bias is not None}, home={self.home}, weight=NF4 in groups of {GROUP_SIZE} "
                f"(K_pad={self.K_pad})")
