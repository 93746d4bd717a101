"""The ``nn.Linear``-shaped seat of the NF4 kernels (``gpu/host/linear.py``)."""

from .linear import CompressedLinear, k_pad, nf4_linear

__all__ = ["CompressedLinear", "k_pad", "nf4_linear"]
