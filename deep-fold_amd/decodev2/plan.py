"""Architecture descriptions the resident decoder can drive.

``ArchSpec`` carries the fields of the reference's spec
(``gpu/decodev2/plan.py:17-84``) plus ``qkv_bias`` for Qwen-style models.  The
three toy specs are the reference's; the four large ones are the shapes the
benchmarks quote (random-init weights, no checkpoints).
"""

from __future__ import annotations

from dataclasses import dataclass, replace

__all__ = [
    "ArchSpec",
    "TINY_LLAMA",
    "TINY_INTERNLM",
    "MEDIUM_LLAMA",
    "QWEN25_3B",
    "QWEN25_14B",
    "INTERNLM25_20B",
    "QWEN25_32B",
    "with_max_seq",
]

_FAMILIES = ("llama_swiglu", "internlm_gqa")


@dataclass(frozen=True)
class ArchSpec:
    """``llama_swiglu`` has separate q/k/v matrices; ``internlm_gqa`` has one
    fused wqkv whose rows are laid out per KV head: its query heads, then K,
    then V."""

    name: str
    family: str
    n_layers: int
    hidden: int
    n_q: int
    n_kv: int
    head_dim: int
    intermediate: int
    vocab: int
    max_seq: int
    rms_eps: float = 1e-6
    rope_theta: float = 10000.0
    eos_id: int = 2
    tied_embed: bool = False
    qkv_bias: bool = False

    def __post_init__(self) -> None:
        if self.family not in _FAMILIES:
            raise ValueError(f"unsupported family {self.family!r}")
        if self.n_layers < 1 or self.max_seq < 2:
            raise ValueError("need at least one layer and max_seq>=2")
        if self.hidden != self.n_q * self.head_dim:
            raise ValueError(f"hidden {self.hidden} != n_q*head_dim {self.n_q * self.head_dim}")
        if self.n_q % self.n_kv != 0:
            raise ValueError(f"n_q={self.n_q} is not a multiple of n_kv={self.n_kv}")
        if self.head_dim % 2 != 0:
            raise ValueError("RoPE needs even head_dim")
        if self.hidden % 64 != 0 or self.intermediate % 64 != 0:
            raise ValueError("hidden and intermediate must be multiples of NF4 group 64")
        if not 0 <= self.eos_id < self.vocab:
            raise ValueError(f"eos_id {self.eos_id} out of vocab {self.vocab}")

    @property
    def n_rep(self) -> int:
        return self.n_q // self.n_kv

    @property
    def q_dim(self) -> int:
        return self.n_q * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.n_kv * self.head_dim

    @property
    def wqkv_out(self) -> int:
        return (self.n_q + 2 * self.n_kv) * self.head_dim

    @property
    def attn_scale(self) -> float:
        return self.head_dim ** -0.5

    def linear_weights(self) -> int:
        """Weights of every packed linear touched by one decode token
        (q, k, v, o, gate, up, down per layer, plus lm_head)."""
        h, kv, f = self.hidden, self.kv_dim, self.intermediate
        per_layer = h * h + 2 * kv * h + h * h + 3 * f * h
        return self.n_layers * per_layer + self.vocab * h

    def weight_bytes_per_token(self) -> int:
        """Packed codes + fp16 scales read per decode token: 0.53125 B / weight."""
        return self.linear_weights() * 17 // 32

    def kv_bytes(self, length: int) -> int:
        """K and V bytes read by one token's attention at context ``length``."""
        return 2 * self.n_layers * int(length) * self.n_kv * self.head_dim * 2


def with_max_seq(spec: ArchSpec, max_seq: int) -> ArchSpec:
    return replace(spec, max_seq=int(max_seq))


TINY_LLAMA = ArchSpec("tiny-llama", "llama_swiglu", 2, 64, 4, 2, 16, 128, 32, 16)
TINY_INTERNLM = ArchSpec("tiny-internlm", "internlm_gqa", 2, 64, 4, 2, 16, 128, 32, 16)
MEDIUM_LLAMA = ArchSpec("medium-llama", "llama_swiglu", 4, 512, 8, 2, 64, 1024, 128, 32)

QWEN25_3B = ArchSpec("qwen2.5-3b-arch", "llama_swiglu", 36, 2048, 16, 2, 128, 11008, 151936, 2048,
                     rms_eps=1e-6, rope_theta=1e6, eos_id=151645, qkv_bias=True)
QWEN25_14B = ArchSpec("qwen2.5-14b-arch", "llama_swiglu", 48, 5120, 40, 8, 128, 13824, 152064, 2048,
                      rms_eps=1e-6, rope_theta=1e6, eos_id=151645, qkv_bias=True)
INTERNLM25_20B = ArchSpec("internlm2.5-20b-arch", "internlm_gqa", 48, 6144, 48, 8, 128, 16384, 92544,
                          2048, rms_eps=1e-5, rope_theta=5e7, eos_id=2)
QWEN25_32B = ArchSpec("qwen2.5-32b-arch", "llama_swiglu", 64, 5120, 40, 8, 128, 27648, 152064, 2048,
                      rms_eps=1e-6, rope_theta=1e6, eos_id=151645, qkv_bias=True)
