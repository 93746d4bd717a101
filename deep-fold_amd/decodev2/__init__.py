"""Resident decoder for NF4 models on one MI355X: device-scalar state, static
arena and KV, eager step, HIP-graph replay, chunked prefill."""

from .arena import Arena
from .chr import weights_from_chr, write_synth_chr
from .embed import PackedEmbed, gather_embed
from .graph import GreedyGraph, capture_greedy
from .kv import GraphSafeKV
from .linear import DeviceLayer, DeviceLinear, DeviceWeights, nf4_linear
from .plan import (INTERNLM25_20B, MEDIUM_LLAMA, QWEN25_3B, QWEN25_14B, QWEN25_32B, TINY_INTERNLM,
                   TINY_LLAMA, ArchSpec, with_max_seq)
from .prefill import ChunkPrefill, forward_prefill, prefill_chunk_width
from .rope import apply_rope_torch, rope_tables_numpy, rope_tables_torch
from .runner import consume_prompt, generate
from .session import DecodeV2Loop, Generation
from .state import DecodeState
from .step import SCHEDULES, forward_decode, greedy_decode, teacher_force_token
from .synth import Nf4Matrix, SynthLayer, SynthModel, build

__all__ = [
    "ArchSpec", "Arena", "ChunkPrefill", "DecodeState", "DecodeV2Loop", "Generation", "DeviceLayer", "DeviceLinear", "DeviceWeights", "GraphSafeKV",
    "GreedyGraph", "PackedEmbed", "Nf4Matrix", "SynthLayer", "SynthModel", "TINY_LLAMA",
    "TINY_INTERNLM", "MEDIUM_LLAMA", "QWEN25_3B", "QWEN25_14B", "INTERNLM25_20B", "QWEN25_32B",
    "apply_rope_torch", "build", "capture_greedy", "consume_prompt", "SCHEDULES", "forward_decode",
    "forward_prefill", "gather_embed", "generate", "greedy_decode", "nf4_linear",
    "prefill_chunk_width", "rope_tables_numpy", "rope_tables_torch", "teacher_force_token",
    "weights_from_chr", "with_max_seq", "write_synth_chr",
]
