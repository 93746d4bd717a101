"""A greedy session with the surface the reference's CLI and chat callers drive
(``DecodeV2Loop``, ``gpu/decodev2/session.py:135-417``; ``Generation``,
``gpu/loop/generate.py:255-300``): ``generate``, ``reset``, ``prefill_from`` / ``forward`` for
an appended suffix, ``seal_last``, ``decode_from_logits``, ``warmup``, ``capture_graphs``.

Built from weights already on the GPU (``from_weights``) or from a ``.chr`` file
(``from_chr``); the reference's ``from_model`` walks an HF module tree, which this
library does not carry.  Prompts go through the feature-major chunk prefill, decode
tokens through the captured step once ``capture_graphs`` has run."""

from __future__ import annotations

import os
import time
from collections.abc import Callable, Sequence
from dataclasses import dataclass, field
from types import SimpleNamespace

import torch

from .embed import PackedEmbed
from .graph import capture_greedy
from .linear import DeviceWeights
from .plan import ArchSpec
from .prefill import ChunkPrefill, prefill_chunk_width
from .runner import consume_prompt
from .state import DecodeState
from .step import greedy_decode, teacher_force_token

__all__ = ["Generation", "DecodeV2Loop"]


@dataclass
class Generation:
    """One greedy request; prefill and decode times are kept apart."""

    prompt_len: int
    tokens: list[int] = field(default_factory=list)
    prefill_ms: float = 0.0
    decode_ms: float = 0.0
    decode_steps: int = 0
    stop_token: int | None = None
    interrupted: bool = False
    prefill_chunk: int = 1
    graph: str = "off"

    @property
    def decode_tok_s(self) -> float:
        return self.decode_steps / (self.decode_ms / 1000.0) if self.decode_ms > 0 else 0.0

    @property
    def prefill_tok_s(self) -> float:
        return self.prompt_len / (self.prefill_ms / 1000.0) if self.prefill_ms > 0 else 0.0


class _KvView:
    """``loop.kv.mib`` and ``loop.kv.seq_len`` as the callers read them."""

    def __init__(self, k: torch.Tensor, v: torch.Tensor) -> None:
        self.seq_len = 0
        self._bytes = k.numel() * k.element_size() + v.numel() * v.element_size()

    @property
    def mib(self) -> float:
        return self._bytes / (1024 * 1024)


def _ids(prompt_ids) -> list[int]:
    if hasattr(prompt_ids, "reshape"):
        return [int(t) for t in prompt_ids.reshape(-1).tolist()]
    return [int(t) for t in prompt_ids]


class DecodeV2Loop:
    def __init__(self, state: DecodeState, weights: DeviceWeights, *, fused_prefill: bool = True) -> None:
        self.state = state
        self.weights = weights
        spec = state.spec
        self.max_seq = int(spec.max_seq)
        self.prefill_chunk = prefill_chunk_width(state)
        self.plan = SimpleNamespace(family=spec.family,
                                    qkv_pack="internlm" if spec.family == "internlm_gqa" else None)
        self.graph_mode = "off"
        self.graph_error: str | None = None
        self._graph = None
        self._prefill = ChunkPrefill(state, weights) if fused_prefill else None
        self.kv = _KvView(state.kv.k, state.kv.v)

    # ---- construction ----------------------------------------------------------------
    @classmethod
    def from_weights(cls, weights: DeviceWeights, **kw) -> "DecodeV2Loop":
        return cls(DecodeState.allocate(weights.spec, device=weights.lm_head.packed.device), weights, **kw)

    @classmethod
    def from_chr(cls, path: str | os.PathLike, spec: ArchSpec, device="cuda", **kw) -> "DecodeV2Loop":
        from .chr import weights_from_chr
        return cls.from_weights(weights_from_chr(path, spec, device), **kw)

    # ---- bookkeeping -------------------------------------------------------------------
    @property
    def device(self) -> torch.device:
        return self.state.device

    @property
    def weight_bytes(self) -> int:
        """Device bytes of every weight tensor, one count per allocation (a tied lm_head
        aliases the embedding rows)."""
        seen: dict[int, int] = {}

        def add(t) -> None:
            if t is not None and t.numel():
                seen[t.data_ptr()] = t.numel() * t.element_size()

        w = self.weights
        for t in ((w.embed.packed, w.embed.scale) if isinstance(w.embed, PackedEmbed) else (w.embed,)):
            add(t)
        add(w.final_norm)
        mats = [w.lm_head]
        for ly in w.layers:
            add(ly.norm1)
            add(ly.norm2)
            mats += [m for m in (ly.q, ly.k, ly.v, ly.wqkv, ly.o, ly.gate, ly.up, ly.down) if m is not None]
        for m in mats:
            add(m.packed)
            add(m.scale)
            add(m.bias)
        return sum(seen.values())

    def _sync(self) -> None:
        torch.cuda.synchronize(self.device)

    def _note_len(self) -> None:
        self.kv.seq_len = int(self.state.valid_len.item())

    def reset(self) -> None:
        self.state.reset()
        self.kv.seq_len = 0

    # ---- prompt ------------------------------------------------------------------------
    @torch.no_grad()
    def prefill_from(self, ids, start_pos: int) -> torch.Tensor:
        """Write ``ids`` into cache slots ``start_pos ..`` and return the logits of the
        last one (a view of the arena)."""
        seq = _ids(ids)
        pos = int(start_pos)
        if not seq:
            raise ValueError("empty prompt")
        if pos < 0 or pos + len(seq) > self.max_seq:
            raise ValueError(f"position {pos}+{len(seq)} past max_seq={self.max_seq}")
        consume_prompt(self.state, self.weights, seq, start=pos, prefill=self._prefill)
        self._note_len()
        return self.state.arena.logits[0]

    @torch.no_grad()
    def forward(self, ids, start_pos: int, *, logits: bool = True, all_positions: bool = False) -> torch.Tensor:
        """``prefill_from`` under the name the chat session calls to rewrite slots."""
        del logits, all_positions
        return self.prefill_from(ids, start_pos)

    @torch.no_grad()
    def seal_last(self, token_id: int) -> None:
        """Write the last sampled token into the cache so that a suffix can be appended."""
        if int(self.state.valid_len.item()) >= self.max_seq:
            return
        teacher_force_token(self.state, self.weights, int(token_id))
        self._note_len()

    # ---- decode ------------------------------------------------------------------------
    @torch.no_grad()
    def decode_from_logits(self, logits, max_new_tokens: int, *, prompt_len: int, stop: Sequence[int] = (),
                           on_token: Callable[[int], None] | None = None,
                           should_stop: Callable[[], bool] | None = None,
                           prefill_ms: float = 0.0) -> Generation:
        """Greedy tokens from the state a prefill left; neither resets nor prefills.  The
        first token is the prefill's pick; each later one costs one decode step and one
        host read."""
        del logits
        stops = frozenset(int(s) for s in stop)
        out = Generation(prompt_len=int(prompt_len), prefill_chunk=self.prefill_chunk,
                         graph=self.graph_mode, prefill_ms=float(prefill_ms))
        step = self._graph if self._graph is not None else greedy_decode
        token = int(self.state.next_token.item())
        seq = int(self.state.valid_len.item())
        self.kv.seq_len = seq
        self.state.token.copy_(self.state.next_token)
        self._sync()
        t0 = time.perf_counter()
        budget = max(0, int(max_new_tokens))
        for i in range(budget):
            if should_stop is not None and should_stop():
                out.interrupted = True
                break
            out.tokens.append(token)
            if on_token is not None:
                on_token(token)
            if token in stops:
                out.stop_token = token
                break
            if i + 1 == budget or seq >= self.max_seq:
                break
            step(self.state, self.weights)
            out.decode_steps += 1
            token = int(self.state.token.item())
            seq += 1
            self.kv.seq_len = seq
        self._sync()
        out.decode_ms = (time.perf_counter() - t0) * 1000.0
        self._note_len()
        return out

    @torch.no_grad()
    def generate(self, prompt_ids, max_new_tokens: int = 64, *, stop: Sequence[int] = (),
                 on_token: Callable[[int], None] | None = None,
                 should_stop: Callable[[], bool] | None = None, speculate: int = 1,
                 draft: str = "none") -> Generation:
        if str(draft) != "none" and int(speculate) > 1:
            raise ValueError("decodev2 does not speculate")
        ids = _ids(prompt_ids)
        if not ids:
            raise ValueError("empty prompt")
        if len(ids) > self.max_seq:
            raise ValueError(f"prompt {len(ids)} exceeds max_seq={self.max_seq}")
        self.reset()
        self._sync()
        t0 = time.perf_counter()
        logits = self.prefill_from(ids, 0)
        self._sync()
        return self.decode_from_logits(logits, max_new_tokens, prompt_len=len(ids), stop=stop,
                                       on_token=on_token, should_stop=should_stop,
                                       prefill_ms=(time.perf_counter() - t0) * 1000.0)

    # ---- preparation -------------------------------------------------------------------
    def warmup(self, *, prompt: int = 8, tokens: int = 8) -> float:
        """Run a short request so that lazy set-up is paid before the first real one."""
        n = max(1, min(int(prompt), self.max_seq - 2))
        self.reset()
        self._sync()
        t0 = time.perf_counter()
        consume_prompt(self.state, self.weights, [1] * n, prefill=self._prefill)
        self.state.token.copy_(self.state.next_token)
        for _ in range(max(0, min(int(tokens), 8))):
            if int(self.state.position.item()) >= self.max_seq:
                break
            greedy_decode(self.state, self.weights)
        self._sync()
        self.reset()
        return (time.perf_counter() - t0) * 1000.0

    def capture_graphs(self) -> str:
        """Capture the decode step; on failure the loop keeps stepping eagerly and
        ``graph_error`` says why."""
        try:
            self._graph = capture_greedy(self.state, self.weights, warmup=2)
            self.graph_mode, self.graph_error = "decodev2", None
        except Exception as exc:  # noqa: BLE001
            self._graph = None
            self.graph_mode, self.graph_error = "off", f"{type(exc).__name__}: {exc}"
        self.reset()
        return self.graph_mode
