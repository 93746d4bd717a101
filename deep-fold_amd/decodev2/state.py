"""GPU-resident decode registers: token, position, valid_len, next id
(``gpu/decodev2/state.py:19-107``).  Everything a step reads or writes is a
device tensor, so one captured graph serves every position."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ..nf4 import dv2_argmax_commit
from .arena import Arena
from .embed import PackedEmbed
from .kv import GraphSafeKV
from .plan import ArchSpec
from .rope import rope_tables_torch

__all__ = ["DecodeState"]


@dataclass
class DecodeState:
    spec: ArchSpec
    token: torch.Tensor
    position: torch.Tensor
    valid_len: torch.Tensor
    next_token: torch.Tensor
    finished: torch.Tensor
    kv: GraphSafeKV
    arena: Arena
    cos: torch.Tensor
    sin: torch.Tensor
    eos_id: torch.Tensor

    @classmethod
    def allocate(cls, spec: ArchSpec, *, device="cuda", dtype: torch.dtype = torch.bfloat16,
                 cos: torch.Tensor | None = None, sin: torch.Tensor | None = None) -> "DecodeState":
        device = torch.device(device)
        if device.type != "cuda":
            raise RuntimeError("the resident decoder runs on the GPU only")
        valid_len = torch.zeros((), dtype=torch.int32, device=device)
        kv = GraphSafeKV(spec, device=device, dtype=dtype, valid_len=valid_len)
        arena = Arena.allocate(spec, device=device, dtype=dtype)
        if cos is None or sin is None:
            cos, sin = rope_tables_torch(spec.max_seq, spec.head_dim, spec.rope_theta,
                                         device=device, dtype=dtype)
        else:
            cos = cos.to(device=device, dtype=dtype).contiguous()
            sin = sin.to(device=device, dtype=dtype).contiguous()

        def scalar(dt, value=0):
            return torch.full((), value, dtype=dt, device=device)

        return cls(spec=spec, token=scalar(torch.int64), position=scalar(torch.int64),
                   valid_len=valid_len, next_token=scalar(torch.int64),
                   finished=scalar(torch.uint8), kv=kv, arena=arena, cos=cos, sin=sin,
                   eos_id=scalar(torch.int64, spec.eos_id))

    @property
    def device(self) -> torch.device:
        return self.token.device

    def reset(self) -> None:
        """New request.  Dirty KV is legal; ``valid_len`` hides it."""
        for t in (self.token, self.position, self.valid_len, self.next_token, self.finished):
            t.zero_()

    def load_token(self, token_id: int) -> None:
        self.token.fill_(int(token_id))

    def pick_next(self, commit: bool) -> None:
        """``next_token = argmax(logits)``; with ``commit`` feed it back without a
        host round trip: ``token = next``, ``position += 1``, ``finished |= eos``."""
        dv2_argmax_commit(self.arena.logits.view(-1), self.next_token, self.token, self.position,
                          self.finished, self.eos_id, commit=commit, ws=self.arena.argmax_ws)

    def commit_step(self) -> None:
        """Feed ``next_token`` back on the device (``gpu/decodev2/state.py:98-103``): the same
        launch as ``pick_next(commit=True)``, which picks the id again from the logits it was
        picked from and then commits it."""
        self.pick_next(commit=True)

    def rope_at_position(self) -> tuple[torch.Tensor, torch.Tensor]:
        """Rows of the RoPE tables at the device-side position, ``[1, head_dim]`` each
        (``gpu/decodev2/state.py:105-107``); the step's kernels index the tables themselves,
        this is for callers that want the rows."""
        at = self.position.reshape(1)
        return self.cos.index_select(0, at), self.sin.index_select(0, at)
