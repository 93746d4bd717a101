"""CPU float32 oracle of one decode step and of greedy decoding.

TEST INFRASTRUCTURE ONLY (see ``nf4_oracle.py``).  Restates the reference's
teacher-forced oracle (``gpu/decodev2/oracle.py:27-166``) on top of the codec
oracle: every linear is "decode the packed matrix to float32, then a float32
matmul", everything else is plain float32 numpy.  It works on any model object
with the fields of the product's ``SynthModel`` (spec, embed, final_norm,
lm_head, layers[*].{norm1,norm2,q,k,v,wqkv,o,gate,up,down}).

Pinned by: each piece against the textbook routine it reduces to (torch
``rms_norm``, ``silu``, ``scaled_dot_product_attention``, rotate-half RoPE) in
``tests/test_step_oracle.py``; the composition (norm placement, residuals, RoPE on
q and k only, GQA head map, bias placement, InternLM's wqkv row order) against
``transformers``' ``LlamaForCausalLM`` / ``Qwen2ForCausalLM`` in float32 on the
dequantised weights of the same seeded models, teacher-forced logits to 2e-5 of
the logit scale and the greedy chain token by token
(``tests/test_step_oracle_hf.py``).  The reference itself stores no expected ids
(its tests compute them at run time).
"""

from __future__ import annotations

from typing import Sequence

import numpy as np

from . import nf4_oracle as oc

NEG = np.float32(-1.0e9)


def rope_tables(max_seq: int, head_dim: int, theta: float) -> tuple[np.ndarray, np.ndarray]:
    """float32 ``[max_seq, head_dim]`` cos/sin, both halves equal
    (``gpu/decodev2/rope.py:20-33``)."""
    i = np.arange(0, head_dim, 2, dtype=np.float32)
    inv = (1.0 / (np.float32(theta) ** (i / np.float32(head_dim)))).astype(np.float32)
    fr = np.outer(np.arange(max_seq, dtype=np.float32), inv).astype(np.float32)
    emb = np.concatenate([fr, fr], axis=-1)
    return np.cos(emb).astype(np.float32), np.sin(emb).astype(np.float32)


def apply_rope(t: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
    """``t`` ``[N, heads, hd]``; ``cos``/``sin`` ``[N, hd]`` (``rope.py:36-44``)."""
    cos, sin = cos[:, None, :], sin[:, None, :]
    d = t.shape[-1] // 2
    rot = np.concatenate((-t[..., d:], t[..., :d]), axis=-1)
    return (t * cos + rot * sin).astype(np.float32)


def rms(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    v = x.astype(np.float32, copy=False)
    mean = (v * v).mean(axis=-1, keepdims=True)
    return (v * np.reciprocal(np.sqrt(mean + np.float32(eps))) * w.astype(np.float32)).astype(np.float32)


def silu(x: np.ndarray) -> np.ndarray:
    v = x.astype(np.float32, copy=False)
    return (v * (1.0 / (1.0 + np.exp(-v)))).astype(np.float32)


class _Decoded:
    """Decoded float32 matrices, cached per model (decode once, reuse per token)."""

    def __init__(self) -> None:
        self.cache: dict[int, np.ndarray] = {}

    def get(self, mat) -> np.ndarray:
        key = id(mat)
        if key not in self.cache:
            self.cache[key] = oc.c_decode(mat.packed, mat.scale, mat.M, mat.K)
        return self.cache[key]


def linear(mat, x: np.ndarray, decoded: _Decoded | None = None) -> np.ndarray:
    """``x`` ``[N, K]`` float32 -> ``[N, M]`` float32 (``oracle.py:42-50``)."""
    w = oc.c_decode(mat.packed, mat.scale, mat.M, mat.K) if decoded is None else decoded.get(mat)
    y = (w @ np.ascontiguousarray(x.astype(np.float32).T)).T
    if getattr(mat, "bias", None) is not None:
        y = y + mat.bias.astype(np.float32)
    return y.astype(np.float32)


def split_internlm(y: np.ndarray, spec):
    """Per KV head: its ``n_rep`` query heads, then K, then V (``oracle.py:53-59``)."""
    n = y.shape[0]
    p = y.reshape(n, spec.n_kv, 2 + spec.n_rep, spec.head_dim)
    q = p[:, :, : spec.n_rep, :].reshape(n, spec.n_q, spec.head_dim)
    return q, p[:, :, -2, :], p[:, :, -1, :]


def attend(q: np.ndarray, k: np.ndarray, v: np.ndarray, spec, valid_len: int) -> np.ndarray:
    """GQA over the first ``valid_len`` cache rows.  ``q`` ``[1, n_q, hd]``;
    ``k``/``v`` ``[max_seq, n_kv, hd]`` (``oracle.py:62-86``)."""
    n = q.shape[0]
    q4 = q.reshape(n, spec.n_kv, spec.n_rep, spec.head_dim)
    k4 = np.transpose(k, (1, 0, 2))[None]
    v4 = np.transpose(v, (1, 0, 2))[None]
    scores = np.einsum("bhrd,bhtd->bhrt", q4, k4).astype(np.float32)
    scores *= np.float32(spec.attn_scale)
    scores[..., int(valid_len):] = NEG
    scores = scores - scores.max(axis=-1, keepdims=True)
    w = np.exp(scores)
    w /= w.sum(axis=-1, keepdims=True)
    return np.einsum("bhrt,bhtd->bhrd", w, v4).astype(np.float32).reshape(n, spec.q_dim)


class OracleCache:
    def __init__(self, spec) -> None:
        shape = (spec.n_layers, spec.max_seq, spec.n_kv, spec.head_dim)
        self.spec = spec
        self.k = np.zeros(shape, dtype=np.float32)
        self.v = np.zeros(shape, dtype=np.float32)
        self.pos = 0
        self.cos, self.sin = rope_tables(spec.max_seq, spec.head_dim, spec.rope_theta)
        self.decoded = _Decoded()

    def reset(self) -> None:
        self.pos = 0


def step_logits(model, cache: OracleCache, token_id: int) -> np.ndarray:
    """Logits after feeding ``token_id`` at ``cache.pos`` (``oracle.py:113-140``)."""
    spec = model.spec
    if cache.pos >= spec.max_seq:
        raise ValueError(f"position {cache.pos} past max_seq={spec.max_seq}")
    dec = cache.decoded
    pos = cache.pos
    x = model.embed[int(token_id): int(token_id) + 1].astype(np.float32)
    cos, sin = cache.cos[pos: pos + 1], cache.sin[pos: pos + 1]
    for li, layer in enumerate(model.layers):
        h = rms(x, layer.norm1, spec.rms_eps)
        if spec.family == "internlm_gqa":
            q, k, v = split_internlm(linear(layer.wqkv, h, dec), spec)
        else:
            q = linear(layer.q, h, dec).reshape(1, spec.n_q, spec.head_dim)
            k = linear(layer.k, h, dec).reshape(1, spec.n_kv, spec.head_dim)
            v = linear(layer.v, h, dec).reshape(1, spec.n_kv, spec.head_dim)
        q = apply_rope(q, cos, sin)
        k = apply_rope(k, cos, sin)
        cache.k[li, pos] = k[0]
        cache.v[li, pos] = v[0]
        a = attend(q, cache.k[li], cache.v[li], spec, pos + 1)
        x = x + linear(layer.o, a, dec)
        h = rms(x, layer.norm2, spec.rms_eps)
        x = x + linear(layer.down, silu(linear(layer.gate, h, dec)) * linear(layer.up, h, dec), dec)
    hidden = rms(x, model.final_norm, spec.rms_eps)
    logits = linear(model.lm_head, hidden, dec)[0]
    cache.pos = pos + 1
    return logits.astype(np.float32)


def teacher_logits(model, token_ids: Sequence[int]) -> np.ndarray:
    cache = OracleCache(model.spec)
    rows = [step_logits(model, cache, int(t)) for t in token_ids]
    if not rows:
        return np.zeros((0, model.spec.vocab), dtype=np.float32)
    return np.stack(rows, axis=0)


def greedy_ids(model, prompt_ids: Sequence[int], n_new: int, *, ignore_eos: bool = False,
               return_margins: bool = False, return_tops: bool = False):
    """Greedy continuation (``oracle.py:151-166``).  With ``return_margins`` also the
    top-1 minus top-2 logit gap of every pick, which says how thin each decision is; with
    ``return_tops`` (and margins) the top-1 logit of every pick as a third list."""
    if not len(prompt_ids):
        raise ValueError("prompt_ids must be non-empty")
    cache = OracleCache(model.spec)
    last = None
    for t in prompt_ids:
        last = step_logits(model, cache, int(t))
    out: list[int] = []
    margins: list[float] = []
    tops: list[float] = []
    eos = int(model.spec.eos_id)
    tok = int(last.argmax())
    for _ in range(int(n_new)):
        out.append(tok)
        top2 = np.partition(last, -2)[-2:]
        margins.append(float(top2[1] - top2[0]))
        tops.append(float(top2[1]))
        if tok == eos and not ignore_eos:
            break
        if cache.pos >= model.spec.max_seq:
            break
        last = step_logits(model, cache, tok)
        tok = int(last.argmax())
    if return_margins and return_tops:
        return out, margins, tops
    return (out, margins) if return_margins else out
