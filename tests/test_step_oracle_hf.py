"""The whole-step CPU oracle against an independent implementation of the same
architecture: ``transformers``' ``LlamaForCausalLM`` / ``Qwen2ForCausalLM`` in float32 on
the dequantised weights of the same seeded synthetic models (CPU only).

The pieces of ``oracle/step_oracle.py`` are pinned one by one in ``test_step_oracle.py``;
this file pins their composition: norm placement, residual adds, RoPE on q and k only
(rotate-half, HF table layout), the GQA head mapping, bias placement, the causal prefix,
and, for the InternLM family, the interleaved wqkv row order.  A dropped residual, a
swapped norm, RoPE applied to v, a wrong q->kv head map or a bias added after RoPE each
moves logits by orders of magnitude more than the float32 tolerance used here.
"""

from __future__ import annotations

from dataclasses import replace

import numpy as np
import pytest
import torch

from deepfold_amd.decodev2 import plan as dplan
from deepfold_amd.decodev2.synth import build
from oracle import nf4_oracle as oc
from oracle import step_oracle as so

transformers = pytest.importorskip("transformers")


def _dec(mat) -> torch.Tensor:
    return torch.from_numpy(oc.c_decode(mat.packed, mat.scale, mat.M, mat.K).copy())


def _hf_config(spec, bias: bool):
    common = dict(vocab_size=spec.vocab, hidden_size=spec.hidden,
                  intermediate_size=spec.intermediate, num_hidden_layers=spec.n_layers,
                  num_attention_heads=spec.n_q, num_key_value_heads=spec.n_kv,
                  head_dim=spec.head_dim, hidden_act="silu",
                  max_position_embeddings=spec.max_seq, rms_norm_eps=spec.rms_eps,
                  rope_theta=spec.rope_theta, tie_word_embeddings=False,
                  attention_dropout=0.0, use_cache=False)
    if bias:
        cfg = transformers.Qwen2Config(**common, use_sliding_window=False)
        cls = transformers.Qwen2ForCausalLM
    else:
        cfg = transformers.LlamaConfig(**common, attention_bias=False, mlp_bias=False)
        cls = transformers.LlamaForCausalLM
    cfg._attn_implementation = "eager"
    return cfg, cls


def _split_wqkv(w: torch.Tensor, spec):
    """Rows of a fused InternLM wqkv, per KV head: its n_rep query heads, then K, then V
    (gpu/loop/generate.py:73-89), as separate q, k, v matrices."""
    hd, rep = spec.head_dim, spec.n_rep
    p = w.reshape(spec.n_kv, rep + 2, hd, spec.hidden)
    q = p[:, :rep].reshape(spec.n_q * hd, spec.hidden)
    k = p[:, rep].reshape(spec.n_kv * hd, spec.hidden)
    v = p[:, rep + 1].reshape(spec.n_kv * hd, spec.hidden)
    return q, k, v


def _load_hf(model, bias: bool):
    spec = model.spec
    cfg, cls = _hf_config(spec, bias)
    with torch.no_grad():
        hf = cls(cfg).to(torch.float32).eval()
        sd = {}
        sd["model.embed_tokens.weight"] = torch.from_numpy(model.embed.astype(np.float32).copy())
        sd["model.norm.weight"] = torch.from_numpy(model.final_norm.astype(np.float32).copy())
        sd["lm_head.weight"] = _dec(model.lm_head)
        for i, layer in enumerate(model.layers):
            p = f"model.layers.{i}."
            if spec.family == "internlm_gqa":
                q, k, v = _split_wqkv(_dec(layer.wqkv), spec)
                qb = kb = vb = None
            else:
                q, k, v = _dec(layer.q), _dec(layer.k), _dec(layer.v)
                qb, kb, vb = layer.q.bias, layer.k.bias, layer.v.bias
            sd[p + "self_attn.q_proj.weight"] = q
            sd[p + "self_attn.k_proj.weight"] = k
            sd[p + "self_attn.v_proj.weight"] = v
            if bias:
                for name, b, m in (("q", qb, q), ("k", kb, k), ("v", vb, v)):
                    sd[p + f"self_attn.{name}_proj.bias"] = (
                        torch.zeros(m.shape[0]) if b is None
                        else torch.from_numpy(np.asarray(b, dtype=np.float32).copy()))
            sd[p + "self_attn.o_proj.weight"] = _dec(layer.o)
            sd[p + "mlp.gate_proj.weight"] = _dec(layer.gate)
            sd[p + "mlp.up_proj.weight"] = _dec(layer.up)
            sd[p + "mlp.down_proj.weight"] = _dec(layer.down)
            sd[p + "input_layernorm.weight"] = torch.from_numpy(layer.norm1.astype(np.float32).copy())
            sd[p + "post_attention_layernorm.weight"] = torch.from_numpy(layer.norm2.astype(np.float32).copy())
        missing, unexpected = hf.load_state_dict(sd, strict=False)
        # rotary tables are buffers built from the config, everything else must be ours
        assert not unexpected, unexpected
        assert all("rotary" in m or "inv_freq" in m for m in missing), missing
    return hf


def _with_bias(model, seed: int):
    """Qwen-style q/k/v biases on a llama_swiglu model (drawn here; the values only have to
    be the same on both sides)."""
    rng = np.random.default_rng(seed)
    for layer in model.layers:
        for m in (layer.q, layer.k, layer.v):
            m.bias = (rng.standard_normal(m.M) * 0.3).astype(np.float32)
    return model


CASES = [
    ("tiny-llama", dplan.TINY_LLAMA, 0, False, [1, 3, 5, 7, 2, 9, 30, 11, 4, 4, 17, 0]),
    ("medium-llama", dplan.MEDIUM_LLAMA, 3, False, list(range(5, 29))),
    ("tiny-qwen-bias", dplan.TINY_LLAMA, 5, True, [6, 2, 8, 31, 1, 0, 19, 7, 7, 3]),
    ("medium-qwen-bias", replace(dplan.MEDIUM_LLAMA, rope_theta=1e6), 9, True,
     [100, 3, 77, 12, 5, 64, 127, 0, 9, 41, 41, 2, 88, 15, 6, 30]),
    ("tiny-internlm", dplan.TINY_INTERNLM, 1, False, [4, 5, 6, 1, 28, 13, 13, 7, 0, 22]),
]


@pytest.mark.parametrize("name,spec,seed,bias,ids", CASES, ids=[c[0] for c in CASES])
def test_teacher_logits_match_transformers(name, spec, seed, bias, ids):
    model = build(spec, seed, encode=oc.c_encode)
    if bias:
        model = _with_bias(model, seed + 100)
    assert len(ids) <= spec.max_seq
    want_model = _load_hf(model, bias)
    with torch.no_grad():
        want = want_model(torch.tensor([ids], dtype=torch.long)).logits[0].numpy()
    got = so.teacher_logits(model, ids)
    assert got.shape == want.shape == (len(ids), spec.vocab)
    scale = float(np.abs(want).max())
    err = float(np.abs(got - want).max())
    # two float32 evaluations in different summation orders (measured: 1e-7 .. 2e-6 of the
    # logit scale); a structural mistake is O(1)
    assert err <= 2e-5 * max(scale, 1.0), (name, err, scale)
    assert (got.argmax(-1) == want.argmax(-1)).all()


def test_greedy_ids_follow_the_transformers_argmax():
    """greedy_ids is the argmax chain of those logits: regenerate it through the independent
    model, one token at a time (full re-evaluation of the prefix, no cache)."""
    spec, seed, prompt = dplan.MEDIUM_LLAMA, 3, [9, 1, 4]
    model = build(spec, seed, encode=oc.c_encode)
    ids, margins = so.greedy_ids(model, prompt, 12, ignore_eos=True, return_margins=True)
    hf = _load_hf(model, False)
    seq = list(prompt)
    for tok, margin in zip(ids, margins):
        with torch.no_grad():
            logits = hf(torch.tensor([seq], dtype=torch.long)).logits[0, -1].numpy()
        if margin > 1e-3:  # a pick thinner than float32 noise says nothing about either side
            assert int(logits.argmax()) == tok, (seq, tok, margin)
        seq.append(tok)
