"""GPU: the session surface the reference's CLI and chat callers drive."""

from __future__ import annotations

import pytest
import torch

from deepfold_amd import decodev2 as dv2
from deepfold_amd.decodev2.synth import build
from oracle import step_oracle as so

pytestmark = pytest.mark.gpu

PROMPT = [4, 5, 6, 7, 1, 2, 3, 4, 9, 8]


ROOMY = dv2.with_max_seq(dv2.TINY_LLAMA, 64)


def make(spec=ROOMY, seed=1, **kw):
    model = build(spec, seed, packed_embed=True)
    loop = dv2.DecodeV2Loop.from_weights(dv2.DeviceWeights.from_synth(model, "cuda"), **kw)
    return model, loop


@pytest.mark.parametrize("spec", [ROOMY, dv2.with_max_seq(dv2.TINY_INTERNLM, 64)])
@pytest.mark.parametrize("graphs", [False, True])
def test_generate_gives_the_oracle_ids(spec, graphs):
    print("session", spec.name, graphs, flush=True)
    model, loop = make(spec)
    want = so.greedy_ids(model, PROMPT, 9, ignore_eos=True)
    if graphs:
        assert loop.warmup() > 0
        assert loop.capture_graphs() == "decodev2" and loop.graph_error is None
    seen = []
    for _ in range(2):  # a second request starts from a clean state
        seen.clear()
        g = loop.generate(torch.tensor(PROMPT), 9, on_token=seen.append)
        assert g.tokens == want == seen
        assert g.prompt_len == len(PROMPT) and g.decode_steps == len(g.tokens) - 1
        assert g.graph == ("decodev2" if graphs else "off") and not g.interrupted and g.stop_token is None
        assert g.prefill_ms > 0 and g.decode_ms > 0 and g.decode_tok_s > 0 and g.prefill_tok_s > 0
        assert loop.kv.seq_len == len(PROMPT) + len(want) - 1 == int(loop.state.valid_len.item())
    assert len(want) == 9
    assert loop.plan.family == spec.family and loop.kv.mib > 0
    assert loop.prefill_chunk == min(32, spec.max_seq)


def test_stop_tokens_budget_and_interruption():
    model, loop = make()
    want = so.greedy_ids(model, PROMPT, 9, ignore_eos=True)
    g = loop.generate(PROMPT, 9, stop=[want[3]])
    cut = want.index(want[3])
    assert g.tokens == want[:cut + 1] and g.stop_token == want[3]
    assert loop.generate(PROMPT, 0).tokens == []
    assert loop.generate(PROMPT, 1).tokens == want[:1]
    calls = []
    g = loop.generate(PROMPT, 9, should_stop=lambda: len(calls) >= 2 or calls.append(0) is not None)
    assert g.interrupted and g.tokens == want[:2]
    with pytest.raises(ValueError):
        loop.generate([], 4)
    with pytest.raises(ValueError):
        loop.generate(list(range(loop.max_seq + 1)), 4)
    with pytest.raises(ValueError):
        loop.generate(PROMPT, 4, speculate=4, draft="ngram")


def test_suffix_after_a_sealed_token_equals_one_long_prompt():
    """A chat turn: prompt, a few generated tokens, then the next user text is appended
    to the cache instead of replaying everything."""
    model, loop = make()
    first = loop.generate(PROMPT, 4)
    loop.seal_last(first.tokens[-1])          # the last sampled token was never fed back
    have = len(PROMPT) + len(first.tokens)
    assert loop.kv.seq_len == have
    suffix = [3, 1, 4, 1, 5]
    logits = loop.forward(suffix, have)
    g = loop.decode_from_logits(logits, 6, prompt_len=have + len(suffix))
    whole = so.greedy_ids(model, PROMPT + first.tokens + suffix, 6, ignore_eos=True)
    assert g.tokens == whole
    with pytest.raises(ValueError):
        loop.prefill_from([], 0)
    with pytest.raises(ValueError):
        loop.prefill_from([1, 2], loop.max_seq - 1)


def test_generation_stops_at_the_end_of_the_cache():
    spec = dv2.with_max_seq(dv2.TINY_LLAMA, 16)
    model, loop = make(spec)
    g = loop.generate(PROMPT, 50)
    assert len(PROMPT) + g.decode_steps == spec.max_seq and len(g.tokens) == g.decode_steps + 1
    assert g.tokens == so.greedy_ids(model, PROMPT, len(g.tokens), ignore_eos=True)
    loop.seal_last(1)  # no room: a no-op
    assert int(loop.state.valid_len.item()) == spec.max_seq


def test_weight_bytes_and_the_torch_glue_path(tmp_path):
    model, loop = make(fused_prefill=False)
    w = loop.weights
    want = w.nbytes + w.embed.nbytes + 2 * (w.final_norm.numel() + sum(ly.norm1.numel() + ly.norm2.numel() for ly in w.layers))
    assert loop.weight_bytes == want
    assert loop.generate(PROMPT, 5).tokens == so.greedy_ids(model, PROMPT, 5, ignore_eos=True)
    path = tmp_path / "m.chr"
    dv2.write_synth_chr(model, path)
    from_file = dv2.DecodeV2Loop.from_chr(path, model.spec)
    assert from_file.weight_bytes == want
    assert from_file.generate(PROMPT, 5).tokens == so.greedy_ids(model, PROMPT, 5, ignore_eos=True)
