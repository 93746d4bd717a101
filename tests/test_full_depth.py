"""GPU: the four decode configurations at their full depth and width, as properties.

The CPU oracle cannot follow a 36- to 64-layer model of these widths, so nothing here is
compared with it (the 2-layer models at the same widths in ``test_decodev2.py`` are).  What a
full-size run must still satisfy by construction is checked instead: the prefill leaves exactly
the prompt in the cache, every logit is finite, the captured graph takes the same steps as the
eager launches, bit for bit, the device-side position and cache length advance by one per
step, and the folded launch schedule stays as close to the reference's sequence of launches as
it does on the small models.  Prompts are what each configuration names: 512 tokens (3B, 14B),
1024 tokens in 32-position chunks (20B), and a cache filled to 1791 of 2048 rows (32B).
"""

from __future__ import annotations

import pytest
import torch

from deepfold_amd import decodev2 as dv2
from deepfold_amd.decodev2 import step as step_mod

pytestmark = pytest.mark.gpu

N_NEW = 16

#: name, spec, prompt tokens, prefill chunk width (None: the launches' own 64)
CONFIGS = [
    ("3b", dv2.QWEN25_3B, 512, None),
    ("14b", dv2.QWEN25_14B, 512, None),
    ("20b", dv2.INTERNLM25_20B, 1024, 32),
    ("32b", dv2.QWEN25_32B, 2048 - 256 - 1, None),
]


def say(*a):
    print(*a, flush=True)


@pytest.mark.parametrize("name,spec,prompt_len,width", CONFIGS, ids=[c[0] for c in CONFIGS])
def test_full_depth_decode(name, spec, prompt_len, width, monkeypatch):
    say("full depth", name, spec.n_layers, "layers, prompt", prompt_len, "chunks of", width or 64)
    weights = dv2.DeviceWeights.random(spec, seed=2027)
    state = dv2.DecodeState.allocate(spec, device="cuda")
    g = torch.Generator(device="cpu")
    g.manual_seed(11)
    prompt = torch.randint(0, spec.vocab, (prompt_len,), generator=g).tolist()
    pre = dv2.ChunkPrefill(state, weights, width=width)
    assert pre.width == (width or 64)

    def prefill():
        state.reset()
        dv2.consume_prompt(state, weights, prompt, prefill=pre)
        torch.cuda.synchronize()
        # the prefill commits nothing: it leaves the prompt in the cache and the next id
        assert int(state.valid_len.item()) == prompt_len and int(state.position.item()) == prompt_len
        assert bool(torch.isfinite(state.arena.logits.float()).all())
        first = int(state.next_token.item())
        assert 0 <= first < spec.vocab
        state.token.copy_(state.next_token)
        return first

    # eager steps
    first = prefill()
    eager, eager_logits = [], []
    for i in range(N_NEW):
        dv2.greedy_decode(state, weights)
        eager.append(int(state.token.item()))
        eager_logits.append(state.arena.logits.clone())
        assert int(state.position.item()) == prompt_len + i + 1
        assert int(state.valid_len.item()) == prompt_len + i + 1
        assert bool(torch.isfinite(state.arena.logits.float()).all()), i
    assert all(0 <= t < spec.vocab for t in eager)

    # the same prefill again (its graphs replayed: same first id), then the steps from a graph
    assert prefill() == first
    graph = dv2.capture_greedy(state, weights, warmup=1)
    assert int(state.position.item()) == prompt_len and int(state.valid_len.item()) == prompt_len
    for i in range(N_NEW):
        graph.replay()
        torch.cuda.synchronize()
        assert int(state.token.item()) == eager[i], (name, i)
        assert torch.equal(state.arena.logits, eager_logits[i]), (name, i)
        assert int(state.position.item()) == prompt_len + i + 1
        assert int(state.valid_len.item()) == prompt_len + i + 1

    # the reference's sequence of launches (separate RMSNorm launches, a merge launch) on the
    # same cache: teacher-forced with the folded schedule's ids, logits close at every step
    # (two bf16 paths through L layers drift apart like a random walk over the 2 L + 1 rounded
    # hand-overs: the form of the bound test_decodev2.py holds the GPU path to against the fp32
    # oracle; measured here 1.7 .. 2.3 of sqrt(2 L + 1) * 2^-9 of the logit scale, 3 allowed)
    assert prefill() == first
    scale = max(float(l.float().abs().max()) for l in eager_logits)
    bound = 3.0 * (2 * spec.n_layers + 1) ** 0.5 * 2.0 ** -9 * scale
    worst = 0.0
    for i in range(N_NEW):
        dv2.greedy_decode(state, weights, schedule="plain")
        diff = float((state.arena.logits.float() - eager_logits[i].float()).abs().max())
        worst = max(worst, diff)
        assert diff <= bound + 1e-3, (name, i, diff, bound, scale)
        state.token.fill_(eager[i])   # stay on the folded schedule's stream
    say(f"  {name}: graph == eager over {N_NEW} steps; plain against folded schedule: worst logit "
        f"difference {worst:.3f}, bound {bound:.3f} (logit scale {scale:.2f})")

    # the folded schedule with every launch summing x^2 for itself instead of taking the sum from
    # the launch that wrote x (all four models take the hand-over: every writer of the stream
    # runs on a kernel that stages x in LDS): the same statistic added in another order, so a few
    # of the normalised activations round the other way and the logits drift as they do between
    # the two schedules above
    assert step_mod._sumsq_handover(weights)
    monkeypatch.setenv("CHR_DV2_SUMSQ", "0")
    assert not step_mod._sumsq_handover(weights)
    assert prefill() == first
    worst = 0.0
    for i in range(N_NEW):
        dv2.greedy_decode(state, weights)
        diff = float((state.arena.logits.float() - eager_logits[i].float()).abs().max())
        worst = max(worst, diff)
        assert diff <= bound + 1e-3, (name, i, diff, bound, scale)
        state.token.fill_(eager[i])
    say(f"  {name}: without the sum-of-squares hand-over: worst logit difference {worst:.3f}")
    monkeypatch.delenv("CHR_DV2_SUMSQ")
    del graph, pre, state, weights
    torch.cuda.empty_cache()
