"""The whole-step CPU oracle, piece by piece, against library routines and
closed forms (CPU only), plus the host-side logic of the synthetic models."""

from __future__ import annotations

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from deepfold_amd.decodev2 import plan as dplan
from deepfold_amd.decodev2.linear import internlm_row_order
from deepfold_amd.decodev2.rope import rope_tables_numpy
from deepfold_amd.decodev2.synth import build
from oracle import nf4_oracle as oc
from oracle import step_oracle as so


def test_rms_and_silu_match_torch():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((3, 96)).astype(np.float32) * 2
    w = (1 + 0.3 * rng.standard_normal(96)).astype(np.float32)
    want = F.rms_norm(torch.from_numpy(x), (96,), torch.from_numpy(w), 1e-6).numpy()
    assert np.allclose(so.rms(x, w, 1e-6), want, rtol=2e-6, atol=2e-6)
    assert np.allclose(so.silu(x), F.silu(torch.from_numpy(x)).numpy(), rtol=2e-6, atol=2e-6)


def test_rope_tables_and_rotation():
    cos, sin = so.rope_tables(32, 16, 10000.0)
    pc, ps = rope_tables_numpy(32, 16, 10000.0)
    assert (cos == pc).all() and (sin == ps).all()           # product tables == oracle tables
    assert (cos[:, :8] == cos[:, 8:]).all() and (sin[0] == 0).all() and (cos[0] == 1).all()
    inv = 1.0 / (10000.0 ** (np.arange(0, 16, 2) / 16.0))
    assert np.allclose(cos[5, :8], np.cos(5 * inv), atol=1e-6)
    rng = np.random.default_rng(1)
    t = rng.standard_normal((4, 3, 16)).astype(np.float32)
    pos = np.array([0, 1, 7, 31])
    r = so.apply_rope(t, cos[pos], sin[pos])
    assert np.allclose(r[0], t[0])                            # position 0 is the identity
    assert np.allclose((r ** 2).sum(-1), (t ** 2).sum(-1), rtol=1e-5)   # a rotation keeps norms
    # pair (d, d+8) rotates by angle pos*inv[d]: check one pair as a complex product
    z = (t[2, 1, 3] + 1j * t[2, 1, 11]) * np.exp(1j * 7 * inv[3])
    assert np.allclose([r[2, 1, 3], r[2, 1, 11]], [z.real, z.imag], atol=1e-5)
    # relative-position property: <rope(q,m), rope(k,n)> depends on m-n only
    q = rng.standard_normal((1, 1, 16)).astype(np.float32)
    k = rng.standard_normal((1, 1, 16)).astype(np.float32)
    d1 = (so.apply_rope(q, cos[9:10], sin[9:10]) * so.apply_rope(k, cos[4:5], sin[4:5])).sum()
    d2 = (so.apply_rope(q, cos[20:21], sin[20:21]) * so.apply_rope(k, cos[15:16], sin[15:16])).sum()
    assert abs(d1 - d2) < 1e-4


def test_attend_matches_sdpa_and_ignores_the_tail():
    spec = dplan.ArchSpec("t", "llama_swiglu", 1, 64, 8, 2, 8, 64, 32, 12)
    rng = np.random.default_rng(2)
    q = rng.standard_normal((1, 8, 8)).astype(np.float32)
    k = rng.standard_normal((12, 2, 8)).astype(np.float32)
    v = rng.standard_normal((12, 2, 8)).astype(np.float32)
    got = so.attend(q, k, v, spec, 7)
    tq = torch.from_numpy(q).reshape(1, 2, 4, 8)
    tk = torch.from_numpy(k[:7]).permute(1, 0, 2).unsqueeze(0)
    tv = torch.from_numpy(v[:7]).permute(1, 0, 2).unsqueeze(0)
    want = F.scaled_dot_product_attention(tq, tk, tv, scale=spec.attn_scale).reshape(1, 64).numpy()
    assert np.allclose(got, want, atol=2e-6)
    k2, v2 = k.copy(), v.copy()
    k2[7:], v2[7:] = 1e4, -1e4
    assert np.allclose(so.attend(q, k2, v2, spec, 7), got, atol=1e-6)


def test_linear_is_decode_then_matmul():
    rng = np.random.default_rng(3)
    w = (rng.standard_normal((10, 130)) * 0.05).astype(np.float32)
    p, s = oc.c_encode(w)

    class M:  # minimal matrix record
        packed, scale, M, K, bias = p, s, 10, 130, rng.standard_normal(10).astype(np.float32)

    x = rng.standard_normal((3, 130)).astype(np.float32)
    want = torch.from_numpy(x) @ torch.from_numpy(oc.c_decode(p, s, 10, 130)).T + torch.from_numpy(M.bias)
    assert np.allclose(so.linear(M, x), want.numpy(), atol=1e-5)


@pytest.mark.parametrize("spec", [dplan.TINY_INTERNLM,
                                  dplan.ArchSpec("i", "internlm_gqa", 1, 128, 8, 2, 16, 64, 16, 8)])
def test_internlm_row_order_equals_the_oracle_split(spec):
    rng = np.random.default_rng(4)
    y = rng.standard_normal((2, spec.wqkv_out)).astype(np.float32)
    q, k, v = so.split_internlm(y, spec)
    perm = y[:, internlm_row_order(spec)]
    assert (perm[:, : spec.q_dim] == q.reshape(2, -1)).all()
    assert (perm[:, spec.q_dim: spec.q_dim + spec.kv_dim] == k.reshape(2, -1)).all()
    assert (perm[:, spec.q_dim + spec.kv_dim:] == v.reshape(2, -1)).all()


def test_synth_build_is_seeded_and_ordered():
    a = build(dplan.TINY_LLAMA, 0, encode=oc.c_encode)
    b = build(dplan.TINY_LLAMA, 0, encode=oc.c_encode)
    c = build(dplan.TINY_LLAMA, 1, encode=oc.c_encode)
    assert (a.layers[1].down.packed == b.layers[1].down.packed).all()
    assert (a.lm_head.packed != c.lm_head.packed).any()
    # first draw of the stream is layer 0's q matrix: [hidden, hidden] * 0.05
    rng = np.random.default_rng(0)
    w0 = rng.standard_normal((64, 64), dtype=np.float32) * np.float32(0.05)
    p0, s0 = oc.c_encode(w0)
    assert (a.layers[0].q.packed == p0).all() and (a.layers[0].q.scale.view(np.uint16) == s0.view(np.uint16)).all()
    assert a.layers[0].q.K_pad == 64 and a.layers[0].down.K == 128 and a.embed.shape == (32, 64)
    i = build(dplan.TINY_INTERNLM, 1, encode=oc.c_encode)
    assert i.layers[0].q is None and i.layers[0].wqkv.M == dplan.TINY_INTERNLM.wqkv_out


def test_arch_spec_rejects_bad_shapes():
    with pytest.raises(ValueError):
        dplan.ArchSpec("x", "gpt", 1, 64, 4, 2, 16, 128, 32, 16)
    with pytest.raises(ValueError):
        dplan.ArchSpec("x", "llama_swiglu", 1, 64, 4, 3, 16, 128, 32, 16)
    with pytest.raises(ValueError):
        dplan.ArchSpec("x", "llama_swiglu", 1, 96, 4, 2, 16, 128, 32, 16)
    with pytest.raises(ValueError):
        dplan.ArchSpec("x", "llama_swiglu", 1, 64, 4, 2, 16, 100, 32, 16)
    with pytest.raises(ValueError):
        dplan.ArchSpec("x", "llama_swiglu", 1, 64, 4, 2, 16, 128, 32, 16, eos_id=40)
    # byte accounting of the benchmark shapes
    assert dplan.QWEN25_14B.weight_bytes_per_token() == 7432519680
    assert dplan.QWEN25_3B.weight_bytes_per_token() == 1639276544
    assert dplan.QWEN25_14B.kv_bytes(2048) == 402653184


@pytest.mark.parametrize("spec,seed,prompt", [(dplan.TINY_LLAMA, 0, [1, 3, 5, 7]),
                                              (dplan.TINY_INTERNLM, 1, [4, 5, 6])])
def test_greedy_oracle_runs_and_is_reproducible(spec, seed, prompt):
    model = build(spec, seed, encode=oc.c_encode)
    ids, margins = so.greedy_ids(model, prompt, 8, return_margins=True)
    assert 1 <= len(ids) <= 8 and all(0 <= t < spec.vocab for t in ids)
    assert ids == so.greedy_ids(model, prompt, 8)
    assert len(margins) == len(ids) and all(m >= 0 for m in margins)
    tl = so.teacher_logits(model, prompt)
    assert tl.shape == (len(prompt), spec.vocab) and int(tl[-1].argmax()) == ids[0]
    # a dirty KV tail cannot change a step
    c1, c2 = so.OracleCache(spec), so.OracleCache(spec)
    so.step_logits(model, c1, 1)
    so.step_logits(model, c2, 1)
    c2.k[:, -1], c2.v[:, -1] = 1e4, 1e4
    assert np.allclose(so.step_logits(model, c1, 3), so.step_logits(model, c2, 3))


def test_wide_gap_stream_fixture_is_what_the_oracle_gives():
    """``tests/golden/greedy_margin_seeds.json`` (made by ``scan_greedy_margins.py``): two of its
    streams recomputed here, ids and smallest gap; the list is sorted by that gap."""
    import importlib.util
    import json
    import os

    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    with open(os.path.join(here, "greedy_margin_seeds.json")) as f:
        fixture = json.load(f)
    spec = importlib.util.spec_from_file_location("scan_greedy_margins",
                                                  os.path.join(here, "scan_greedy_margins.py"))
    scan = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(scan)
    assert fixture["prompt"] == scan.PROMPT and fixture["n_new"] == scan.N_NEW
    gaps = [r["min_gap_bf16_steps"] for r in fixture["streams"]]
    assert gaps == sorted(gaps, reverse=True) and len(gaps) >= 8 and gaps[7] >= 2.0
    for row in (fixture["streams"][0], fixture["streams"][7]):
        again = scan.one(row["seed"])
        assert again["ids"] == row["ids"] and len(row["ids"]) == 64
        assert abs(again["min_gap_bf16_steps"] - row["min_gap_bf16_steps"]) < 1e-9
