"""GPU parity: every NF4 kernel, through the C ABI, against the CPU oracle."""

from __future__ import annotations

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from deepfold_amd import nf4
from deepfold_amd.nf4 import plan as pyplan
from oracle import nf4_oracle as oc

from helpers import (DEV, MAX_REL, bf16_bits, bf16_tensor, check_linear, rand_x, to_f32, ulp_bf16, up,
                     up_scale, staged_gemv_model, takes_staged_gemv)

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def blobs(m, k, seed, **kw):
    p, s = oc.toy_blobs(m, k, seed, **kw)
    return p, s, up(p), up_scale(s)


def quantized(m, k, seed, sigma=0.02):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((m, k)) * sigma).astype(np.float32)
    p, s = oc.c_encode(w)
    return w, p, s, up(p), up_scale(s)


# ---------------------------------------------------------------- codec twins
@pytest.mark.parametrize("m,k", [(1, 64), (128, 256), (130, 65), (7, 1), (33, 5120), (4, 200)])
def test_dequant_bit_exact(m, k):
    say("dequant", m, k)
    p, s, dp, ds = blobs(m, k, 100 + m + k)
    got = nf4.nf4_dequant(dp, ds, m, k, oc.k_pad(k)).cpu().numpy()
    want = oc.c_decode(p, s, m, k)
    assert (got.view(np.uint32) == want.view(np.uint32)).all()


def test_dequant_every_scale_pattern():
    # all finite positive binary16 scales (incl. subnormals) x all 16 codes
    bits = np.arange(1, 0x7C00, dtype=np.uint16)
    m = bits.size
    s = bits.view(np.float16).reshape(m, 1)
    codes = np.tile(np.arange(16, dtype=np.uint8), 4)[None, :].repeat(m, 0)
    p = oc.np_pack(codes)
    got = nf4.nf4_dequant(up(p), up_scale(s), m, 64, 64).cpu().numpy()
    want = oc.c_decode(p, s, m, 64)
    assert (got.view(np.uint32) == want.view(np.uint32)).all()


def test_dequant_golden_row():
    w = (np.arange(64, dtype=np.float32) / np.float32(63)).reshape(1, 64)
    p, s = oc.c_encode(w)
    got = nf4.nf4_dequant(up(p), up_scale(s), 1, 64, 64).cpu().numpy()
    assert (got.view(np.uint32) == oc.c_decode(p, s, 1, 64).view(np.uint32)).all()
    # zero matrix decodes to +0 bits
    z = nf4.nf4_dequant(up(np.full((3, 32), 0x77, np.uint8)), up_scale(np.full((3, 1), 1.0, np.float16)), 3, 64, 64)
    assert (z.cpu().numpy().view(np.uint32) == 0).all()


@pytest.mark.parametrize("m,k,sigma", [(1, 64, 1.0), (2, 64, 1.0), (64, 256, 0.02), (130, 65, 0.05),
                                       (17, 5120, 0.02), (5, 1, 3.0), (9, 200, 1e-3)])
def test_quantize_bit_exact(m, k, sigma):
    say("quantize", m, k)
    rng = np.random.default_rng(m * 1000 + k)
    w = (rng.standard_normal((m, k)) * sigma).astype(np.float32)
    if m == 2 and k == 64:
        i = np.arange(64, dtype=np.float32)
        w = np.stack([i / np.float32(63), (np.float32(2) * i - np.float32(63)) / np.float32(63)]).astype(np.float32)
    dp, ds = nf4.nf4_quantize(up(w))
    p, s = oc.c_encode(w)
    assert (dp.cpu().numpy() == p).all()
    assert (ds.cpu().numpy().view(np.uint16) == s.view(np.uint16)).all()


def test_quantize_edge_groups():
    w = np.zeros((6, 64), dtype=np.float32)
    w[1] = 1e-12            # scale underflows binary16 -> zero group
    w[2] = 1e6              # scale overflows -> clamp to 65504
    w[3] = -2.25
    w[4, :] = np.linspace(-1, 1, 64)
    w[5, 0] = 6.1e-5        # binary16 subnormal/normal boundary
    dp, ds = nf4.nf4_quantize(up(w))
    p, s = oc.c_encode(w)
    assert (dp.cpu().numpy() == p).all()
    assert (ds.cpu().numpy().view(np.uint16) == s.view(np.uint16)).all()
    bad = w.copy()
    bad[2, 5] = np.nan
    with pytest.raises(ValueError):
        nf4.nf4_quantize(up(bad))
    bad[2, 5] = np.inf
    with pytest.raises(ValueError):
        nf4.nf4_quantize(up(bad))


def test_quantize_midpoint_neighbourhood():
    mids = np.array([0xBF591CD8, 0xBF1C5270, 0xBEEB8480, 0xBEADEA76, 0xBE703CEC, 0xBE0D38BC,
                     0xBD3A7871, 0x3D22FAFF, 0x3DF64862, 0x3E5067E0, 0x3E9582D4, 0x3EC753F9,
                     0x3F006D04, 0x3F248DAF, 0x3F5C89DA], dtype=np.int64)
    near = (mids[:, None] + np.arange(-33, 30)[None, :]).astype(np.uint32).view(np.float32)
    w = np.concatenate([np.ones((15, 1), np.float32), near], axis=1)  # scale pinned to 1
    dp, ds = nf4.nf4_quantize(up(w))
    p, s = oc.c_encode(w)
    assert (dp.cpu().numpy() == p).all() and (ds.cpu().numpy().view(np.uint16) == s.view(np.uint16)).all()


def test_embed_rows_bit_exact():
    m, k = 300, 200
    p, s, dp, ds = blobs(m, k, 77)
    ids = np.array([0, 299, 5, 5, 17, 128], dtype=np.int64)
    got = nf4.nf4_embed_rows(dp, ds, up(ids), k)
    want = oc.bf16_round_bits(oc.c_decode(p, s, m, k)[ids])
    assert (bf16_bits(got) == want).all()


# ---------------------------------------------------------------------- GEMV
GEMV_SHAPES = [(128, 256), (130, 65), (4, 64), (1, 2048), (37, 5120), (260, 13824), (2050, 1024),
               (8200, 128), (16, 11008), (3, 192)]


@pytest.mark.parametrize("m,k", GEMV_SHAPES)
def test_gemv_toy_blobs(m, k):
    say("gemv", m, k)
    p, s, dp, ds = blobs(m, k, 20260912 + m + k)
    x = rand_x(k, None, m)
    y = nf4.nf4_gemv(dp, ds, bf16_tensor(x), m, k, oc.k_pad(k))
    assert tuple(y.shape) == (m, 1)
    ref = oc.c_matmul_f64(oc.c_decode(p, s, m, k), x[:, None])
    model = staged_gemv_model(p, s, m, k, x) if takes_staged_gemv(m, k) else None
    check_linear(y, ref, what=f"gemv {m}x{k}", model=model)
    # same inputs, same bits
    y2 = nf4.nf4_gemv(dp, ds, bf16_tensor(x), m, k, oc.k_pad(k))
    assert (bf16_bits(y) == bf16_bits(y2)).all()


@pytest.mark.parametrize("m,k", [(152064, 5120), (151936, 2048), (92544, 6144), (27648, 5120),
                                 (5120, 13824), (5120, 27648)])
def test_gemv_full_size_sampled_rows(m, k, monkeypatch):
    """The vocabulary and FFN shapes of the benchmark architectures at full size: every
    wavefront of the staged launch walks several row groups.  2048 sampled rows are held to
    the full bounds (oracle, and the staged kernel's arithmetic written out on the CPU); all
    rows must agree with the plain kernel on the same inputs."""
    say("gemv full size", m, k)
    gen = torch.Generator(device=DEV)
    gen.manual_seed(m + k)
    w = torch.randn((m, k), generator=gen, device=DEV, dtype=torch.float32) * 0.02
    dp, ds = nf4.nf4_quantize(w)
    del w
    x = rand_x(k, None, 21)
    dx = bf16_tensor(x)
    assert takes_staged_gemv(m, k)
    y = nf4.nf4_gemv(dp, ds, dx, m, k, k)
    monkeypatch.setenv("CHR_NF4_GEMV_STAGED", "0")
    y0 = nf4.nf4_gemv(dp, ds, dx, m, k, k)
    a, b = to_f32(y).reshape(-1), to_f32(y0).reshape(-1)
    assert np.abs(a - b).max() <= MAX_REL * np.abs(b).max()
    rows = np.sort(np.random.default_rng(5).choice(m, 2048, replace=False))
    idx = torch.from_numpy(rows).to(DEV)
    p = dp.view(m, -1)[idx].cpu().numpy()
    sc = ds.view(m, -1)[idx].cpu().numpy()
    ref = oc.c_matmul_f64(oc.c_decode(p, sc, len(rows), k), x[:, None])
    check_linear(y.view(-1)[idx], ref, what=f"staged {m}x{k}, sampled rows",
                 model=staged_gemv_model(p, sc, len(rows), k, x))
    check_linear(y0.view(-1)[idx], ref, what=f"plain {m}x{k}, sampled rows")


def test_gemv_pad_codes_do_not_matter():
    m, k = 130, 65
    pa, sa = oc.toy_blobs(m, k, 5, pad_garbage=True)
    pb, _ = oc.toy_blobs(m, k, 5, pad_garbage=False)
    assert (pa != pb).any()
    x = bf16_tensor(rand_x(k, None, 1))
    ya = nf4.nf4_gemv(up(pa), up_scale(sa), x, m, k, 128)
    yb = nf4.nf4_gemv(up(pb), up_scale(sa), x, m, k, 128)
    assert (bf16_bits(ya) == bf16_bits(yb)).all()
    xn = bf16_tensor(rand_x(k, 5, 2))
    ga = nf4.nf4_gemm(up(pa), up_scale(sa), xn, m, k, 128)
    gb = nf4.nf4_gemm(up(pb), up_scale(sa), xn, m, k, 128)
    assert (bf16_bits(ga) == bf16_bits(gb)).all()


def test_gemv_zero_level_matrix():
    m, k = 64, 256
    _, s = oc.toy_blobs(m, k, 9)
    p = np.full((m, k // 2), 0x77, np.uint8)
    y = nf4.nf4_gemv(up(p), up_scale(s), bf16_tensor(rand_x(k, None, 3)), m, k, k)
    assert (to_f32(y) == 0).all()


def test_gemv_config1_shape_quantized_weights(monkeypatch):
    m, k = 13824, 5120
    say("gemv config 1", m, k)
    w, p, s, dp, ds = quantized(m, k, 1)
    x = rand_x(k, None, 2)
    y = nf4.nf4_gemv(dp, ds, bf16_tensor(x), m, k, k)
    ref = oc.c_matmul_f64(oc.c_decode(p, s, m, k), x[:, None])
    assert takes_staged_gemv(m, k)
    model = staged_gemv_model(p, s, m, k, x)
    check_linear(y, ref, what="config 1", model=model)
    # the float32 two-pass CPU linear of the reference agrees to the same bounds
    check_linear(y, oc.c_linear(p, s, m, k, x[:, None]), what="config 1 vs f32 oracle", ulps=1.5,
                 model=model)
    # the plain kernel (fp32 levels) on the same inputs: the tight bound against the oracle itself
    monkeypatch.setenv("CHR_NF4_GEMV_STAGED", "0")
    y0 = nf4.nf4_gemv(dp, ds, bf16_tensor(x), m, k, k)
    check_linear(y0, ref, what="config 1, plain kernel")


@pytest.mark.parametrize("staged", [0, 1])
@pytest.mark.parametrize("rows", [1, 2, 4])
def test_gemv_rows_per_wavefront_agree(rows, staged, monkeypatch):
    m, k = 1030, 5120
    p, s, dp, ds = blobs(m, k, 31)
    x = rand_x(k, None, 4)
    monkeypatch.setenv("CHR_NF4_GEMV_NR", str(rows))
    monkeypatch.setenv("CHR_NF4_GEMV_STAGED", str(staged))
    y = nf4.nf4_gemv(dp, ds, bf16_tensor(x), m, k, k)
    model = staged_gemv_model(p, s, m, k, x) if staged else None
    check_linear(y, oc.c_matmul_f64(oc.c_decode(p, s, m, k), x[:, None]),
                 what=f"NR={rows} staged={staged}", model=model)


@pytest.mark.parametrize("m,k", [(4100, 5120), (700, 13824), (2100, 6208), (9000, 2048)])
def test_gemv_staged_walks_many_groups_per_wavefront(m, k, monkeypatch):
    """More row groups than the 4096 wavefronts of a launch on some shapes, fewer on others, a
    K whose last half step is partly filled (6208), items that span two row groups."""
    p, s, dp, ds = blobs(m, k, 33)
    x = rand_x(k, None, 6)
    monkeypatch.setenv("CHR_NF4_GEMV_STAGED", "1")
    for rows in (1, 2):
        monkeypatch.setenv("CHR_NF4_GEMV_NR", str(rows))
        y = nf4.nf4_gemv(dp, ds, bf16_tensor(x), m, k, oc.k_pad(k))
        check_linear(y, oc.c_matmul_f64(oc.c_decode(p, s, m, k), x[:, None]),
                     what=f"staged {m}x{k} NR={rows}", model=staged_gemv_model(p, s, m, k, x))


def test_gemv_residual_add_may_alias_out():
    m, k = 2048, 2048
    p, s, dp, ds = blobs(m, k, 41)
    x = rand_x(k, None, 5)
    res = oc.bf16_round(np.random.default_rng(6).standard_normal(m).astype(np.float32))
    dest = bf16_tensor(res)
    out = nf4.nf4_gemv(dp, ds, bf16_tensor(x), m, k, k, dest, dest)
    assert out.data_ptr() == dest.data_ptr()
    ref = oc.c_matmul_f64(oc.c_decode(p, s, m, k), x[:, None]).reshape(-1) + res.astype(np.float64)
    check_linear(dest, ref, what="residual")
    # separate out and add give the same bits
    out2 = torch.empty(m, dtype=torch.bfloat16, device=DEV)
    nf4.nf4_gemv(dp, ds, bf16_tensor(x), m, k, k, out2, bf16_tensor(res))
    assert (bf16_bits(out2) == bf16_bits(dest)).all()


@pytest.mark.parametrize("m,k", [(256, 2048), (130, 65)])
def test_gemv_fused_rms(m, k, monkeypatch):
    p, s, dp, ds = blobs(m, k, 51)
    rng = np.random.default_rng(7)
    x = oc.bf16_round(rng.standard_normal(k).astype(np.float32) * 3)
    g = oc.bf16_round(1 + 0.1 * rng.standard_normal(k).astype(np.float32))
    eps = 1e-6
    y = nf4.nf4_gemv(dp, ds, bf16_tensor(x), m, k, oc.k_pad(k), rms_w=bf16_tensor(g), rms_eps=eps)
    inv = 1.0 / np.sqrt((x.astype(np.float64) ** 2).mean() + eps)
    xh = oc.bf16_round(((g.astype(np.float64) * x) * inv).astype(np.float32))
    # normalised x is rounded to bf16 before the dots; allow one bf16 step of x
    ref = oc.c_matmul_f64(oc.c_decode(p, s, m, k), xh[:, None])
    check_linear(y, ref, what="fused rms", ulps=4, model=staged_gemv_model(p, s, m, k, xh))
    # equals the two-launch form (same kernel family) bit for bit when the RMS rounding agrees
    h = torch.empty(k, dtype=torch.bfloat16, device=DEV)
    nf4.nf4_rms(bf16_tensor(x), bf16_tensor(g), h, eps)
    monkeypatch.setenv("CHR_NF4_GEMV_STAGED", "1")
    y2 = nf4.nf4_gemv(dp, ds, h, m, k, oc.k_pad(k))
    check_linear(y, to_f32(y2), what="fused rms vs rms+gemv", ulps=1)


@pytest.mark.parametrize("m,k", [(64, 512), (96, 1088), (40, 5120), (8, 13824)])
def test_gemv_fused_rms_is_deterministic_with_a_partial_tail_step(m, k, monkeypatch):
    """K whose last step is only partly filled: the staged copy of x zero-fills the unused
    slots and must never touch the used ones, whatever order the lanes run in."""
    p, s, dp, ds = blobs(m, k, 77)
    rng = np.random.default_rng(k)
    x = bf16_tensor(oc.bf16_round(rng.standard_normal(k).astype(np.float32)))
    g = bf16_tensor(oc.bf16_round(1 + 0.1 * rng.standard_normal(k).astype(np.float32)))
    h = torch.empty(k, dtype=torch.bfloat16, device=DEV)
    nf4.nf4_rms(x, g, h, 1e-6)
    monkeypatch.setenv("CHR_NF4_GEMV_STAGED", "1")  # the two-launch form in the same kernel family
    want = nf4.nf4_gemv(dp, ds, h, m, k, oc.k_pad(k))
    first = None
    for rep in range(25):
        y = nf4.nf4_gemv(dp, ds, x, m, k, oc.k_pad(k), rms_w=g, rms_eps=1e-6)
        bits = bf16_bits(y)
        if first is None:
            first = bits
            check_linear(y, to_f32(want), what="fused rms, partial tail", ulps=1)
        assert (bits == first).all(), rep


def test_gemv_nan_behaviour():
    m, k = 256, 512
    p, s, dp, ds = blobs(m, k, 61)
    x = rand_x(k, None, 8)
    xn = x.copy()
    xn[17] = np.nan
    y = to_f32(nf4.nf4_gemv(dp, ds, bf16_tensor(xn), m, k, k))
    assert not np.isfinite(y).any()        # a NaN in x poisons every row
    s2 = s.copy()
    s2[5, 3] = np.float16(np.nan)
    y = to_f32(nf4.nf4_gemv(dp, up_scale(s2), bf16_tensor(x), m, k, k)).reshape(-1)
    assert not np.isfinite(y[5])           # a NaN scale poisons its own row ...
    assert np.isfinite(np.delete(y, 5)).all()  # ... and only that row


def test_wrapper_rejects_lying_arguments():
    m, k = 128, 256
    p, s, dp, ds = blobs(m, k, 71)
    x = bf16_tensor(rand_x(k, None, 9))
    for bad in (
        lambda: nf4.nf4_gemv(dp[: m // 2], ds, x, m, k, k),
        lambda: nf4.nf4_gemv(dp, ds[: m // 2], x, m, k, k),
        lambda: nf4.nf4_gemv(dp, ds, x, m, k, k + 64),
        lambda: nf4.nf4_gemv(dp, ds, x[: k - 8], m, k, k),
        lambda: nf4.nf4_gemv(dp, ds, x.cpu(), m, k, k),
        lambda: nf4.nf4_gemv(dp, ds, x.to(torch.float16), m, k, k),
        lambda: nf4.nf4_gemm(dp, ds, x.reshape(k, 1).repeat(1, 33), m, k, k),
        lambda: nf4.nf4_gemm(dp[: m // 2], ds, x.reshape(k, 1).repeat(1, 4), m, k, k),
    ):
        with pytest.raises(RuntimeError):
            bad()
    # the context is still healthy
    check_linear(nf4.nf4_gemv(dp, ds, x, m, k, k),
                 oc.c_matmul_f64(oc.c_decode(p, s, m, k), to_f32(x)[:, None]), what="after refusals")


# ----------------------------------------------------------------- QKV / SwiGLU
@pytest.mark.parametrize("mq,mk,k,bias", [(2048, 256, 2048, True), (5120, 1024, 5120, True),
                                          (64, 32, 64, False), (130, 33, 65, True)])
def test_qkv_equals_three_gemvs(mq, mk, k, bias):
    say("qkv", mq, mk, k)
    kp = oc.k_pad(k)
    mats = [blobs(mq, k, 81), blobs(mk, k, 82), blobs(mk, k, 83)]
    rng = np.random.default_rng(10)
    x = rand_x(k, None, 11)
    biases = [oc.bf16_round(rng.standard_normal(m).astype(np.float32)) if bias else None
              for m in (mq, mk, mk)]
    outs = [torch.empty(m, dtype=torch.bfloat16, device=DEV) for m in (mq, mk, mk)]
    dx = bf16_tensor(x)
    nf4.nf4_qkv(mats[0][2], mats[0][3], mats[1][2], mats[1][3], mats[2][2], mats[2][3], dx,
                mq, mk, mk, k, kp, outs[0], outs[1], outs[2],
                *[None if b is None else bf16_tensor(b) for b in biases])
    for (p, s, dp, ds), m, b, o in zip(mats, (mq, mk, mk), biases, outs):
        ref = oc.c_matmul_f64(oc.c_decode(p, s, m, k), x[:, None]).reshape(-1)
        if b is not None:
            ref = ref + b
        model = None
        if takes_staged_gemv(mq + 2 * mk, k):
            model = staged_gemv_model(p, s, m, k, x) + (0 if b is None else b)
        check_linear(o, ref, what="qkv", model=model)
        single = torch.empty(m, dtype=torch.bfloat16, device=DEV)
        nf4.nf4_gemv(dp, ds, dx, m, k, kp, single, None if b is None else bf16_tensor(b))
        assert np.abs(to_f32(single) - to_f32(o)).max() <= 1e-3 + np.abs(to_f32(o)).max() * 2 ** -7


@pytest.mark.parametrize("m,k", [(11008, 2048), (512, 5120), (130, 65), (4100, 256)])
def test_swiglu_equals_pair(m, k):
    say("swiglu", m, k)
    kp = oc.k_pad(k)
    pg, sg, dpg, dsg = blobs(m, k, 91)
    pu, su, dpu, dsu = blobs(m, k, 92)
    x = rand_x(k, None, 12)
    out = torch.empty(m, dtype=torch.bfloat16, device=DEV)
    nf4.nf4_swiglu(dpg, dsg, dpu, dsu, bf16_tensor(x), m, k, kp, out)
    g = oc.c_matmul_f64(oc.c_decode(pg, sg, m, k), x[:, None]).reshape(-1)
    u = oc.c_matmul_f64(oc.c_decode(pu, su, m, k), x[:, None]).reshape(-1)
    ref = g / (1 + np.exp(-g)) * u
    model = None
    if takes_staged_gemv(2 * m, k):
        gm = staged_gemv_model(pg, sg, m, k, x)
        model = gm / (1 + np.exp(-gm)) * staged_gemv_model(pu, su, m, k, x)
    check_linear(out, ref, what="swiglu", ulps=1.5, model=model)


# ----------------------------------------------------------------- ring GEMV kernels
# The ring kernels take every staged launch whose row length is a multiple of 4..7 half steps
# of 1024 weights or one half step short of a
# multiple of 5..8; CHR_NF4_GEMV_RING=0 keeps such launches on the compiler-pipelined kernel.
RING_ROWS = [
    (4100, 4096),   # 4 half steps, x of the row in registers; a pass and four rows more
    (9000, 5120),   # 5 half steps, two passes and a part of a third
    (3, 5120),      # fewer rows than wavefronts
    (4500, 6144), (4200, 7168), (4100, 8192),   # one piece of 6, of 7; two pieces of 4
    (700, 13824),   # two pieces of 7 half steps
    (300, 16384),   # four pieces of 4
    (4300, 6208),   # last half step partly filled (4 of 64 lanes)
    (4200, 5056),   # the same with x in registers
    (4100, 4000),   # K below K_pad
    (4200, 11008),  # 11 half steps: two pieces of 6, the last with an empty slot
    (600, 27648),   # 27: four pieces of 7, the last with an empty slot
    (4200, 10950),  # 11 half steps, the last partly filled, then the empty slot
    (500, 19456),   # 19: four pieces of 5 with an empty slot (x stays in LDS)
    (400, 23552),   # 23: four pieces of 6 with an empty slot
    (300, 31744),   # 31: four pieces of 8 with an empty slot (the only lengths that take 8)
]


@pytest.mark.parametrize("terms", [1, 2, 3])
@pytest.mark.parametrize("m,k", RING_ROWS)
def test_ring_gemv(m, k, terms, monkeypatch):
    say("ring gemv", m, k, terms)
    monkeypatch.setenv("CHR_NF4_GEMV_STAGED", "1")
    monkeypatch.setenv("CHR_NF4_GEMV_RING", "1")
    monkeypatch.setenv("CHR_NF4_GEMV_TERMS", str(terms))
    p, s, dp, ds = blobs(m, k, 700 + m + k)
    x = rand_x(k, None, 13)
    res = oc.bf16_round(np.random.default_rng(m).standard_normal(m).astype(np.float32))
    y = nf4.nf4_gemv(dp, ds, bf16_tensor(x), m, k, oc.k_pad(k))
    ref = oc.c_matmul_f64(oc.c_decode(p, s, m, k), x[:, None]).reshape(-1)
    model = staged_gemv_model(p, s, m, k, x, terms=terms)
    check_linear(y, ref, what=f"ring {m}x{k}", model=model)
    # with a residual, and the same bits on a second launch
    out = torch.empty(m, dtype=torch.bfloat16, device=DEV)
    nf4.nf4_gemv(dp, ds, bf16_tensor(x), m, k, oc.k_pad(k), out, bf16_tensor(res))
    check_linear(out, ref + res, what=f"ring {m}x{k} + residual", model=model + res)
    out2 = torch.empty(m, dtype=torch.bfloat16, device=DEV)
    nf4.nf4_gemv(dp, ds, bf16_tensor(x), m, k, oc.k_pad(k), out2, bf16_tensor(res))
    assert (bf16_bits(out) == bf16_bits(out2)).all()
    # the compiler-pipelined kernel on the same inputs: same arithmetic, another order of sums
    monkeypatch.setenv("CHR_NF4_GEMV_RING", "0")
    y0 = nf4.nf4_gemv(dp, ds, bf16_tensor(x), m, k, oc.k_pad(k))
    check_linear(y, to_f32(y0), what=f"ring {m}x{k} vs pipelined", ulps=1)


@pytest.mark.parametrize("m,k", [(70000, 5120), (45000, 6144), (33000, 7168), (20000, 13824), (12000, 16384)])
def test_ring_gemv_many_rows_per_wavefront(m, k, monkeypatch):
    """The ring in its steady state (4 to 17 rows per wavefront, every slot requested again a
    few steps after it was consumed, waits by count): against the compiler-pipelined kernel,
    whose waits are the compiler's own, to one bf16 step, sampled rows against the fp64 oracle,
    and the same bits on every one of five launches."""
    say("ring gemv, many rows", m, k)
    monkeypatch.setenv("CHR_NF4_GEMV_STAGED", "1")
    monkeypatch.setenv("CHR_NF4_GEMV_TERMS", "3")
    g = torch.Generator(device=DEV).manual_seed(m + k)
    w = torch.randn((m, k), generator=g, device=DEV, dtype=torch.float32) * 0.02
    dp, ds = nf4.nf4_quantize(w)
    del w
    x = rand_x(k, None, 31)
    dx = bf16_tensor(x)
    monkeypatch.setenv("CHR_NF4_GEMV_RING", "1")
    runs = [nf4.nf4_gemv(dp, ds, dx, m, k, oc.k_pad(k)) for _ in range(5)]
    torch.cuda.synchronize()
    for r in runs[1:]:
        assert torch.equal(runs[0].view(torch.int16), r.view(torch.int16))
    monkeypatch.setenv("CHR_NF4_GEMV_RING", "0")
    y0 = nf4.nf4_gemv(dp, ds, dx, m, k, oc.k_pad(k))
    check_linear(runs[0], to_f32(y0), what=f"ring {m}x{k} vs pipelined", ulps=1)
    rows = torch.arange(0, m, 997, device=DEV)
    wd = nf4.nf4_dequant(dp, ds, m, k, oc.k_pad(k))[rows].double()
    want = (wd @ torch.from_numpy(x.astype(np.float64)).to(DEV)).cpu().numpy()
    got = to_f32(runs[0][rows]).reshape(-1)
    assert np.abs(got - want).max() <= 1e-2 * np.abs(want).max() + 0.05


# Form 3 stages x as binary16, every 16 consecutive elements times the power of two that puts
# the largest of them in [2^14, 2^15).  Every element within 2^-29 of that largest converts
# exactly; the cases below are the ones a fixed binary16 conversion would break (overflow above
# 65504, underflow of a vector that is tiny as a whole) and the ones the scaling itself could
# (all zero, one huge outlier among tiny elements, elements so far below their neighbours that
# they land on the subnormal grid, neighbouring groups of 16 of very different size).
def _x_cases(k):
    rng = np.random.default_rng(5)
    base = rng.standard_normal(k).astype(np.float32)
    spike = base * 1e-3
    spike[k // 3] = 3.0e6
    wide = base * np.exp2(rng.integers(-40, 10, k)).astype(np.float32)
    return {
        "large": base * 4.0e5,            # far above binary16's 65504
        "tiny": base * 1.0e-20,           # far below binary16's smallest subnormal
        "zero": np.zeros(k, np.float32),
        "spike": spike,                   # one element 2^30 above the rest
        "wide": wide,                     # fifty binades in one vector
        "bf16_max": np.where(np.arange(k) % 97 == 0, 1.0e38, base).astype(np.float32),  # near the end of the range
    }


@pytest.mark.parametrize("case", ["large", "tiny", "zero", "spike", "wide", "bf16_max"])
@pytest.mark.parametrize("m,k,ring", [(4100, 4096, "1"), (300, 16384, "1"), (200, 2048, "0"), (130, 200, "0")])
def test_binary16_staging_range(m, k, ring, case, monkeypatch):
    say("binary16 staging", m, k, ring, case)
    monkeypatch.setenv("CHR_NF4_GEMV_STAGED", "1")
    monkeypatch.setenv("CHR_NF4_GEMV_RING", ring)
    monkeypatch.setenv("CHR_NF4_GEMV_TERMS", "3")
    p, s, dp, ds = blobs(m, k, 900 + m)
    x = oc.bf16_round(_x_cases(k)[case])
    y = nf4.nf4_gemv(dp, ds, bf16_tensor(x), m, k, oc.k_pad(k))
    got = to_f32(y).astype(np.float64).reshape(-1)
    model = staged_gemv_model(p, s, m, k, x, terms=3).reshape(-1)
    if case == "zero":
        assert (got == 0).all()
        return
    assert np.isfinite(got).all()
    # relative to the output's own size (the absolute floors of check_linear mean nothing at
    # 1e-20 or 1e5): one bf16 step, plus 1e-3 of the rms for rows that cancel
    rms = np.sqrt((model ** 2).mean())
    assert rms > 0
    assert (np.abs(got - model) <= ulp_bf16(model) + 1e-3 * rms).all(), (
        case, float(np.max(np.abs(got - model) / (ulp_bf16(model) + 1e-3 * rms))))
    # and the fused norm on the same vector (the largest normalised value is bounded from the
    # two maxima, not searched for): against the same model on the normalised vector
    if case in ("large", "wide") and k % 64 == 0:
        g = oc.bf16_round((1 + 0.25 * np.random.default_rng(2).standard_normal(k)).astype(np.float32) * 37.0)
        eps = 1e-6
        y2 = nf4.nf4_gemv(dp, ds, bf16_tensor(x), m, k, oc.k_pad(k), rms_w=bf16_tensor(g), rms_eps=eps)
        x64 = x.astype(np.float64)
        inv = np.float32(1.0) / np.sqrt(np.float32((x64 ** 2).sum() / k + eps))
        xh = oc.bf16_round(((g * x).astype(np.float32) * np.float32(inv)).astype(np.float32))
        m2 = staged_gemv_model(p, s, m, k, xh, terms=3).reshape(-1)
        got2 = to_f32(y2).astype(np.float64).reshape(-1)
        rms2 = np.sqrt((m2 ** 2).mean())
        assert np.isfinite(got2).all() and rms2 > 0
        assert (np.abs(got2 - m2) <= 4 * ulp_bf16(m2) + 4e-3 * rms2).all(), case


@pytest.mark.parametrize("terms", [1, 2, 3])
@pytest.mark.parametrize("mq,mk,k,fused", [(5120, 1024, 5120, True), (4096, 512, 4096, False),
                                           (130, 33, 6144, True), (3000, 777, 7168, False)])
def test_ring_qkv(mq, mk, k, fused, terms, monkeypatch):
    """Three row segments through one ring launch (q/k/v), biases, with and without the folded
    RMSNorm, against the oracle and against three separate GEMVs."""
    say("ring qkv", mq, mk, k, fused, terms)
    monkeypatch.setenv("CHR_NF4_GEMV_STAGED", "1")
    monkeypatch.setenv("CHR_NF4_GEMV_RING", "1")
    monkeypatch.setenv("CHR_NF4_GEMV_TERMS", str(terms))
    mats = [blobs(mq, k, 181), blobs(mk, k, 182), blobs(mk, k, 183)]
    rng = np.random.default_rng(19)
    x = rand_x(k, None, 21)
    g = oc.bf16_round(1 + 0.1 * rng.standard_normal(k).astype(np.float32))
    biases = [oc.bf16_round(rng.standard_normal(m).astype(np.float32)) for m in (mq, mk, mk)]
    outs = [torch.empty(m, dtype=torch.bfloat16, device=DEV) for m in (mq, mk, mk)]
    dx = bf16_tensor(x)
    rms = (bf16_tensor(g), 1e-6) if fused else (None, 0.0)
    nf4.nf4_qkv(mats[0][2], mats[0][3], mats[1][2], mats[1][3], mats[2][2], mats[2][3], dx,
                mq, mk, mk, k, k, outs[0], outs[1], outs[2], *[bf16_tensor(b) for b in biases], *rms)
    xh = x
    if fused:
        h = torch.empty(k, dtype=torch.bfloat16, device=DEV)
        nf4.nf4_rms(dx, bf16_tensor(g), h, 1e-6)
        xh = to_f32(h).reshape(-1)
    for (p, s, dp, ds), m, b, o in zip(mats, (mq, mk, mk), biases, outs):
        ref = oc.c_matmul_f64(oc.c_decode(p, s, m, k), xh[:, None]).reshape(-1) + b
        model = staged_gemv_model(p, s, m, k, xh, terms=terms) + b
        check_linear(o, ref, what="ring qkv", model=model)
        single = torch.empty(m, dtype=torch.bfloat16, device=DEV)
        nf4.nf4_gemv(dp, ds, dx, m, k, k, single, bf16_tensor(b), *rms)
        check_linear(o, to_f32(single), what="ring qkv vs single", ulps=1)


@pytest.mark.parametrize("terms", [1, 2, 3])
@pytest.mark.parametrize("m,k", [(4100, 5120), (520, 4096), (2100, 6208)])
def test_ring_gemv_fused_rms(m, k, terms, monkeypatch):
    monkeypatch.setenv("CHR_NF4_GEMV_RING", "1")
    monkeypatch.setenv("CHR_NF4_GEMV_TERMS", str(terms))
    p, s, dp, ds = blobs(m, k, 53)
    rng = np.random.default_rng(8)
    x = oc.bf16_round(rng.standard_normal(k).astype(np.float32) * 3)
    g = oc.bf16_round(1 + 0.1 * rng.standard_normal(k).astype(np.float32))
    eps = 1e-6
    y = nf4.nf4_gemv(dp, ds, bf16_tensor(x), m, k, oc.k_pad(k), rms_w=bf16_tensor(g), rms_eps=eps)
    h = torch.empty(k, dtype=torch.bfloat16, device=DEV)
    nf4.nf4_rms(bf16_tensor(x), bf16_tensor(g), h, eps)
    xh = to_f32(h).reshape(-1)
    ref = oc.c_matmul_f64(oc.c_decode(p, s, m, k), xh[:, None])
    check_linear(y, ref, what="ring fused rms", ulps=4, model=staged_gemv_model(p, s, m, k, xh, terms=terms))
    monkeypatch.setenv("CHR_NF4_GEMV_STAGED", "1")
    y2 = nf4.nf4_gemv(dp, ds, h, m, k, oc.k_pad(k))
    check_linear(y, to_f32(y2), what="ring fused rms vs rms+gemv", ulps=1)


@pytest.mark.parametrize("terms", [1, 2, 3])
@pytest.mark.parametrize("m,k", [
    (4100, 4096), (4400, 5120), (20, 5120), (2300, 6144), (1100, 12288), (2100, 5056),
    (2200, 7168), (2100, 8192),    # rows of 7 half steps, and of 8 (two pieces of 4)
    (700, 13824),                  # two pieces of 7
    (2200, 11008),                 # 11 half steps: two pieces of 6, the last with an empty slot
    (2100, 4000),                  # K below K_pad
])
def test_ring_swiglu(m, k, terms, monkeypatch):
    """A gate row and the up row of the same index go through the ring one after the other."""
    say("ring swiglu", m, k, terms)
    monkeypatch.setenv("CHR_NF4_GEMV_STAGED", "1")
    monkeypatch.setenv("CHR_NF4_GEMV_RING", "1")
    monkeypatch.setenv("CHR_NF4_GEMV_TERMS", str(terms))
    kp = oc.k_pad(k)
    pg, sg, dpg, dsg = blobs(m, k, 93)
    pu, su, dpu, dsu = blobs(m, k, 94)
    x = rand_x(k, None, 14)
    out = torch.empty(m, dtype=torch.bfloat16, device=DEV)
    nf4.nf4_swiglu(dpg, dsg, dpu, dsu, bf16_tensor(x), m, k, kp, out)
    g = oc.c_matmul_f64(oc.c_decode(pg, sg, m, k), x[:, None]).reshape(-1)
    u = oc.c_matmul_f64(oc.c_decode(pu, su, m, k), x[:, None]).reshape(-1)
    gm = staged_gemv_model(pg, sg, m, k, x, terms=terms)
    model = gm / (1 + np.exp(-gm)) * staged_gemv_model(pu, su, m, k, x, terms=terms)
    # (levels rounded to bf16 put 2^-9 of every weight into a gate sum of 13824 terms that is then
    # multiplied by an up sum of the same size: past the absolute floor the reference keeps for
    # one linear; the kernel's own arithmetic, the tight bound, is held to all the same)
    check_linear(out, g / (1 + np.exp(-g)) * u, what="ring swiglu", ulps=1.5, model=model,
                 floor=not (terms == 1 and k > 12288))
    out2 = torch.empty(m, dtype=torch.bfloat16, device=DEV)
    nf4.nf4_swiglu(dpg, dsg, dpu, dsu, bf16_tensor(x), m, k, kp, out2)
    assert (bf16_bits(out) == bf16_bits(out2)).all()


# ------------------------------------ sum of squares handed from a vector's writer to its reader
def gpu_blobs(m, k, seed):
    """Quantised N(0, 0.02) weights made on the GPU (shapes too large for the toy blobs)."""
    g = torch.Generator(device=DEV)
    g.manual_seed(seed)
    w = torch.randn((m, k), generator=g, device=DEV, dtype=torch.float32) * 0.02
    return nf4.nf4_quantize(w)


def parts_of(y, grid):
    """What the writer leaves: workgroup b sums the squares of rows b, b + grid, ..."""
    sq = to_f32(y).reshape(-1).astype(np.float64) ** 2
    parts = np.zeros(nf4.dv2_sumsq_parts())
    for b in range(min(grid, sq.size)):
        parts[b] = sq[b::grid].sum()
    return parts


@pytest.mark.parametrize("terms", [1, 3])
@pytest.mark.parametrize("m,k,merges,ring", [
    (5120, 13824, False, "1"), (5120, 5120, True, "1"), (2100, 8192, False, "1"), (6144, 16384, False, "1"),
    (1040, 27648, False, "1"),
    (5120, 5120, True, "0"), (2100, 8192, False, "0"),   # the compiler-pipelined kernel
    (2048, 2048, True, "1"), (8200, 2048, False, "1"),   # rows of 2 half steps: no ring kernel takes them
    (4099, 5120, False, "1"), (4099, 5120, False, "0"),  # a last workgroup pass that is not full
    (300, 5120, True, "1"),                              # fewer workgroups than parts: zeros behind them
])
def test_gemv_leaves_the_sum_of_squares_of_what_it_stored(m, k, merges, ring, terms, monkeypatch):
    """``sumsq_out``: the same y, bit for bit, and in the parts buffer the squares of the stored
    bf16 values, workgroup by workgroup, zeros behind them (whatever the buffer held before)."""
    say("sumsq writer", m, k, merges, ring, terms)
    monkeypatch.setenv("CHR_NF4_GEMV_TERMS", str(terms))
    monkeypatch.setenv("CHR_NF4_GEMV_RING", ring)
    assert nf4.dv2_sumsq_ok(m, k, k, merges)
    dp, ds = gpu_blobs(m, k, 71)
    res = bf16_tensor(np.random.default_rng(3).standard_normal(m).astype(np.float32))
    n_parts = nf4.dv2_sumsq_parts()
    grid = min(torch.cuda.get_device_properties(0).multi_processor_count, -(-m // 16))
    for rep in range(2):
        parts = torch.full((n_parts,), float("nan"), dtype=torch.float32, device=DEV)
        y0 = torch.empty(m, dtype=torch.bfloat16, device=DEV)
        y1 = torch.empty(m, dtype=torch.bfloat16, device=DEV)
        if merges:
            n_q, hd = k // 128, 128
            st = torch.randn(nf4.dv2_attn_state_floats(n_q, hd), device=DEV).abs()
            nf4.dv2_gemv_attn(dp, ds, st, n_q, hd, m, k, k, y0, res)
            nf4.dv2_gemv_attn(dp, ds, st, n_q, hd, m, k, k, y1, res, sumsq_out=parts)
        else:
            x = bf16_tensor(rand_x(k, None, 5 + rep))
            nf4.nf4_gemv(dp, ds, x, m, k, k, y0, res)
            nf4.nf4_gemv(dp, ds, x, m, k, k, y1, res, sumsq_out=parts)
        assert (bf16_bits(y0) == bf16_bits(y1)).all()
        got = parts.cpu().numpy().astype(np.float64)
        want = parts_of(y1, grid)
        assert np.isfinite(got).all() and (got[grid:] == 0).all()
        assert np.abs(got - want).max() <= 1e-5 * want.max(), (rep, np.abs(got - want).max(), want.max())


def test_sumsq_hand_over_is_refused_where_no_kernel_serves_it(monkeypatch):
    """A launch of the plain kernel (too few codes for the kernels that stage x), a reader
    without a norm, a launch forced onto the plain kernel: error -8, nothing launched."""
    parts = torch.zeros(nf4.dv2_sumsq_parts(), dtype=torch.float32, device=DEV)
    for m, k in [(300, 7168), (4096, 2048)]:
        assert not nf4.dv2_sumsq_ok(m, k, k)
        dp, ds = gpu_blobs(m, k, 72)
        x = bf16_tensor(rand_x(k, None, 6))
        with pytest.raises(RuntimeError, match="-8"):
            nf4.nf4_gemv(dp, ds, x, m, k, k, sumsq_out=parts)
        with pytest.raises(RuntimeError, match="-8"):
            nf4.nf4_gemv(dp, ds, x, m, k, k, sumsq_in=parts)          # no rms_w
    m, k = 5120, 5120
    dp, ds = gpu_blobs(m, k, 73)
    x = bf16_tensor(rand_x(k, None, 7))
    assert nf4.dv2_sumsq_ok(m, k, k)
    monkeypatch.setenv("CHR_NF4_GEMV_STAGED", "0")
    assert not nf4.dv2_sumsq_ok(m, k, k)
    with pytest.raises(RuntimeError, match="-8"):
        nf4.nf4_gemv(dp, ds, x, m, k, k, sumsq_out=parts)
    with pytest.raises(RuntimeError):
        nf4.nf4_gemv(dp, ds, x, m, k, k, sumsq_in=parts[1:])            # not 16-byte aligned, too short


@pytest.mark.parametrize("ring", ["1", "0"])
@pytest.mark.parametrize("terms", [1, 3])
@pytest.mark.parametrize("k", [5120, 6144, 2048, 4000, 13824])
def test_norm_folded_into_a_gemv_takes_the_sum_of_squares_it_is_handed(k, terms, ring, monkeypatch):
    """``sumsq_in``: q/k/v, gate/up and a single matrix normalise x with the sum the parts hold
    instead of summing x: with the parts of x itself the result is the launch's own to the last
    bf16 step of a few elements (another order of the same additions); with four times those
    parts it is the result for x / 2: the parts are what is used."""
    say("sumsq reader", k, terms, ring)
    monkeypatch.setenv("CHR_NF4_GEMV_TERMS", str(terms))
    monkeypatch.setenv("CHR_NF4_GEMV_RING", ring)
    monkeypatch.setenv("CHR_NF4_GEMV_STAGED", "1")
    rng = np.random.default_rng(k)
    xh = oc.bf16_round(rng.standard_normal(k).astype(np.float32) * 3)
    x = bf16_tensor(xh)
    g = bf16_tensor(oc.bf16_round(1 + 0.1 * rng.standard_normal(k).astype(np.float32)))
    n_parts = nf4.dv2_sumsq_parts()
    sq = xh.astype(np.float64) ** 2
    own = np.zeros(n_parts)
    for b in range(n_parts):
        own[b] = sq[b::n_parts].sum()
    parts = torch.tensor(own, dtype=torch.float32, device=DEV)
    m = 4100
    dp, ds = gpu_blobs(m, k, 74)
    mq, mk = 2048, 512
    dq, sq_ = gpu_blobs(mq, k, 75)
    dk, sk = gpu_blobs(mk, k, 76)
    dv, sv = gpu_blobs(mk, k, 77)
    bias = [bf16_tensor(rng.standard_normal(n).astype(np.float32)) for n in (mq, mk, mk)]

    kp = oc.k_pad(k)

    def run(p):
        kw = {} if p is None else {"sumsq_in": p}
        y = nf4.nf4_gemv(dp, ds, x, m, k, kp, rms_w=g, **kw).reshape(-1).clone()
        o = [torch.empty(n, dtype=torch.bfloat16, device=DEV) for n in (mq, mk, mk)]
        nf4.nf4_qkv(dq, sq_, dk, sk, dv, sv, x, mq, mk, mk, k, kp, *o, *bias, rms_w=g, **kw)
        s = torch.empty(mq, dtype=torch.bfloat16, device=DEV)
        nf4.nf4_swiglu(dq, sq_, dp[:mq], ds[:mq], x, mq, k, kp, s, rms_w=g, **kw)
        return [y, *o, s]

    base, handed, scaled = run(None), run(parts), run(parts * 4)
    for a, b, c in zip(base, handed, scaled):
        fa, fb, fc = to_f32(a).reshape(-1), to_f32(b).reshape(-1), to_f32(c).reshape(-1)
        lim = 2.0 ** -7 * np.maximum(np.abs(fa), 2.0 ** -6 * np.abs(fa).max())
        assert (np.abs(fa - fb) <= lim).all(), np.abs(fa - fb).max()
        assert (bf16_bits(a) != bf16_bits(b)).mean() <= 0.02
        # x / 2 (no bias rows only: the single matrix and the SwiGLU's gate * up ~ 1/4 .. 1/2)
    y, y4 = to_f32(base[0]).reshape(-1), to_f32(scaled[0]).reshape(-1)
    assert np.abs(y4 - 0.5 * y).max() <= 2.0 ** -6 * np.abs(y).max()


def test_sum_of_squares_from_the_writer_to_the_reader(monkeypatch):
    """The hand-over as the decode step uses it, at the 14B shapes: the down projection (residual
    added) leaves the parts, gate/up of the next layer normalises with them; the prologue leaves
    them for the first q/k/v.  Against the reader summing for itself."""
    k5, ffn = 5120, 13824
    dd, sd = gpu_blobs(k5, ffn, 81)
    dg, sg = gpu_blobs(4096, k5, 82)
    du, su = gpu_blobs(4096, k5, 83)
    rng = np.random.default_rng(9)
    xin = bf16_tensor(rand_x(ffn, None, 10))
    res = bf16_tensor(rng.standard_normal(k5).astype(np.float32))
    g = bf16_tensor(oc.bf16_round(1 + 0.1 * rng.standard_normal(k5).astype(np.float32)))
    parts = torch.zeros(nf4.dv2_sumsq_parts(), dtype=torch.float32, device=DEV)
    h = torch.empty(k5, dtype=torch.bfloat16, device=DEV)
    nf4.nf4_gemv(dd, sd, xin, k5, ffn, ffn, h, res, sumsq_out=parts)
    assert abs(float(parts.double().sum()) - float((h.double() ** 2).sum())) <= 1e-5 * float((h.double() ** 2).sum())
    a = torch.empty(4096, dtype=torch.bfloat16, device=DEV)
    b = torch.empty(4096, dtype=torch.bfloat16, device=DEV)
    nf4.nf4_swiglu(dg, sg, du, su, h, 4096, k5, k5, a, rms_w=g)
    nf4.nf4_swiglu(dg, sg, du, su, h, 4096, k5, k5, b, rms_w=g, sumsq_in=parts)
    fa, fb = to_f32(a).reshape(-1), to_f32(b).reshape(-1)
    assert (np.abs(fa - fb) <= 2.0 ** -7 * np.maximum(np.abs(fa), 2.0 ** -6 * np.abs(fa).max())).all()
    # the prologue: the embedding row and its sum of squares
    emb_p, emb_s = gpu_blobs(1000, k5, 84)
    tok = torch.tensor(123, dtype=torch.int64, device=DEV)
    pos = torch.tensor(17, dtype=torch.int64, device=DEV)
    vl0 = torch.zeros((), dtype=torch.int32, device=DEV)
    vl1 = torch.zeros((), dtype=torch.int32, device=DEV)
    x0 = torch.empty(k5, dtype=torch.bfloat16, device=DEV)
    x1 = torch.empty(k5, dtype=torch.bfloat16, device=DEV)
    parts.fill_(float("nan"))
    nf4.dv2_begin_step(emb_p, emb_s, k5, tok, pos, vl0, x0)
    nf4.dv2_begin_step(emb_p, emb_s, k5, tok, pos, vl1, x1, sumsq_out=parts)
    assert torch.equal(x0, x1) and int(vl0) == int(vl1) == 18
    want = float((x1.double() ** 2).sum())
    assert abs(float(parts.double().sum()) - want) <= 1e-5 * want and float(parts[16:].abs().max()) == 0.0


# ------------------------------------------------------------------------ RMS
@pytest.mark.parametrize("n", [64, 2048, 5120, 6144, 100])
def test_rms(n):
    rng = np.random.default_rng(n)
    x = oc.bf16_round(rng.standard_normal(n).astype(np.float32) * 2)
    w = oc.bf16_round(1 + 0.2 * rng.standard_normal(n).astype(np.float32))
    y = torch.empty(n, dtype=torch.bfloat16, device=DEV)
    nf4.nf4_rms(bf16_tensor(x), bf16_tensor(w), y, 1e-6)
    ref = (w.astype(np.float64) * x) / np.sqrt((x.astype(np.float64) ** 2).mean() + 1e-6)
    check_linear(y, ref, what="rms", ulps=1)
    tref = F.rms_norm(torch.from_numpy(x), (n,), torch.from_numpy(w), 1e-6).numpy()
    check_linear(y, tref, what="rms vs torch", ulps=1)


# ----------------------------------------------------------------------- GEMM
def gemm_expected(p, s, m, k, x, plan):
    """What a prefill launch computes, in float64, by the tile its plan names.  The stream
    tile (the only one with 32- or 64-row blocks) multiplies bf16(level) and applies the fp16 scale
    to each 64-wide group's sum; the two older tiles multiply bf16(level * scale), the
    reference kernel's weights (gpu/nf4/nf4_gemm.cu:312-323)."""
    if plan["bm"] in (32, 64):
        return staged_gemv_model(p, s, m, k, x, terms=1)
    return oc.c_matmul_f64(oc.bf16_round(oc.c_decode(p, s, m, k)), x)


GEMM_SHAPES = [(128, 256), (130, 65), (64, 2048), (300, 5120), (129, 13824), (5120, 512)]


@pytest.mark.parametrize("m,k", GEMM_SHAPES)
@pytest.mark.parametrize("n", [2, 3, 8, 16, 17, 32])
def test_gemm_vs_oracle(m, k, n):
    say("gemm", m, k, n)
    p, s, dp, ds = blobs(m, k, 200 + m + k)
    x = rand_x(k, n, n)
    y = nf4.nf4_gemm(dp, ds, bf16_tensor(x), m, k, oc.k_pad(k))
    assert tuple(y.shape) == (m, n)
    w = oc.c_decode(p, s, m, k)
    # against the arithmetic of the tile that ran (each rounds a weight to bf16 once)
    ref_b = gemm_expected(p, s, m, k, x, nf4.nf4_plan(m, k, n))
    check_linear(y, ref_b, what=f"gemm {m}x{k} n{n} (bf16 weights)")
    # and stays inside the reference's floor-1 bound against unrounded weights
    ref = oc.c_matmul_f64(w, x)
    err = np.abs(to_f32(y).astype(np.float64) - ref)
    assert (err <= np.maximum(0.05, 2 ** (np.floor(np.log2(np.maximum(np.abs(ref), 1e-30))) - 8))).all()
    assert err.max() / np.abs(ref).max() <= 1e-2


@pytest.mark.parametrize("wide,narrow", [(16, 8), (32, 16), (7, 3)])
def test_gemm_column_subset_equals_padded(wide, narrow):
    """Columns do not mix: a chunk whose extra columns are zero gives the narrower chunk's
    bits (within one tile family: whole-vector widths run the stream tile, others not)."""
    m, k = 256, 1024
    p, s, dp, ds = blobs(m, k, 301)
    x = rand_x(k, wide, 13)
    xz = x.copy()
    xz[:, narrow:] = 0
    y_wide = nf4.nf4_gemm(dp, ds, bf16_tensor(xz), m, k, k)
    y_narrow = nf4.nf4_gemm(dp, ds, bf16_tensor(np.ascontiguousarray(x[:, :narrow])), m, k, k)
    assert (bf16_bits(y_narrow) == bf16_bits(y_wide[:, :narrow].contiguous())).all()
    assert (to_f32(y_wide[:, narrow:]) == 0).all()


@pytest.mark.parametrize("n", [8, 32, 5])
def test_gemm_every_split_agrees(n):
    """Forced splits (the two split-K tiles; the stream tile has no split): each against the
    arithmetic of the tile its plan names, and against each other within two bf16 steps
    (summation order only)."""
    m, k = 512, 4096
    p, s, dp, ds = blobs(m, k, 302)
    xh = rand_x(k, n, 14)
    x = bf16_tensor(xh)
    outs = []
    try:
        for split in (1, 2, 3, 5, 16):
            nf4.nf4_set_tuning(split_k=split)
            plan = nf4.nf4_plan(m, k, n)
            assert plan["bm"] == 128 and (plan["grid_y"] == min(split, 16) or split == 5)
            y = nf4.nf4_gemm(dp, ds, x, m, k, k)
            check_linear(y, gemm_expected(p, s, m, k, xh, plan), what=f"split {split} n{n}")
            outs.append(to_f32(y))
    finally:
        nf4.nf4_set_tuning()
    for o in outs[1:]:
        d = np.abs(o - outs[0])
        assert (d <= 2.0 ** (np.floor(np.log2(np.maximum(np.abs(outs[0]), 2.0 ** -120))) - 7) + 1e-30).all()


STREAM_CASES = [
    # m, k, n
    (32, 256, 8), (130, 512, 16), (200, 768, 24),   # a ragged last block; a last chunk of 256
    (1, 512, 8), (33, 256, 32),                      # one row; one row past a block
    (96, 1000, 32),                                  # K below K_pad
    (256, 5120, 32), (70, 6144, 8),                  # ten and twelve chunks
    (2048, 2048, 32), (5120, 5120, 8), (7168, 5120, 16),
    (8192, 1024, 32),                                # as many workgroups as compute units
    # 64 rows a workgroup: more 32-row blocks than compute units
    (8224, 256, 8), (8193, 512, 32), (9000, 1000, 24), (13824, 5120, 16),
    (32768, 4096, 8),                                # two workgroups for every compute unit
    # K split over workgroups that meet in the tile: 5 to 8, 3 and 2 splits
    (256, 5120, 32), (1024, 5120, 8), (5120, 13824, 8), (5120, 5120, 32), (3072, 8192, 16),
    (5000, 13560, 16),                               # ragged rows, K below K_pad, a last chunk of 256
    # more rounds of workgroups than one: four unsplit, two of six splits each
    (55296, 3072, 8), (5120, 27648, 24),
    # 64 columns: 64 rows a workgroup, chunks of 256
    (64, 256, 64), (100, 2304, 64), (130, 1000, 64),  # one chunk; ragged rows; K below K_pad
    (200, 5120, 64), (70, 10240, 64),                 # twenty chunks; splits of twenty
    (5120, 5120, 64), (7168, 5120, 64), (13824, 5120, 64), (5120, 13824, 64),
]


@pytest.mark.parametrize("m,k,n", STREAM_CASES)
def test_gemm_stream_tile(m, k, n):
    """The tile without a reduce launch (32 or 64 rows per workgroup and all of K, or K split
    over workgroups of which the last to finish adds up the partials in split order; bf16(level)
    times the activations, the scale applied to each group's sum): against that arithmetic in
    float64, bit-identical on a second launch, and its fused epilogue against the separate
    adds."""
    say("gemm stream", m, k, n)
    p, s, dp, ds = blobs(m, k, 900 + m + k + n)
    xh = rand_x(k, n, 19)
    x = bf16_tensor(xh)
    kp = oc.k_pad(k)
    nf4.nf4_gemm_stream_policy(1)  # wherever it fits: the planner leaves small launches to the split tiles
    try:
        _stream_tile_case(m, k, n, p, s, dp, ds, xh, x, kp)
    finally:
        nf4.nf4_gemm_stream_policy(0)


def _stream_tile_case(m, k, n, p, s, dp, ds, xh, x, kp):
    plan = nf4.nf4_plan(m, k, n)
    want = pyplan.plan(m, k, n, one_wave=256, stream_policy=1)
    assert all(plan[key] == getattr(want, key) for key in plan), (plan, want)
    bm, split = plan["bm"], plan["grid_y"]
    assert bm in (32, 64) and plan["block"] == 1024 and plan["grid_x"] == -(-m // bm)
    assert plan["ws_floats"] == (split * m * n if split > 1 else 0)
    assert plan["ctas"] <= 4 * 256
    if n == 64:
        assert bm == 64 and -(-kp // 256) <= split * 20
        assert plan["smem_bytes"] == 32768 + 2 * 64 * 264 * 2 + 2 * 64 * 144 + 80 * 64 * 2
    else:
        assert -(-kp // 512) <= split * 12
        assert plan["smem_bytes"] == 32768 + 2 * 33280 + 2 * bm * 272 + 96 * bm * 2
    y = nf4.nf4_gemm(dp, ds, x, m, k, kp, 64)
    check_linear(y, staged_gemv_model(p, s, m, k, xh, terms=1), what=f"stream {m}x{k} n{n}")
    ref = oc.c_matmul_f64(oc.c_decode(p, s, m, k), xh)
    err = np.abs(to_f32(y).astype(np.float64) - ref)
    assert (err <= np.maximum(0.05, 2 ** (np.floor(np.log2(np.maximum(np.abs(ref), 1e-30))) - 8))).all()
    assert (bf16_bits(nf4.nf4_gemm(dp, ds, x, m, k, kp, 64)) == bf16_bits(y)).all()
    rng = np.random.default_rng(m + n)
    bias = bf16_tensor(oc.bf16_round(rng.standard_normal(m).astype(np.float32)))
    res = bf16_tensor(oc.bf16_round(rng.standard_normal((m, n)).astype(np.float32)))
    want = res + (y + bias[:, None])
    got = nf4.nf4_gemm(dp, ds, x, m, k, kp, 64, bias=bias, residual=res)
    assert (bf16_bits(got) == bf16_bits(want)).all()


def test_gemm_stream_tile_random_shapes():
    """Sixty seeded random launches of the tile that finishes its rows itself, taken wherever it
    fits (rows 1..12000, K_pad 256..9984 with K at or below it, every chunk width it has):
    each against its arithmetic in float64 and bit-identical on a second launch."""
    rng = np.random.default_rng(2024)
    nf4.nf4_gemm_stream_policy(1)
    try:
        forms, done = set(), 0
        while done < 60:
            n = int(rng.choice([8, 16, 24, 32, 64]))
            kp = int(rng.integers(1, 40)) * 256
            k = kp - int(rng.integers(0, 64)) if rng.random() < 0.5 else kp
            m = int(rng.integers(1, 3000)) if rng.random() < 0.7 else int(rng.integers(3000, 12000))
            if m * kp > 40_000_000:
                continue
            plan = nf4.nf4_plan(m, k, n)
            if plan["block"] != 1024 or plan["bm"] not in (32, 64):
                continue
            say("gemm stream, random", m, k, n, plan["bm"], plan["grid_x"], plan["grid_y"])
            p, s = oc.toy_blobs(m, k, int(rng.integers(1 << 30)))
            dp, ds = up(p), up_scale(s)
            xh = rand_x(k, n, int(rng.integers(1000)))
            x = bf16_tensor(xh)
            y = nf4.nf4_gemm(dp, ds, x, m, k, oc.k_pad(k), 64)
            assert (bf16_bits(nf4.nf4_gemm(dp, ds, x, m, k, oc.k_pad(k), 64)) == bf16_bits(y)).all()
            check_linear(y, staged_gemv_model(p, s, m, k, xh, terms=1), what=f"stream {m}x{k} n{n}")
            forms.add((plan["bm"], plan["grid_y"] > 1, n == 64))
            done += 1
        assert len(forms) >= 5, forms  # 32 and 64 rows, split and not, the 64-column form
    finally:
        nf4.nf4_gemm_stream_policy(0)


def test_gemm_stream_splits_on_many_streams():
    """Launches whose workgroups share K count their arrivals in a row of a table the library
    owns, one row per stream (owners beyond its 512 rows get the reduce kernel on the same
    partials).  Forty streams, each launching twice: every result equals the first bit for bit."""
    m, k, n = 5120, 13824, 8
    say("gemm stream, many streams", m, k, n)
    assert nf4.nf4_plan(m, k, n)["grid_y"] == 3 and nf4.nf4_plan(m, k, n)["block"] == 1024
    p, s, dp, ds = blobs(m, k, 77)
    x = bf16_tensor(rand_x(k, n, 5))
    first = bf16_bits(nf4.nf4_gemm(dp, ds, x, m, k, k))
    torch.cuda.synchronize()
    outs = []
    for _ in range(40):
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            outs.append(nf4.nf4_gemm(dp, ds, x, m, k, k))
            outs.append(nf4.nf4_gemm(dp, ds, x, m, k, k))
    torch.cuda.synchronize()
    for o in outs:
        assert (bf16_bits(o) == first).all()


def test_gemm_stream_splits_in_a_replayed_graph():
    """Three launches with K shared by workgroups, captured in one graph: every replay, with
    eager launches of the same tile between the replays, gives the eager results bit for bit
    (the arrival counts must be back at zero after every launch)."""
    shapes = [(5120, 13824, 8), (5120, 13824, 32), (3072, 8192, 16)]
    mats, xs, eager = [], [], []
    for i, (m, k, n) in enumerate(shapes):
        say("gemm stream, graph", m, k, n)
        assert nf4.nf4_plan(m, k, n)["grid_y"] > 1 and nf4.nf4_plan(m, k, n)["block"] == 1024
        p, s, dp, ds = blobs(m, k, 31 + i)
        mats.append((dp, ds))
        xs.append(bf16_tensor(rand_x(k, n, 40 + i)))
        eager.append(bf16_bits(nf4.nf4_gemm(dp, ds, xs[i], m, k, k)))
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = [nf4.nf4_gemm(mats[i][0], mats[i][1], xs[i], m, k, k) for i, (m, k, n) in enumerate(shapes)]
    for _ in range(4):
        for o in outs:
            o.zero_()
        graph.replay()
        torch.cuda.synchronize()
        for o, want in zip(outs, eager):
            assert (bf16_bits(o) == want).all()
        m, k, n = shapes[0]
        assert (bf16_bits(nf4.nf4_gemm(mats[0][0], mats[0][1], xs[0], m, k, k)) == eager[0]).all()


def test_gemm_stream_graph_replayed_beside_eager_launches():
    """A split launch recorded during capture owns a row of arrival counts of its own, so the
    graph can be replayed on a second stream while eager split launches of the same shape run
    on the stream it was captured from: all results equal those of the same launches made one
    at a time, bit for bit, on every one of several overlapping rounds."""
    m, k, n = 5120, 13824, 8
    say("gemm stream, graph beside eager", m, k, n)
    assert nf4.nf4_plan(m, k, n)["grid_y"] == 3 and nf4.nf4_plan(m, k, n)["block"] == 1024
    p, s, dp, ds = blobs(m, k, 78)
    p2, s2, dp2, ds2 = blobs(m, k, 79)
    xa, xb = bf16_tensor(rand_x(k, n, 6)), bf16_tensor(rand_x(k, n, 7))
    # the same launches one at a time on an idle device (their sums are the reduce kernel's, in
    # split order whoever arrives last: test_gemm_add_sq compares the two bit for bit)
    want_a = bf16_bits(nf4.nf4_gemm(dp, ds, xa, m, k, k))
    torch.cuda.synchronize()
    want_b = bf16_bits(nf4.nf4_gemm(dp2, ds2, xb, m, k, k))
    torch.cuda.synchronize()
    cap = torch.cuda.Stream()
    other = torch.cuda.Stream()
    with torch.cuda.stream(cap):
        nf4.nf4_gemm(dp, ds, xa, m, k, k)  # eager launches on the capture stream own its row
        cap.synchronize()
        graph = torch.cuda.CUDAGraph()
        graph.capture_begin()
        held = [nf4.nf4_gemm(dp, ds, xa, m, k, k) for _ in range(6)]
        graph.capture_end()
    torch.cuda.synchronize()
    for _ in range(5):
        eager = []
        with torch.cuda.stream(other):
            graph.replay()
        with torch.cuda.stream(cap):
            for _ in range(6):
                eager.append(nf4.nf4_gemm(dp2, ds2, xb, m, k, k))
        torch.cuda.synchronize()
        for o in held:
            assert (bf16_bits(o) == want_a).all()
            o.zero_()
        for o in eager:
            assert (bf16_bits(o) == want_b).all()


@pytest.mark.parametrize("n", [5, 8, 16, 24, 32, 40, 64])
@pytest.mark.parametrize("k,split,tiles", [(1024, 1, 4), (1000, 2, 2), (1024, 4, 1), (768, 1, 3),
                                           (2048, 1, 8), (2048, 8, 1)])
def test_gemm_every_tile_variant(n, k, split, tiles):
    """The two split-K tiles under forced splits: slice lengths of one to four K tiles (the
    row-streaming tile, one build per length and per 16-column block count; two tiles at most
    above 32 columns) and an eight-tile slice (the K-tiled kernel), with whole-vector and
    ragged column counts and a ragged row block."""
    m = 200
    say("gemm variant", m, k, n, split)
    p, s, dp, ds = blobs(m, k, 310 + k)
    x = rand_x(k, n, 17)
    try:
        nf4.nf4_set_tuning(split_k=split)
        plan = nf4.nf4_plan(m, k, n)
        assert (plan["grid_y"], plan["tiles_per_split"]) == (split, tiles)
        streams_rows = tiles <= (2 if n > 32 else 4)
        assert plan["bm"] == 128 and plan["block"] == (512 if streams_rows else 256)
        y = nf4.nf4_gemm(dp, ds, bf16_tensor(x), m, k, oc.k_pad(k), max_n=64)
    finally:
        nf4.nf4_set_tuning()
    check_linear(y, gemm_expected(p, s, m, k, x, plan), what=f"gemm {m}x{k} n{n} split {split}")


def test_gemm_n1_routes_to_gemv():
    m, k = 384, 2048
    p, s, dp, ds = blobs(m, k, 303)
    x = bf16_tensor(rand_x(k, None, 15))
    y = nf4.nf4_gemm(dp, ds, x, m, k, k)
    assert tuple(y.shape) == (m, 1)
    assert (bf16_bits(y) == bf16_bits(nf4.nf4_gemv(dp, ds, x, m, k, k))).all()


PREFILL_14B = [("qkv", 7168, 5120), ("o", 5120, 5120), ("gate_up", 13824, 5120), ("down", 5120, 13824)]


@pytest.mark.parametrize("name,m,k", PREFILL_14B, ids=[s[0] for s in PREFILL_14B])
def test_gemm_full_14b_shapes(name, m, k):
    """Every 14B linear shape at N = 8, 16, 32 through ``nf4_gemm`` at full size, all rows
    against the oracle's weights rounded the way the launch's tile rounds them, and against
    the unrounded oracle product within the reference's bounds."""
    w, p, s, dp, ds = quantized(m, k, 21 + m % 97)
    exact_w = oc.c_decode(p, s, m, k)
    for n in (8, 16, 32):
        say("gemm 14B shape", name, m, k, n)
        x = rand_x(k, n, 16 + n)
        y = nf4.nf4_gemm(dp, ds, bf16_tensor(x), m, k, k)
        plan = nf4.nf4_plan(m, k, n)
        # every one of them on the tile whose workgroups finish their rows themselves: 32 rows
        # and all of K (q/k/v, o), 64 rows (gate, up), 64 rows and K over three workgroups (down)
        form = {"qkv": (32, 1), "o": (32, 1), "gate_up": (64, 1), "down": (64, 3)}
        assert (plan["bm"], plan["grid_y"]) == form[name], name
        assert plan["block"] == 1024
        ref = oc.c_matmul_f64(exact_w, x)
        err = np.abs(to_f32(y).astype(np.float64) - ref)
        assert (err <= np.maximum(0.05, 2 ** (np.floor(np.log2(np.maximum(np.abs(ref), 1e-30))) - 8))).all()
        assert err.max() / np.abs(ref).max() <= 1e-2
        check_linear(y, gemm_expected(p, s, m, k, x, plan), what=f"prefill {name} n{n} (tile)")


# ------------------------------------------------------------------ attention
def rope_tables(max_seq, hd, theta=10000.0):
    inv = 1.0 / (np.float32(theta) ** (np.arange(0, hd, 2, dtype=np.float32) / np.float32(hd)))
    fr = np.outer(np.arange(max_seq, dtype=np.float32), inv.astype(np.float32)).astype(np.float32)
    emb = np.concatenate([fr, fr], axis=-1)
    return oc.bf16_round(np.cos(emb).astype(np.float32)), oc.bf16_round(np.sin(emb).astype(np.float32))


def rot_half(t, cos, sin):
    d = t.shape[-1] // 2
    rot = np.concatenate([-t[..., d:], t[..., :d]], axis=-1)
    return t * cos + rot * sin


def attn_ref(q, kc, vc, valid, scale, n_rep):
    """q [n_q,hd] float64; kc/vc [T,n_kv,hd]; softmax over t < valid."""
    n_q, hd = q.shape
    out = np.zeros((n_q, hd))
    for h in range(n_q):
        kv = h // n_rep
        sc = (kc[:valid, kv] @ q[h]) * scale
        w = np.exp(sc - sc.max())
        w /= w.sum()
        out[h] = w @ vc[:valid, kv]
    return out


#: Attention output against a float64 softmax: the kernel accumulates in fp32 and rounds once
#: to bf16, so an element is within one bf16 step of the exact value (half a step from the
#: rounding, the rest from fp32 sums and the fast exponential: measured 0.48 at worst), plus a
#: floor for elements that cancel to almost nothing.
ATTN_ULPS = 1.0
ATTN_FLOOR = 2e-4


def check_attn(got: np.ndarray, ref: np.ndarray, what: str) -> None:
    err = np.abs(got.astype(np.float64) - ref.astype(np.float64))
    bound = ATTN_ULPS * ulp_bf16(ref.astype(np.float64)) + ATTN_FLOOR
    worst = float((err / bound).max())
    say(f"  {what}: worst error {worst:.3f} of the bound, max abs {err.max():.2e}")
    assert worst <= 1.0, (what, worst)


@pytest.mark.parametrize("n_q,n_kv,hd,max_seq,valid", [
    (4, 2, 16, 16, 5), (8, 2, 64, 32, 32), (16, 2, 128, 256, 200), (40, 8, 128, 2048, 2048),
    (4, 4, 32, 64, 1), (6, 3, 256, 40, 33), (4, 2, 48, 64, 50), (16, 2, 128, 300, 37)])
def test_attn_plain(n_q, n_kv, hd, max_seq, valid):
    say("attn", n_q, n_kv, hd, max_seq, valid)
    rng = np.random.default_rng(hd + valid)
    q = oc.bf16_round(rng.standard_normal((n_q, hd)).astype(np.float32))
    kc = oc.bf16_round(rng.standard_normal((max_seq, n_kv, hd)).astype(np.float32))
    vc = oc.bf16_round(rng.standard_normal((max_seq, n_kv, hd)).astype(np.float32))
    kc[valid:] = 1e4  # a dirty tail must be ignored
    vc[valid:] = -1e4
    out = torch.zeros(n_q * hd, dtype=torch.bfloat16, device=DEV)
    vl = torch.tensor(valid, dtype=torch.int32, device=DEV)
    scale = hd ** -0.5
    nf4.nf4_attn(bf16_tensor(q), bf16_tensor(kc), bf16_tensor(vc), out, vl, scale)
    ref = attn_ref(q.astype(np.float64), kc.astype(np.float64), vc.astype(np.float64), valid, scale,
                   n_q // n_kv)
    got = to_f32(out).reshape(n_q, hd)
    check_attn(got, ref, "attn vs f64")
    # library cross-check: torch SDPA in float32
    tq = torch.from_numpy(q).reshape(1, n_kv, n_q // n_kv, hd)
    tk = torch.from_numpy(kc[:valid]).permute(1, 0, 2).unsqueeze(0)
    tv = torch.from_numpy(vc[:valid]).permute(1, 0, 2).unsqueeze(0)
    sd = F.scaled_dot_product_attention(tq, tk, tv, scale=scale).reshape(n_q, hd).numpy()
    check_attn(got, sd, "attn vs SDPA")


@pytest.mark.parametrize("n_q,n_kv,hd,max_seq,pos", [(4, 2, 16, 16, 0), (4, 2, 16, 16, 7),
                                                     (16, 2, 128, 128, 100), (40, 8, 128, 2048, 1500),
                                                     (4, 2, 48, 32, 9)])
def test_attn_fused_rope_and_cache_write(n_q, n_kv, hd, max_seq, pos):
    say("attn fused", n_q, n_kv, hd, max_seq, pos)
    rng = np.random.default_rng(pos + hd)
    cos, sin = rope_tables(max_seq, hd)
    q = oc.bf16_round(rng.standard_normal((n_q, hd)).astype(np.float32))
    ka = oc.bf16_round(rng.standard_normal((n_kv, hd)).astype(np.float32))
    va = oc.bf16_round(rng.standard_normal((n_kv, hd)).astype(np.float32))
    kc = oc.bf16_round(rng.standard_normal((max_seq, n_kv, hd)).astype(np.float32))
    vc = oc.bf16_round(rng.standard_normal((max_seq, n_kv, hd)).astype(np.float32))
    dk, dv = bf16_tensor(kc), bf16_tensor(vc)
    out = torch.zeros(n_q * hd, dtype=torch.bfloat16, device=DEV)
    vl = torch.tensor(pos + 1, dtype=torch.int32, device=DEV)
    position = torch.tensor(pos, dtype=torch.int64, device=DEV)
    scale = hd ** -0.5
    nf4.nf4_attn(bf16_tensor(q), dk, dv, out, vl, scale, None, nf4.ATTN_SPLIT, bf16_tensor(ka),
                 bf16_tensor(va), bf16_tensor(cos), bf16_tensor(sin), position)
    qr = rot_half(q.astype(np.float64), cos[pos], sin[pos])
    kr = rot_half(ka.astype(np.float64), cos[pos], sin[pos])
    # cache row pos now holds bf16(k_rot) and v; every other row is untouched
    kc2 = to_f32(dk)
    vc2 = to_f32(dv)
    assert (oc.bf16_round_bits(kr.astype(np.float32)) == bf16_bits(dk[pos])).mean() > 0.99
    assert np.abs(kc2[pos] - kr).max() <= 2 ** -6
    assert (vc2[pos] == va).all()
    mask = np.ones(max_seq, bool)
    mask[pos] = False
    assert (kc2[mask] == kc[mask]).all() and (vc2[mask] == vc[mask]).all()
    # attention uses the unrounded rotated key for the current slot
    kfull = kc.astype(np.float64).copy()
    vfull = vc.astype(np.float64).copy()
    kfull[pos], vfull[pos] = kr, va
    ref = attn_ref(qr, kfull, vfull, pos + 1, scale, n_q // n_kv)
    # q is rotated in fp32 and not rounded again, so the same bound holds with the fusion
    check_attn(to_f32(out).reshape(n_q, hd), ref, "fused attn vs f64")


def test_attn_empty_prefix_gives_zero():
    n_q, n_kv, hd, max_seq = 4, 2, 64, 16
    out = torch.ones(n_q * hd, dtype=torch.bfloat16, device=DEV)
    z = torch.zeros((max_seq, n_kv, hd), dtype=torch.bfloat16, device=DEV)
    nf4.nf4_attn(torch.ones((n_q, hd), dtype=torch.bfloat16, device=DEV), z, z, out,
                 torch.tensor(0, dtype=torch.int32, device=DEV), 0.125)
    assert (to_f32(out) == 0).all()


@pytest.mark.parametrize("n_q,n_kv,hd,pos", [(4, 2, 16, 3), (16, 2, 128, 60), (6, 3, 256, 0)])
def test_rope_kv(n_q, n_kv, hd, pos):
    max_seq = 64
    rng = np.random.default_rng(hd)
    cos, sin = rope_tables(max_seq, hd)
    q = oc.bf16_round(rng.standard_normal((n_q, hd)).astype(np.float32))
    k = oc.bf16_round(rng.standard_normal((n_kv, hd)).astype(np.float32))
    v = oc.bf16_round(rng.standard_normal((n_kv, hd)).astype(np.float32))
    dq, dk, dv = bf16_tensor(q), bf16_tensor(k), bf16_tensor(v)
    kc = torch.zeros((max_seq, n_kv, hd), dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros_like(kc)
    nf4.nf4_rope_kv(dq, dk, dv, kc, vc, bf16_tensor(cos), bf16_tensor(sin),
                    torch.tensor(pos, dtype=torch.int64, device=DEV))
    qr = rot_half(q.astype(np.float64), cos[pos], sin[pos])
    kr = rot_half(k.astype(np.float64), cos[pos], sin[pos])
    assert np.abs(to_f32(dq) - qr).max() <= 2 ** -6
    assert np.abs(to_f32(dk) - kr).max() <= 2 ** -6
    assert (bf16_bits(kc[pos]) == bf16_bits(dk)).all()
    assert (to_f32(vc[pos]) == v).all()
    assert (to_f32(kc[:pos]) == 0).all() and (to_f32(kc[pos + 1:]) == 0).all()


# ---- fused decode-step launches ----------------------------------------------------

@pytest.mark.parametrize("n_q,n_kv,hd,max_seq,pos", [(4, 2, 16, 16, 0), (16, 2, 128, 128, 100),
                                                     (40, 8, 128, 2048, 1500), (4, 2, 48, 32, 9),
                                                     (40, 8, 128, 2048, 2047),
                                                     # 264 query heads on one KV head: past the
                                                     # range of the kernel's reciprocal index
                                                     # arithmetic, the integer division runs
                                                     (264, 1, 16, 64, 20)])
def test_dv2_attn_equals_the_two_launch_form(n_q, n_kv, hd, max_seq, pos):
    """One workgroup per head against split kernel + merge: the same online softmax over
    another partition of the rows, so the outputs agree to bf16 rounding; the cache row
    written is bit-identical."""
    say("dv2_attn", n_q, n_kv, hd, max_seq, pos)
    rng = np.random.default_rng(hd + pos)
    cos, sin = rope_tables(max_seq, hd)
    q = bf16_tensor(rng.standard_normal((n_q, hd)).astype(np.float32))
    k_act = bf16_tensor(rng.standard_normal((n_kv, hd)).astype(np.float32))
    v_act = bf16_tensor(rng.standard_normal((n_kv, hd)).astype(np.float32))
    kc0 = bf16_tensor(rng.standard_normal((max_seq, n_kv, hd)).astype(np.float32))
    vc0 = bf16_tensor(rng.standard_normal((max_seq, n_kv, hd)).astype(np.float32))
    tcos, tsin = bf16_tensor(cos), bf16_tensor(sin)
    vl = torch.tensor(pos + 1, dtype=torch.int32, device=DEV)
    position = torch.tensor(pos, dtype=torch.int64, device=DEV)
    scale = hd ** -0.5
    kc_a, vc_a = kc0.clone(), vc0.clone()
    out_a = torch.zeros(n_q * hd, dtype=torch.bfloat16, device=DEV)
    nf4.nf4_attn(q, kc_a, vc_a, out_a, vl, scale, None, nf4.ATTN_SPLIT, k_act, v_act, tcos, tsin,
                 position)
    for waves in (16, 5, 1):
        kc_b, vc_b = kc0.clone(), vc0.clone()
        out_b = torch.full((n_q * hd,), 3.0, dtype=torch.bfloat16, device=DEV)
        nf4.dv2_attn(q, kc_b, vc_b, out_b, vl, scale, waves, k_act, v_act, tcos, tsin, position)
        # two orders of merging the same fp32 partial states: one bf16 step apart at most
        check_attn(to_f32(out_b), to_f32(out_a), f"one launch ({waves} wavefronts) vs two")
        assert (bf16_bits(kc_a) == bf16_bits(kc_b)).all() and (bf16_bits(vc_a) == bf16_bits(vc_b)).all()
    # without RoPE / cache-write fusion, against the float64 reference
    out_d = torch.zeros(n_q * hd, dtype=torch.bfloat16, device=DEV)
    nf4.dv2_attn(q, kc_a, vc_a, out_d, vl, scale)
    ref = attn_ref(to_f32(q).astype(np.float64), to_f32(kc_a).astype(np.float64),
                   to_f32(vc_a).astype(np.float64), pos + 1, scale, n_q // n_kv)
    check_attn(to_f32(out_d).reshape(n_q, hd), ref, "one-launch attn vs f64")
    with pytest.raises(RuntimeError):
        nf4.dv2_attn(q, kc_a, vc_a, out_d, vl, scale, 17)


def test_dv2_attn_empty_prefix_gives_zero():
    q = bf16_tensor(np.ones((4, 16), dtype=np.float32))
    kc = bf16_tensor(np.ones((8, 2, 16), dtype=np.float32))
    out = torch.full((64,), 5.0, dtype=torch.bfloat16, device=DEV)
    nf4.dv2_attn(q, kc, kc, out, torch.tensor(0, dtype=torch.int32, device=DEV), 0.25)
    assert float(out.float().abs().max()) == 0.0


@pytest.mark.parametrize("vocab,k", [(1000, 256), (50, 5120), (7, 100), (300, 8256)])
def test_begin_step(vocab, k):
    say("begin_step", vocab, k)
    w = (np.random.default_rng(k).standard_normal((vocab, k)) * 0.5).astype(np.float32)
    dp, ds = nf4.nf4_quantize(torch.from_numpy(w).to(DEV))
    g = bf16_tensor(oc.bf16_round(1 + 0.1 * np.random.default_rng(1).standard_normal(k).astype(np.float32)))
    eps = 1e-5
    for tok, pos in ((0, 0), (vocab - 1, 41), (vocab // 2, 7)):
        token = torch.tensor(tok, dtype=torch.int64, device=DEV)
        position = torch.tensor(pos, dtype=torch.int64, device=DEV)
        valid = torch.zeros((), dtype=torch.int32, device=DEV)
        x = torch.zeros(k, dtype=torch.bfloat16, device=DEV)
        h = torch.zeros(k, dtype=torch.bfloat16, device=DEV)
        nf4.dv2_begin_step(dp, ds, k, token, position, valid, x, g, eps, h)
        assert int(valid.item()) == pos + 1
        x2 = torch.zeros(k, dtype=torch.bfloat16, device=DEV)
        valid2 = torch.zeros((), dtype=torch.int32, device=DEV)
        nf4.dv2_begin_step(dp, ds, k, token, position, valid2, x2)       # gather only
        assert (bf16_bits(x2) == bf16_bits(x)).all() and int(valid2.item()) == pos + 1
        row = nf4.nf4_embed_rows(dp, ds, token.reshape(1), k).reshape(-1)
        assert (bf16_bits(x) == bf16_bits(row)).all()
        h2 = torch.empty(k, dtype=torch.bfloat16, device=DEV)
        nf4.nf4_rms(row, g, h2, eps)
        a, b = to_f32(h).astype(np.float64), to_f32(h2).astype(np.float64)
        assert (np.abs(a - b) <= ulp_bf16(b)).all()
        xv = to_f32(row).astype(np.float64)
        ref = to_f32(g).astype(np.float64) * xv / np.sqrt((xv ** 2).mean() + eps)
        assert (np.abs(a - ref) <= ulp_bf16(ref)).all()


@pytest.mark.parametrize("n_q,n_kv,hd,max_seq,pos,parts,waves", [
    (4, 2, 16, 16, 0, 8, 4), (16, 2, 128, 128, 100, 8, 4), (40, 8, 128, 2048, 1500, 8, 4),
    (4, 2, 48, 32, 9, 3, 2), (40, 8, 128, 2048, 2047, 5, 16), (8, 8, 64, 64, 33, 1, 1),
    # what the decode step launches (4 parts of 8 wavefronts: heads placed by die, a block of rows
    # read ahead), at a context of one block, of two, and of the whole cache
    (40, 8, 128, 2048, 300, 4, 8), (40, 8, 128, 2048, 700, 4, 8), (40, 8, 128, 2048, 2047, 4, 8)])
def test_attention_merged_by_the_o_projection(n_q, n_kv, hd, max_seq, pos, parts, waves):
    """dv2_attn_parts + dv2_gemv_attn against nf4_attn + nf4_gemv(add) (each checked against
    float64 above): the same softmax over another partition of the rows, merged inside the
    GEMV's staging."""
    say("attn parts", n_q, n_kv, hd, max_seq, pos, parts, waves)
    rng = np.random.default_rng(hd + pos + parts)
    cos, sin = rope_tables(max_seq, hd)
    q = bf16_tensor(rng.standard_normal((n_q, hd)).astype(np.float32))
    k_act = bf16_tensor(rng.standard_normal((n_kv, hd)).astype(np.float32))
    v_act = bf16_tensor(rng.standard_normal((n_kv, hd)).astype(np.float32))
    kc0 = bf16_tensor(rng.standard_normal((max_seq, n_kv, hd)).astype(np.float32))
    vc0 = bf16_tensor(rng.standard_normal((max_seq, n_kv, hd)).astype(np.float32))
    kc0[pos + 1:] = 1e4      # a dirty tail must be ignored
    vc0[pos + 1:] = -1e4
    tcos, tsin = bf16_tensor(cos), bf16_tensor(sin)
    vl = torch.tensor(pos + 1, dtype=torch.int32, device=DEV)
    position = torch.tensor(pos, dtype=torch.int64, device=DEV)
    scale = hd ** -0.5
    hidden = n_q * hd
    m = 192
    p, s, dp, ds = blobs(m, hidden, 91)
    res = bf16_tensor(rng.standard_normal(m).astype(np.float32))
    # reference sequence
    kc_a, vc_a = kc0.clone(), vc0.clone()
    attn = torch.zeros(hidden, dtype=torch.bfloat16, device=DEV)
    nf4.nf4_attn(q, kc_a, vc_a, attn, vl, scale, None, nf4.ATTN_SPLIT, k_act, v_act, tcos, tsin, position)
    want = res.clone()
    nf4.nf4_gemv(dp, ds, attn, m, hidden, hidden, want, want)
    # two launches
    state = torch.full((nf4.dv2_attn_state_floats(n_q, hd, parts),), float("nan"), dtype=torch.float32,
                       device=DEV)
    for rep in range(2):
        kc_b, vc_b = kc0.clone(), vc0.clone()
        nf4.dv2_attn_parts(q, kc_b, vc_b, vl, scale, state, parts, waves, k_act, v_act, tcos, tsin, position)
        got = res.clone()
        nf4.dv2_gemv_attn(dp, ds, state, n_q, hd, m, hidden, hidden, got, got, parts)
        assert (bf16_bits(kc_a) == bf16_bits(kc_b)).all() and (bf16_bits(vc_a) == bf16_bits(vc_b)).all()
        assert torch.isfinite(got.float()).all()
        # the merged activations differ from the two-launch ones by bf16 rounding at most
        err = np.abs(to_f32(got) - to_f32(want)).max()
        assert err <= 0.02 * max(1.0, float(np.abs(to_f32(want)).max())), (rep, err)


def test_gemv_attn_rejects_bad_arguments():
    p, s, dp, ds = blobs(64, 128, 5)
    state = torch.zeros(nf4.dv2_attn_state_floats(2, 64, 4), dtype=torch.float32, device=DEV)
    y = torch.zeros(64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError):
        nf4.dv2_gemv_attn(dp, ds, state, 3, 64, 64, 128, 128, y, None, 4)      # K != n_q*hd
    with pytest.raises(RuntimeError):
        nf4.dv2_gemv_attn(dp, ds, state[:10], 2, 64, 64, 128, 128, y, None, 4)  # state too small
    nf4.dv2_gemv_attn(dp, ds, state, 2, 64, 64, 128, 128, y, None, 4)           # zero states -> zeros
    assert float(y.float().abs().max()) == 0.0


# ---- argmax + commit ----------------------------------------------------------------------

@pytest.mark.parametrize("n", [5, 1000, 16384, 50001, 152064])
@pytest.mark.parametrize("two_launch", [False, True])
def test_argmax_commit(n, two_launch):
    say("argmax", n, two_launch)
    rng = np.random.default_rng(n)
    ws = torch.zeros(nf4.dv2_argmax_ws_bytes() // 8, dtype=torch.int64, device=DEV) if two_launch else None

    def run(logits, commit=False, eos=7):
        nt = torch.full((), -1, dtype=torch.int64, device=DEV)
        tok = torch.full((), -1, dtype=torch.int64, device=DEV)
        pos = torch.full((), 10, dtype=torch.int64, device=DEV)
        fin = torch.zeros((), dtype=torch.uint8, device=DEV)
        nf4.dv2_argmax_commit(logits, nt, tok, pos, fin, torch.tensor(eos, dtype=torch.int64, device=DEV),
                              commit=commit, ws=ws)
        return int(nt.item()), int(tok.item()), int(pos.item()), int(fin.item())

    vals = oc.bf16_round(rng.standard_normal(n).astype(np.float32))
    assert run(bf16_tensor(vals))[0] == int(np.argmax(vals))        # numpy: first maximum
    # ties: the lowest index wins, wherever the equal values sit
    for where in ([0, n - 1], [n // 2, n // 2 + 1], [n - 1]):
        t = vals.copy()
        t[where] = 9.0
        assert run(bf16_tensor(t))[0] == min(where)
    flat = np.zeros(n, dtype=np.float32)
    assert run(bf16_tensor(flat))[0] == 0
    t = vals.copy()
    t[n // 3] = np.nan                                               # a NaN logit is surfaced
    t[n - 1] = np.inf
    assert run(bf16_tensor(t))[0] == n // 3
    # commit feeds the pick back and flags eos
    t = vals.copy()
    t[min(7, n - 1)] = 50.0
    pick = min(7, n - 1)
    assert run(bf16_tensor(t), commit=True, eos=pick) == (pick, pick, 11, 1)
    assert run(bf16_tensor(t), commit=True, eos=pick + 1) == (pick, pick, 11, 0)
    assert run(bf16_tensor(t), commit=False) == (pick, -1, 10, 0)
