"""The CPU oracle against the reference's own golden vectors.

Every expected value here is data the reference's tests hold
(``internal/nf4/nf4_test.go``, ``internal/f16/f16_test.go``,
``docs/spec/nf4.md`` sections 1, 2.3, 5, 6, 8, 9) or something mathematics fixes
(IEEE conversions brute-forced against numpy/torch, midpoints of the level
grid).  Both restatements (C and numpy) must pass each check.
"""

from __future__ import annotations

import json
import os

import numpy as np
import pytest

from oracle import nf4_oracle as oc

# tests/golden/nf4_golden.json holds the vectors, each with the reference line it comes from
_G = {k: v["value"] for k, v in json.load(open(os.path.join(os.path.dirname(__file__), "golden",
                                                             "nf4_golden.json"))).items()
      if isinstance(v, dict)}
GOLDEN64_HEX = _G["golden64_hex"]
GOLDEN2X64_ROW1_HEX = _G["golden2x64_row1_hex"]
PAD01_HEX = _G["pad01_hex"]
GOLDEN64_IDX = _G["golden64_idx"]
LEVEL_LITERALS = _G["level_literals"]
MIDPOINT_BITS = [int(b, 16) for b in _G["midpoint_bits"]]

ENCODERS = [pytest.param(oc.c_encode, id="c"), pytest.param(oc.np_encode, id="numpy")]
DECODERS = [pytest.param(oc.c_decode, id="c"), pytest.param(oc.np_decode, id="numpy")]


def row_i_over_63():
    return (np.arange(64, dtype=np.float32) / np.float32(63)).reshape(1, 64)


def fixture_2x64():
    i = np.arange(64, dtype=np.float32)
    return np.stack([i / np.float32(63), (np.float32(2) * i - np.float32(63)) / np.float32(63)]).astype(np.float32)


def hexs(a):
    return np.ascontiguousarray(a).tobytes().hex().upper()


def bits16(scale):
    return np.asarray(scale).view(np.uint16)


def test_lut_bits():
    lut = np.zeros(16, dtype=np.float32)
    oc.lib().or_nf4_lut(lut.ctypes.data)
    assert [int(b) for b in lut.view(np.uint32)] == list(oc.LUT_BITS)
    assert [int(b) for b in np.array(LEVEL_LITERALS, dtype=np.float32).view(np.uint32)] == list(oc.LUT_BITS)
    assert int(oc.LUT.view(np.uint32)[7]) == 0  # plus zero, not minus zero
    assert all(oc.LUT[i] < oc.LUT[i + 1] for i in range(15))


@pytest.mark.parametrize("enc", ENCODERS)
def test_golden64(enc):
    data, scale = enc(row_i_over_63())
    assert hexs(data) == GOLDEN64_HEX
    assert bits16(scale).tolist() == [[0x3C00]]
    assert oc.np_unpack(data)[0].tolist() == GOLDEN64_IDX


@pytest.mark.parametrize("enc", ENCODERS)
@pytest.mark.parametrize("dec", DECODERS)
def test_golden_2x64_and_metrics(enc, dec):
    w = fixture_2x64()
    data, scale = enc(w)
    assert data.size == 64
    assert hexs(data[0]) == GOLDEN64_HEX
    assert hexs(data[1]) == GOLDEN2X64_ROW1_HEX
    assert bits16(scale).reshape(-1).tolist() == [0x3C00, 0x3C00]
    err = (dec(data, scale, 2, 64) - w).astype(np.float64)
    assert np.sqrt((err ** 2).mean()) <= 0.05185
    assert np.abs(err).max() <= 0.14508
    assert np.abs(err).mean() <= 0.03980


@pytest.mark.parametrize("enc", ENCODERS)
def test_nibble_order(enc):
    assert enc(np.array([[0, 1]], dtype=np.float32))[0][0, 0] == 0xF7
    assert enc(np.array([[1, 0]], dtype=np.float32))[0][0, 0] == 0x7F
    w = np.zeros((1, 64), dtype=np.float32)
    w[0, 0], w[0, 1], w[0, 2] = oc.LUT[3], oc.LUT[12], 1
    data, scale = enc(w)
    assert bits16(scale)[0, 0] == 0x3C00
    assert data[0, 0] == 0xC3


@pytest.mark.parametrize("enc", ENCODERS)
@pytest.mark.parametrize("dec", DECODERS)
@pytest.mark.parametrize("shape", [(3, 64), (1, 65)])
def test_zero_matrix(enc, dec, shape):
    w = np.zeros(shape, dtype=np.float32)
    data, scale = enc(w)
    assert data.shape == (shape[0], oc.k_pad(shape[1]) // 2)
    assert (data == 0x77).all()
    assert (bits16(scale) == 0x3C00).all()
    hat = dec(data, scale, *shape)
    assert hat.shape == shape
    assert (hat.view(np.uint32) == 0).all()  # +0 bits


@pytest.mark.parametrize("enc", ENCODERS)
@pytest.mark.parametrize("dec", DECODERS)
@pytest.mark.parametrize("value,scale_bits,byte", [(-2.25, 0x4080, 0x00), (0.5, 0x3800, 0xFF)])
def test_constant_rows(enc, dec, value, scale_bits, byte):
    w = np.full((1, 64), value, dtype=np.float32)
    data, scale = enc(w)
    assert bits16(scale)[0, 0] == scale_bits
    assert (data == byte).all()
    assert (dec(data, scale, 1, 64) == np.float32(value)).all()


@pytest.mark.parametrize("enc", ENCODERS)
@pytest.mark.parametrize("dec", DECODERS)
@pytest.mark.parametrize("make", [row_i_over_63, fixture_2x64])
def test_idempotent(enc, dec, make):
    w = make()
    m, k = w.shape
    d1, s1 = enc(w)
    hat = dec(d1, s1, m, k)
    d2, s2 = enc(hat)
    assert (d1 == d2).all() and (bits16(s1) == bits16(s2)).all()
    assert (dec(d2, s2, m, k).view(np.uint32) == hat.view(np.uint32)).all()


@pytest.mark.parametrize("enc", ENCODERS)
@pytest.mark.parametrize("dec", DECODERS)
def test_pad_to_64(enc, dec):
    data, scale = enc(np.array([[0, 1]], dtype=np.float32))
    assert hexs(data) == PAD01_HEX
    assert bits16(scale).tolist() == [[0x3C00]]
    hat = dec(data, scale, 1, 2)
    assert hat.shape == (1, 2) and hat[0, 0] == 0 and hat[0, 1] == 1


@pytest.mark.parametrize("enc", ENCODERS)
def test_tiny_group_is_a_zero_group(enc):
    data, scale = enc(np.full((1, 64), 1e-12, dtype=np.float32))
    assert bits16(scale)[0, 0] == 0x3C00  # scale flushed to zero in binary16 -> scale 1
    assert (data == 0x77).all()


@pytest.mark.parametrize("enc", ENCODERS)
def test_huge_group_clamps_to_f16_max(enc):
    data, scale = enc(np.full((1, 64), 1e6, dtype=np.float32))
    assert bits16(scale)[0, 0] == 0x7BFF  # 65504
    assert (data == 0xFF).all()


@pytest.mark.parametrize("enc", ENCODERS)
@pytest.mark.parametrize("bad", [np.nan, np.inf, -np.inf])
def test_reject_non_finite(enc, bad):
    w = row_i_over_63()
    w[0, 3] = bad
    with pytest.raises(ValueError):
        enc(w)


@pytest.mark.parametrize("enc", ENCODERS)
def test_reject_empty(enc):
    with pytest.raises(ValueError):
        enc(np.zeros((0, 64), dtype=np.float32))
    with pytest.raises(ValueError):
        enc(np.zeros((1, 0), dtype=np.float32))
    with pytest.raises(ValueError):
        oc.c_decode(np.zeros(0, np.uint8), np.zeros(0, np.float16), 0, 64)
    with pytest.raises(ValueError):
        oc.c_decode(np.zeros(0, np.uint8), np.zeros(0, np.float16), 1, 0)


@pytest.mark.parametrize("enc", ENCODERS)
@pytest.mark.parametrize("dec", DECODERS)
def test_decode_exact_and_stable(enc, dec):
    data, scale = enc(row_i_over_63())
    hat = dec(data, scale, 1, 64)
    want = oc.LUT[np.array(GOLDEN64_IDX)]
    assert (hat.view(np.uint32)[0] == want.view(np.uint32)).all()
    assert (dec(data, scale, 1, 64).view(np.uint32) == hat.view(np.uint32)).all()


def test_scale_is_little_endian_binary16():
    _, scale = oc.c_encode(row_i_over_63())
    assert scale.tobytes() == b"\x00\x3c"


# ---- IEEE conversions: closed forms brute-forced against numpy / torch ----------
def test_f16_to_f32_all_patterns():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = oc.f16_bits_to_f32(bits)
    nan = np.isnan(want)
    assert (got.view(np.uint32)[~nan] == want.view(np.uint32)[~nan]).all()
    assert np.isnan(got[nan]).all()


def test_f32_to_f16_round_trip_and_rne():
    L = oc.lib()
    for v, b in [(0.0, 0), (1.0, 0x3C00), (-1.0, 0xBC00), (0.5, 0x3800), (2.0, 0x4000),
                 (2.25, 0x4080), (2.5, 0x4100), (65504.0, 0x7BFF)]:
        assert L.or_f32_to_f16(v) == b
        assert L.or_f16_to_f32(b) == v
    assert L.or_f32_to_f16(float("inf")) == 0x7C00
    n = L.or_f32_to_f16(float("nan"))
    assert n & 0x7C00 == 0x7C00 and n & 0x3FF != 0
    h = L.or_f32_to_f16(1e-5)  # a binary16 subnormal
    assert h & 0x7C00 == 0 and 0 < L.or_f16_to_f32(h) <= 2e-5
    # Every binary16 value, and the float32 values just beside the halfway
    # points between neighbours, against numpy's IEEE conversion.
    rng = np.random.default_rng(7)
    vals = np.concatenate([
        np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32),
        rng.standard_normal(200000).astype(np.float32) * np.float32(3),
        (rng.standard_normal(50000) * 1e-6).astype(np.float32),
        (rng.standard_normal(50000) * 4e4).astype(np.float32),
    ])
    vals = vals[np.isfinite(vals)]
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = oc.f32_to_f16_bits(vals)
    assert (got == want).all()
    # exact ties between consecutive binary16 values go to even
    h16 = np.arange(0x0001, 0x7BFF, 37, dtype=np.uint16)
    lo = h16.view(np.float16).astype(np.float64)
    hi = (h16 + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    mid = ((lo + hi) / 2).astype(np.float32)  # exact: one extra bit
    got = oc.f32_to_f16_bits(mid)
    want = np.where(h16 % 2 == 0, h16, h16 + 1)
    assert (got == want).all()


def test_bf16_round_against_torch():
    import torch

    rng = np.random.default_rng(3)
    vals = np.concatenate([
        rng.standard_normal(300000).astype(np.float32),
        (rng.standard_normal(100000) * 1e-30).astype(np.float32),
        (rng.standard_normal(100000) * 1e30).astype(np.float32),
        np.array([0.0, -0.0, 1.0, np.inf, -np.inf, 3.3895314e38], dtype=np.float32),
    ])
    want = torch.from_numpy(vals).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert (oc.bf16_round_bits(vals) == want).all()
    L = oc.lib()
    for v, w in zip(vals[::997], want[::997]):
        assert L.or_f32_to_bf16(float(v)) == int(w)
    assert L.or_bf16_to_f32(0x3F80) == 1.0
    # exact ties: bf16 value + half an ulp rounds to the even neighbour
    b = np.arange(0x3F80, 0x4080, dtype=np.uint32)
    tie = ((b << 16) | 0x8000).astype(np.uint32).view(np.float32)
    got = oc.bf16_round_bits(tie)
    assert (got == np.where(b % 2 == 0, b, b + 1)).all()
    assert np.isnan(oc.bf16_bits_to_f32(oc.bf16_round_bits(np.array([np.nan], np.float32)))).all()


# ---- nearest level: the squared-distance search against the midpoint rule -------
@pytest.mark.parametrize("enc", ENCODERS)
def test_nearest_level_matches_midpoints(enc):
    mids = np.array(MIDPOINT_BITS, dtype=np.uint32).view(np.float32)
    # the published midpoints are float32((L[j] + L[j+1]) / 2)
    calc = ((oc.LUT[:-1].astype(np.float64) + oc.LUT[1:].astype(np.float64)) / 2).astype(np.float32)
    assert (calc.view(np.uint32) == mids.view(np.uint32)).all()
    # Dense sweep of [-1, 1] plus every float32 within 64 ulp of each midpoint.
    sweep = np.linspace(-1, 1, 64 * 4096 - 1, dtype=np.float64).astype(np.float32)
    near = (np.array(MIDPOINT_BITS, dtype=np.int64)[:, None] + np.arange(-64, 65)[None, :])
    near = near.astype(np.uint32).view(np.float32).reshape(-1)
    u = np.concatenate([sweep, near])
    u = u[: (u.size // 64) * 64]
    w = u.reshape(-1, 64).copy()
    w[:, 0] = 1.0  # pins every group's scale to exactly 1 so u is the weight itself
    data, scale = enc(w)
    assert (bits16(scale) == 0x3C00).all()
    got = oc.np_unpack(data).reshape(-1)
    flat = w.reshape(-1).astype(np.float64)
    # In exact arithmetic the nearest level is the count of midpoints below u,
    # ties to the lower index.  float32 (u-L)^2 can only disagree within a few
    # ulp of a midpoint, and then by one level.
    exact_mid = (oc.LUT[:-1].astype(np.float64) + oc.LUT[1:].astype(np.float64)) / 2
    want = np.searchsorted(exact_mid, flat, side="left")
    differ = got != want
    dist = np.abs(flat[:, None] - exact_mid[None, :]).min(axis=1)
    assert (np.abs(got.astype(int) - want)[differ] == 1).all()
    assert (dist[differ] <= 4 * np.spacing(np.abs(flat[differ]).astype(np.float32))).all()
    assert differ.mean() < 1e-3


def test_c_and_numpy_restatements_agree_on_random_matrices():
    rng = np.random.default_rng(11)
    for m, k, sigma in [(7, 64, 0.02), (5, 130, 0.05), (33, 65, 1.0), (16, 512, 0.02), (3, 1, 2.0)]:
        w = (rng.standard_normal((m, k)) * sigma).astype(np.float32)
        dc, sc = oc.c_encode(w)
        dn, sn = oc.np_encode(w)
        assert (dc == dn).all() and (bits16(sc) == bits16(sn)).all()
        hc = oc.c_decode(dc, sc, m, k)
        hn = oc.np_decode(dc, sc, m, k)
        assert (hc.view(np.uint32) == hn.view(np.uint32)).all()
        # round-trip error is bounded by half the widest level gap times the scale
        assert np.abs(hc - w).max() <= 0.16 * np.abs(w).max() * 1.001


def test_matmul_and_linear():
    rng = np.random.default_rng(5)
    w = rng.standard_normal((9, 70)).astype(np.float32)
    x = rng.standard_normal((70, 3)).astype(np.float32)
    y = oc.c_matmul_f32(w, x)
    y64 = oc.c_matmul_f64(w, x)
    assert np.allclose(y64, w.astype(np.float64) @ x.astype(np.float64), rtol=0, atol=1e-12)
    assert np.abs(y - y64).max() < 1e-4
    d, s = oc.c_encode(w)
    assert (oc.c_linear(d, s, 9, 70, x) == oc.c_matmul_f32(oc.c_decode(d, s, 9, 70), x)).all()
    # a matrix of level 7 (zero) gives y == 0 whatever the scales are
    zp, zs = oc.toy_blobs(4, 128, 1)
    zp[:] = 0x77
    assert (oc.c_linear(zp, zs, 4, 128, rng.standard_normal((128, 2)).astype(np.float32)) == 0).all()
