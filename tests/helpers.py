"""Helpers shared by the GPU parity tests: uploads, bf16 views, error bounds."""

from __future__ import annotations

import os

import numpy as np
import torch

from deepfold_amd.nf4 import plan as pyplan
from oracle import nf4_oracle as oc

DEV = "cuda"

#: Floor-1 bound of the reference's kernel checks at rms(x) ~ 1
#: (gpu/nf4/verify.py:70, gpu/nf4/numerics.py:191-202).
MAXABS_FLOOR = 0.05
#: max |y - y_ref| / max |y_ref| bound for bf16 outputs with fp32 accumulation.
MAX_REL = 1e-2


def up(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def up_scale(scale: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(scale).view(np.float16)).to(DEV)


def bf16_tensor(a: np.ndarray) -> torch.Tensor:
    """float32 array -> bf16 tensor on the GPU (rounded on the host, by torch)."""
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16).to(DEV)


def to_f32(t: torch.Tensor) -> np.ndarray:
    return t.detach().float().cpu().numpy()


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def rand_x(k: int, n: int | None, seed: int) -> np.ndarray:
    """N(0,1) activations already rounded to bf16 (as float32), so input rounding
    is not charged to the kernel (gpu/tests/oracle_gate.py:113-124)."""
    rng = np.random.default_rng(seed)
    shape = (k,) if n is None else (k, n)
    return oc.bf16_round(rng.standard_normal(shape).astype(np.float32))


def ulp_bf16(v: np.ndarray) -> np.ndarray:
    a = np.abs(np.asarray(v, dtype=np.float64))
    e = np.floor(np.log2(np.maximum(a, 2.0 ** -126)))
    return 2.0 ** (e - 7)


def takes_staged_gemv(m: int, k: int, *, fused: bool = False) -> bool:
    """Whether a GEMV launch of m rows takes the staged kernel (x in LDS: fused RMSNorm,
    ragged K, attention merge, and every matrix from 16M codes up).  That kernel multiplies
    levels rounded to binary16 (or kept as two bf16 terms, or rounded to bf16:
    ``staged_levels``); the reference's tensor-core path rounds the whole dequantised weight to
    bf16 (gpu/nf4/nf4_gemm.cu:322)."""
    return fused or pyplan.gemv_is_staged(m, k)


#: form of the levels the library takes when CHR_NF4_GEMV_TERMS is not set
DEFAULT_TERMS = 3


def env_terms() -> int:
    return {"1": 1, "2": 2, "3": 3, "f16": 3}.get(os.environ.get("CHR_NF4_GEMV_TERMS", ""), DEFAULT_TERMS)


def staged_levels(terms: int | None = None) -> np.ndarray:
    """The 16 levels as the staged GEMV multiplies them, in float64: rounded to binary16
    (form 3, the default; x is staged as binary16, every 16 consecutive elements times a power
    of two of their own, which is exact for every element within 2^-29 of the largest of its
    16, so the model leaves x alone), head = bf16(level) plus
    tail = bf16(level - head) (form 2), or the head alone (form 1)."""
    if terms is None:
        terms = env_terms()
    lut32 = oc.LUT.astype(np.float32)
    if terms == 3:
        return lut32.astype(np.float16).astype(np.float64)
    head = oc.bf16_round(lut32)
    if terms == 1:
        return head.astype(np.float64)
    tail = oc.bf16_round((lut32 - head).astype(np.float32))
    return head.astype(np.float64) + tail.astype(np.float64)


def staged_gemv_model(packed: np.ndarray, scale: np.ndarray, m: int, k: int,
                      x: np.ndarray, terms: int | None = None) -> np.ndarray:
    """The staged GEMV's arithmetic in float64: levels as ``staged_levels`` gives them,
    products exact, the fp16 scale applied to each group's sum.  x is [k] or [k, n]."""
    kp = oc.k_pad(k)
    g = kp // oc.GROUP
    packed = np.asarray(packed).reshape(m, kp // 2)
    sc = np.ascontiguousarray(scale).view(np.float16).reshape(m, g).astype(np.float64)
    lut = staged_levels(terms)
    xs = np.zeros((kp,) + tuple(np.shape(x)[1:]), dtype=np.float64)
    xs[:k] = np.asarray(x, dtype=np.float64)
    xg = xs.reshape((g, oc.GROUP) + xs.shape[1:])
    out = np.empty((m,) + xs.shape[1:], dtype=np.float64)
    for r0 in range(0, m, 512):  # row blocks keep the float64 level array small
        r1 = min(m, r0 + 512)
        lv = lut[oc.np_unpack(packed[r0:r1])].reshape(r1 - r0, g, oc.GROUP)
        part = np.einsum("mgk,gk...->mg...", lv, xg)
        out[r0:r1] = np.einsum("mg...,mg->m...", part, sc[r0:r1])
    return out


def check_linear(y: torch.Tensor, y_ref: np.ndarray, *, what: str = "", ulps: float = 1.0,
                 model: np.ndarray | None = None, floor: bool = True) -> dict:
    """y (bf16 on GPU) against a float32/float64 oracle result of the same shape.

    Three bounds: the reference's floor-1 bound max(0.05, ULP/2); max-rel 1e-2;
    and a tighter one of this build: within ``ulps`` bf16 ULP of the expected value
    (plus 1e-3 of the output's rms for cancellation-heavy rows).  The expected value of
    the tight bound is ``model`` when given (the kernel's own arithmetic written out on
    the CPU, e.g. ``staged_gemv_model``), else the oracle value."""
    got = to_f32(y).reshape(-1).astype(np.float64)
    ref = np.asarray(y_ref, dtype=np.float64).reshape(-1)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    err = np.abs(got - ref)
    u = ulp_bf16(ref)
    rms = float(np.sqrt((ref ** 2).mean())) if ref.size else 0.0
    if floor:  # (a bound for one linear at rms(x) ~ 1; not for a product of two long ones)
        assert (err <= np.maximum(MAXABS_FLOOR, 0.5 * u) + 1e-12).all(), f"{what}: maxabs {err.max():.6f}"
    denom = np.abs(ref).max()
    if denom > 0:
        assert err.max() / denom <= MAX_REL, f"{what}: max-rel {err.max() / denom:.3e}"
    tight = ref if model is None else np.asarray(model, dtype=np.float64).reshape(-1)
    assert tight.shape == ref.shape, (tight.shape, ref.shape)
    terr = np.abs(got - tight)
    tu = ulp_bf16(tight)
    assert (terr <= ulps * tu + 1e-3 * rms + 1e-30).all(), (
        f"{what}: worst {np.max(terr / (tu + 1e-30)):.2f} bf16 ULP")
    return {"maxabs": float(err.max()), "rms": rms}
