"""CPU oracle for group-64 NF4: ctypes face of ``nf4_oracle.c`` plus a numpy twin.

TEST INFRASTRUCTURE ONLY.  The shipped package never imports this module; it is
for ``tests/``, the smoke check and the bench's ``cpu_baseline`` leg.

Two independent restatements live here so that each pins the other:

* ``c_*``  functions call the C restatement of the reference's Go codec
  (``internal/nf4/nf4.go:46-121``, ``internal/f16/f16.go:8-106``).
* ``np_*`` functions restate the reference's numpy oracle
  (``gpu/tests/nf4_oracle.py:100-180``) with vectorised numpy.

Both are checked against the reference's golden vectors in
``tests/test_oracle_golden.py``.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

GROUP = 64

#: binary32 bit patterns of the sixteen levels (``internal/nf4/nf4_test.go:12-29``).
LUT_BITS = (
    0xBF800000, 0xBF3239B1, 0xBF066B30, 0xBECA32A0, 0xBE91A24D, 0xBE3D353F,
    0xBDBA7871, 0x00000000, 0x3DA2FAFF, 0x3E24CAE3, 0x3E7C04DD, 0x3EAD033A,
    0x3EE1A4B8, 0x3F1007AB, 0x3F3913B3, 0x3F800000,
)
LUT = np.array(LUT_BITS, dtype=np.uint32).view(np.float32)

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libnf4_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile ``nf4_oracle.c`` with the Makefile beside it."""
    if force or not os.path.exists(_SO) or (
        os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "nf4_oracle.c"))
    ):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libnf4_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        c = ctypes
        L.or_f16_to_f32.restype = c.c_float
        L.or_f16_to_f32.argtypes = [c.c_uint16]
        L.or_f32_to_f16.restype = c.c_uint16
        L.or_f32_to_f16.argtypes = [c.c_float]
        L.or_bf16_to_f32.restype = c.c_float
        L.or_bf16_to_f32.argtypes = [c.c_uint16]
        L.or_f32_to_bf16.restype = c.c_uint16
        L.or_f32_to_bf16.argtypes = [c.c_float]
        L.or_nf4_lut.argtypes = [c.c_void_p]
        L.or_nf4_encode.restype = c.c_int
        L.or_nf4_encode.argtypes = [c.c_void_p, c.c_int, c.c_int, c.c_void_p, c.c_void_p]
        L.or_nf4_decode.restype = c.c_int
        L.or_nf4_decode.argtypes = [c.c_void_p, c.c_void_p, c.c_int, c.c_int, c.c_void_p]
        L.or_matmul_f32.argtypes = [c.c_void_p, c.c_void_p, c.c_int, c.c_int, c.c_int, c.c_void_p]
        L.or_matmul_f64.argtypes = [c.c_void_p, c.c_void_p, c.c_int, c.c_int, c.c_int, c.c_void_p]
        L.or_linear_two_pass.restype = c.c_int
        L.or_linear_two_pass.argtypes = [c.c_void_p, c.c_void_p, c.c_int, c.c_int, c.c_void_p,
                                         c.c_int, c.c_void_p, c.c_void_p]
        L.or_gemv_fused.argtypes = [c.c_void_p, c.c_void_p, c.c_int, c.c_int, c.c_void_p, c.c_void_p]
        L.or_set_threads.argtypes = [c.c_int]
        L.or_max_threads.restype = c.c_int
        _lib = L
    return _lib


def k_pad(k: int) -> int:
    if k < 1:
        raise ValueError(f"K must be >= 1, got {k}")
    return GROUP * ((int(k) + GROUP - 1) // GROUP)


def _ptr(a: np.ndarray) -> int:
    return a.ctypes.data


# ----------------------------------------------------------------------------
# C restatement
# ----------------------------------------------------------------------------
class EncodeError(ValueError):
    pass


_ENC_ERR = {-1: "empty shape", -2: "non-finite weight", -3: "scale is not finite positive"}


def c_encode(w: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """float32 ``[M, K]`` -> (packed uint8 ``[M, K_pad/2]``, scale float16 ``[M, K_pad/64]``)."""
    if w.ndim != 2:
        raise EncodeError("encode wants a 2-D matrix")
    m, k = w.shape
    if m < 1 or k < 1:
        raise EncodeError(_ENC_ERR[-1])
    w = np.ascontiguousarray(w, dtype=np.float32)
    kp = k_pad(k)
    packed = np.zeros((m, kp // 2), dtype=np.uint8)
    scale = np.zeros((m, kp // GROUP), dtype=np.uint16)
    rc = lib().or_nf4_encode(_ptr(w), m, k, _ptr(packed), _ptr(scale))
    if rc != 0:
        raise EncodeError(_ENC_ERR.get(rc, f"rc={rc}"))
    return packed, scale.view(np.float16)


def c_decode(packed: np.ndarray, scale: np.ndarray, m: int, k: int) -> np.ndarray:
    """Packed blobs -> float32 ``[M, K]`` (padding dropped)."""
    if m < 1 or k < 1:
        raise ValueError("empty shape")
    kp = k_pad(k)
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    scale = np.ascontiguousarray(scale).view(np.uint16)
    if packed.size != m * kp // 2:
        raise ValueError(f"len(data)={packed.size} want {m * kp // 2}")
    if scale.size != m * kp // GROUP:
        raise ValueError(f"len(scale)={scale.size} want {m * kp // GROUP}")
    out = np.empty((m, k), dtype=np.float32)
    rc = lib().or_nf4_decode(_ptr(packed), _ptr(scale), m, k, _ptr(out))
    if rc != 0:
        raise ValueError(f"decode rc={rc}")
    return out


def c_matmul_f32(w: np.ndarray, x: np.ndarray) -> np.ndarray:
    """``[M,K] @ [K,N]`` in float32, accumulation in k order."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    x = np.ascontiguousarray(x, dtype=np.float32)
    if x.ndim == 1:
        x = x[:, None]
    m, k = w.shape
    n = x.shape[1]
    y = np.empty((m, n), dtype=np.float32)
    lib().or_matmul_f32(_ptr(w), _ptr(x), m, k, n, _ptr(y))
    return y


def c_matmul_f64(w: np.ndarray, x: np.ndarray) -> np.ndarray:
    w = np.ascontiguousarray(w, dtype=np.float32)
    x = np.ascontiguousarray(x, dtype=np.float32)
    if x.ndim == 1:
        x = x[:, None]
    m, k = w.shape
    n = x.shape[1]
    y = np.empty((m, n), dtype=np.float64)
    lib().or_matmul_f64(_ptr(w), _ptr(x), m, k, n, _ptr(y))
    return y


def c_linear(packed: np.ndarray, scale: np.ndarray, m: int, k: int, x: np.ndarray) -> np.ndarray:
    """The reference's CPU linear: decode to float32, then float32 matmul."""
    return c_matmul_f32(c_decode(packed, scale, m, k), x)


def f32_to_f16_bits(a: np.ndarray) -> np.ndarray:
    L = lib()
    flat = np.asarray(a, dtype=np.float32).reshape(-1)
    return np.array([L.or_f32_to_f16(float(v)) for v in flat], dtype=np.uint16).reshape(np.shape(a))


def f16_bits_to_f32(a: np.ndarray) -> np.ndarray:
    L = lib()
    flat = np.asarray(a, dtype=np.uint16).reshape(-1)
    return np.array([L.or_f16_to_f32(int(v)) for v in flat], dtype=np.float32).reshape(np.shape(a))


# ----------------------------------------------------------------------------
# bf16 helpers in numpy (closed form of internal/f16/f16.go:93-106)
# ----------------------------------------------------------------------------
def bf16_round_bits(a: np.ndarray) -> np.ndarray:
    """float32 -> bfloat16 bit patterns, round to nearest even, NaN kept NaN."""
    b = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (b & 0x7FFFFFFF) > 0x7F800000
    r = ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)
    n = (b >> 16).astype(np.uint16)
    n = np.where((n & 0x7F) == 0, n | 1, n).astype(np.uint16)
    return np.where(nan, n, r).astype(np.uint16)


def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def bf16_round(a: np.ndarray) -> np.ndarray:
    """float32 values rounded to the nearest bfloat16, returned as float32."""
    return bf16_bits_to_f32(bf16_round_bits(a)).reshape(np.shape(a))


# ----------------------------------------------------------------------------
# numpy restatement (independent of the C one)
# ----------------------------------------------------------------------------
def np_unpack(packed: np.ndarray) -> np.ndarray:
    """``[M, K_pad/2]`` bytes -> ``[M, K_pad]`` codes; low nibble is the even column."""
    packed = np.asarray(packed, dtype=np.uint8)
    m, half = packed.shape
    codes = np.empty((m, 2 * half), dtype=np.uint8)
    codes[:, 0::2] = packed & 0x0F
    codes[:, 1::2] = packed >> 4
    return codes


def np_pack(codes: np.ndarray) -> np.ndarray:
    codes = np.asarray(codes, dtype=np.uint8)
    return ((codes[:, 1::2] << 4) | codes[:, 0::2]).astype(np.uint8)


def np_decode(packed: np.ndarray, scale: np.ndarray, m: int, k: int) -> np.ndarray:
    kp = k_pad(k)
    ng = kp // GROUP
    packed = np.asarray(packed, dtype=np.uint8).reshape(m, kp // 2)
    s = np.asarray(scale).view(np.float16).reshape(m, ng).astype(np.float32)
    w = LUT[np_unpack(packed)].reshape(m, ng, GROUP) * s[:, :, None]
    return np.ascontiguousarray(w.reshape(m, kp)[:, :k])


def np_encode(w: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """Vectorised encode, including the tiny/huge scale clamp of the Go codec."""
    w = np.asarray(w, dtype=np.float32)
    if w.ndim != 2 or w.shape[0] < 1 or w.shape[1] < 1:
        raise EncodeError("empty shape")
    if not np.isfinite(w).all():
        raise EncodeError("non-finite weight")
    m, k = w.shape
    kp = k_pad(k)
    ng = kp // GROUP
    g = np.zeros((m, kp), dtype=np.float32)
    g[:, :k] = w
    g = g.reshape(m, ng, GROUP)
    s32 = np.abs(g).max(axis=2).astype(np.float32)
    s32 = np.where(s32 == 0, np.float32(1), s32).astype(np.float32)
    with np.errstate(over="ignore"):
        s16 = s32.astype(np.float16)
    bad = ~np.isfinite(s16) | (s16 <= 0)
    if bad.any():
        fix = np.where(s32 > np.float32(65504), np.float32(65504), np.float32(1)).astype(np.float32)
        s16 = np.where(bad, fix.astype(np.float16), s16)
    s = s16.astype(np.float32)
    u = np.clip(g / s[:, :, None], np.float32(-1), np.float32(1)).astype(np.float32)
    d = (u[..., None] - LUT).astype(np.float32)
    codes = np.argmin((d * d).astype(np.float32), axis=-1).astype(np.uint8).reshape(m, kp)
    return np_pack(codes), s16


def toy_blobs(m: int, k: int, seed: int, *, pad_garbage: bool = True):
    """Uniform random codes and weight-like scales, the shape of the reference's
    toy fixture (``gpu/tests/nf4_oracle.py:295-319``): codes cover all sixteen
    levels, scales sit in [0.012, 0.055] so |y| stays O(1) at rms(x) ~ 1, and the
    padding columns hold garbage unless asked otherwise."""
    kp = k_pad(k)
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 16, size=(m, kp), dtype=np.uint8)
    if not pad_garbage and kp > k:
        codes[:, k:] = 7
    scale = rng.uniform(0.012, 0.055, size=(m, kp // GROUP)).astype(np.float16)
    return np_pack(codes), scale
