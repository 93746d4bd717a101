"""The C-ABI library without a GPU: it loads, exports every symbol the header
declares, refuses bad arguments before any launch, and its planner agrees with
the pure-Python mirror."""

from __future__ import annotations

import ctypes
import os
import re

import numpy as np
import pytest

from deepfold_amd import nf4
from deepfold_amd.nf4 import plan as pyplan

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "chr_nf4_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(chr_(?:nf4|dv2)_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = nf4._load_ext()
    names = header_symbols()
    assert len(names) >= 15
    for name in names:
        assert getattr(lib, name) is not None, name
    assert sorted(n for n, _, _ in nf4.EXPORTS) == names
    assert lib.chr_nf4_abi_version() == 1


def test_struct_layout_matches_the_reference_header():
    # chr_nf4_dev_t: three int32 then two pointers (chr_gpu.h:11-17)
    assert nf4._Dev.M.offset == 0 and nf4._Dev.K.offset == 4 and nf4._Dev.K_pad.offset == 8
    assert nf4._Dev.packed.offset == 16 and nf4._Dev.scale.offset == 24
    assert ctypes.sizeof(nf4._Dev) == 32
    # chr_nf4_plan_t: ten int32 then one int64 (chr_gpu.h:48-60)
    assert nf4._Plan.ws_floats.offset == 40 and ctypes.sizeof(nf4._Plan) == 48


def dev(M, K, K_pad, packed=0x1000, scale=0x2000):
    return nf4._Dev(M, K, K_pad, packed, scale)


def test_argument_checks_return_before_any_launch():
    lib = nf4._load_ext()
    x = y = 0x4000
    good = dev(128, 256, 256)
    # -1 null
    assert lib.chr_nf4_gemv(None, x, y, None, None, None, 0.0) == -1
    assert lib.chr_nf4_gemv(ctypes.byref(good), None, y, None, None, None, 0.0) == -1
    assert lib.chr_nf4_gemm(ctypes.byref(good), None, y, 2, None) == -1
    assert lib.chr_nf4_gemm_plan(ctypes.byref(good), 1, 1, None) == -1
    assert lib.chr_nf4_rms(None, x, y, 8, 1e-6, None) == -1
    assert lib.chr_nf4_attn(None, x, x, y, x, None, 4, 2, 16, 32, 1.0, None, None, None, None, None, None, 16) == -1
    assert lib.chr_nf4_rope_kv(None, x, x, x, x, x, x, x, 4, 2, 16, 16, None) == -1
    # -2 N out of range
    assert lib.chr_nf4_gemm(ctypes.byref(good), x, y, 0, None) == -2
    assert lib.chr_nf4_gemm(ctypes.byref(good), x, y, 33, None) == -2
    assert lib.chr_nf4_gemm_ws_max(ctypes.byref(good), x, y, 40, None, 0, None, 64) == -2
    assert lib.chr_nf4_gemm_ws_max(ctypes.byref(good), x, y, 2, None, 0, None, 65) == -2
    p = nf4._Plan()
    assert lib.chr_nf4_gemm_plan(ctypes.byref(good), 65, 1, ctypes.byref(p)) == -2
    assert lib.chr_nf4_gemm_plan(ctypes.byref(good), 64, 1, ctypes.byref(p)) == 0
    # -3 bad dims / null blobs
    assert lib.chr_nf4_gemv(ctypes.byref(dev(0, 256, 256)), x, y, None, None, None, 0.0) == -3
    assert lib.chr_nf4_gemv(ctypes.byref(dev(128, 256, 256, packed=None)), x, y, None, None, None, 0.0) == -3
    assert lib.chr_nf4_gemm(ctypes.byref(dev(128, 0, 0)), x, y, 2, None) == -3
    assert lib.chr_nf4_rms(x, x, y, 0, 1e-6, None) == -3
    assert lib.chr_nf4_attn(x, x, x, y, x, x, 5, 2, 16, 32, 1.0, None, None, None, None, None, None, 16) == -3
    assert lib.chr_nf4_attn(x, x, x, y, x, x, 4, 2, 257, 32, 1.0, None, None, None, None, None, None, 16) == -3
    assert lib.chr_nf4_attn(x, x, x, y, x, x, 4, 2, 16, 65, 1.0, None, None, None, None, None, None, 16) == -3
    g, u = dev(128, 256, 256), dev(64, 256, 256)
    assert lib.chr_nf4_gemv_swiglu(ctypes.byref(g), ctypes.byref(u), x, y, None, None, 0.0) == -3
    q, k = dev(128, 256, 256), dev(32, 128, 128)
    assert lib.chr_nf4_gemv_qkv(ctypes.byref(q), ctypes.byref(k), ctypes.byref(k), x, y, y, y,
                                None, None, None, None, None, 0.0) == -3
    # -4 K_pad
    assert lib.chr_nf4_gemv(ctypes.byref(dev(128, 200, 200)), x, y, None, None, None, 0.0) == -4
    assert lib.chr_nf4_gemv(ctypes.byref(dev(128, 192, 256)), x, y, None, None, None, 0.0) == -4
    assert lib.chr_nf4_gemm(ctypes.byref(dev(128, 65, 64)), x, y, 2, None) == -4
    # -5 alignment
    assert lib.chr_nf4_gemv(ctypes.byref(dev(128, 256, 256, packed=0x1008)), x, y, None, None, None, 0.0) == -5
    assert lib.chr_nf4_gemv(ctypes.byref(good), 0x4002, y, None, None, None, 0.0) == -5
    assert lib.chr_nf4_gemm(ctypes.byref(dev(128, 256, 256, scale=0x2001)), x, y, 2, None) == -5
    # -7 workspace smaller than the plan
    nf4.nf4_set_tuning(split_k=4, one_wave=256)
    try:
        assert lib.chr_nf4_gemm_ws(ctypes.byref(dev(128, 2048, 2048)), x, y, 8, 0x8000, 16, None) == -7
    finally:
        nf4.nf4_set_tuning()


def test_wrapper_turns_codes_into_runtime_errors():
    with pytest.raises(RuntimeError, match=r"chr_nf4_gemm_plan failed \(-4\): K_pad"):
        nf4.nf4_plan(128, 100, 1, K_pad=192)
    with pytest.raises(RuntimeError, match=r"\(-2\)"):
        nf4.nf4_plan(128, 128, 65)


SHAPES = [(13824, 5120), (5120, 13824), (5120, 5120), (7168, 5120), (2048, 2048), (256, 2048),
          (151936, 2048), (128, 256), (130, 65), (27648, 5120), (1, 1)]


@pytest.mark.parametrize("have_ws", [True, False])
def test_python_plan_mirrors_the_library(have_ws):
    nf4.nf4_set_tuning(one_wave=256)
    try:
        for M, K in SHAPES:
            for N in (1, 2, 3, 8, 9, 16, 17, 32, 33, 64):
                c = nf4.nf4_plan(M, K, N, have_ws=have_ws)
                p = pyplan.plan(M, K, N, have_ws=have_ws, one_wave=256)
                for key, val in c.items():
                    assert getattr(p, key) == val, (M, K, N, key)
                assert c["ctas"] == c["grid_x"] * c["grid_y"]
                if N > 1 and have_ws:
                    # every split owns at least one K tile and together they cover K
                    assert (c["grid_y"] - 1) * c["tiles_per_split"] < c["n_ktiles"] <= c["grid_y"] * c["tiles_per_split"]
                if not have_ws:
                    assert c["grid_y"] == 1 and c["ws_floats"] == 0
    finally:
        nf4.nf4_set_tuning()


def test_forced_split_and_one_wave():
    nf4.nf4_set_tuning(split_k=3, one_wave=0)
    try:
        c = nf4.nf4_plan(5120, 5120, 16)
        p = pyplan.plan(5120, 5120, 16, force_split=3)
        assert c["grid_y"] == p.grid_y == 3 and c["ws_floats"] == 3 * 5120 * 16
    finally:
        nf4.nf4_set_tuning()


def test_no_cpu_fallback():
    import torch

    packed = torch.zeros((128, 128), dtype=torch.uint8)
    scale = torch.ones((128, 4), dtype=torch.float16)
    x = torch.zeros(256, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="CUDA"):
        nf4.nf4_gemv(packed, scale, x, 128, 256, 256)
    with pytest.raises(RuntimeError, match="CUDA"):
        nf4.nf4_gemm(packed, scale, x.reshape(256, 1).repeat(1, 2), 128, 256, 256)


def test_attention_index_division_by_reciprocal_is_exact_where_the_kernel_uses_it():
    """The decode attention finds (head, part) of a workgroup with ``int((x + 0.5f) * (1.f / d))``
    instead of an integer division (``small_div`` in ``csrc/nf4_attn.hip``); the host passes the
    reciprocal only for x < 2^22 and d <= 256.  The same float32 arithmetic here, every such
    pair."""
    x = np.arange(0, 1 << 22, dtype=np.int64)
    xf = x.astype(np.float32) + np.float32(0.5)
    for d in range(1, 257):
        q = (xf * (np.float32(1.0) / np.float32(d))).astype(np.int64)
        assert np.array_equal(q, x // d), d
