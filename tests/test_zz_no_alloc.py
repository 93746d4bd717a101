"""GPU: ``chr_nf4_gemm_noalloc`` (split-K partials in the library's own device array) against
``chr_nf4_gemm_ws`` with a caller-allocated workspace of the same size, through the C ABI:
bit-equal outputs on two calls in a row, the second on a smaller problem; a launch whose
partials do not fit is refused with -7 by both."""

from __future__ import annotations

import ctypes

import numpy as np
import pytest
import torch

from deepfold_amd import nf4
from oracle import nf4_oracle as oc

pytestmark = pytest.mark.gpu


def _blobs(m, k, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    w = torch.randn((m, k), generator=g, device="cuda", dtype=torch.float32) * 0.02
    return nf4.nf4_quantize(w)


def _both(lib, m, k, n, seed, ws, ws_floats):
    packed, scale = _blobs(m, k, seed)
    g = torch.Generator(device="cuda").manual_seed(seed + 1)
    x = torch.randn((k, n), generator=g, device="cuda").to(torch.bfloat16)
    dev = nf4._dev(packed, scale, m, k, oc.k_pad(k))
    stream = nf4._stream()
    y_ws = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    y_na = torch.ones((m, n), dtype=torch.bfloat16, device="cuda")
    rc_ws = lib.chr_nf4_gemm_ws(ctypes.byref(dev), x.data_ptr(), y_ws.data_ptr(), n, ws.data_ptr(),
                                ws_floats, stream)
    # neither torch's allocator nor the driver hands out memory during the call: the allocator's
    # own count, and the device's free bytes as the driver reports them (a hipMalloc inside the
    # library would show there and only there)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before, _ = torch.cuda.mem_get_info()
    rc_na = lib.chr_nf4_gemm_noalloc(ctypes.byref(dev), x.data_ptr(), y_na.data_ptr(), n, stream)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert torch.cuda.memory_allocated() == before
    assert free_after >= free_before, (free_before, free_after)
    return rc_ws, rc_na, y_ws, y_na, (packed, scale, x)


def test_noalloc_equals_workspace_entry_twice_second_smaller():
    lib = nf4._load_ext()
    ws_floats = int(lib.chr_nf4_gemm_noalloc_max_floats())
    assert ws_floats == 4 << 20
    ws = torch.empty(ws_floats, dtype=torch.float32, device="cuda")
    # first call: a 14B down chunk, split-K over several slices of partials
    m, k, n = 5120, 13824, 32
    plan = nf4.nf4_plan(m, k, n)
    assert plan["grid_y"] > 1 and 0 < plan["ws_floats"] <= ws_floats
    rc_ws, rc_na, y_ws, y_na, (packed, scale, x) = _both(lib, m, k, n, 5, ws, ws_floats)
    assert rc_ws == 0 and rc_na == 0
    assert torch.equal(y_ws.view(torch.int16), y_na.view(torch.int16))
    # and it is the right answer, not two equal wrong ones: sampled rows against the oracle
    rows = np.arange(0, m, 97)
    wd = nf4.nf4_dequant(packed, scale, m, k, k)[torch.from_numpy(rows).cuda()].to(torch.bfloat16).double()
    want = wd @ x.double()
    got = y_na[torch.from_numpy(rows).cuda()].double()
    assert float((got - want).abs().max()) <= 1e-2 * float(want.abs().max())
    # second call, smaller, straight after: stale partials of the first must not show
    m2, k2, n2 = 640, 2048, 5
    assert nf4.nf4_plan(m2, k2, n2)["grid_y"] > 1
    rc_ws, rc_na, y_ws, y_na, _ = _both(lib, m2, k2, n2, 9, ws, ws_floats)
    assert rc_ws == 0 and rc_na == 0
    assert torch.equal(y_ws.view(torch.int16), y_na.view(torch.int16))
    # a chunk that needs no partials (a workgroup takes all of K), through both entries alike
    assert nf4.nf4_plan(7168, 5120, 8)["grid_y"] == 1
    rc_ws, rc_na, y_ws, y_na, _ = _both(lib, 7168, 5120, 8, 10, ws, ws_floats)
    assert rc_ws == 0 and rc_na == 0 and torch.equal(y_ws.view(torch.int16), y_na.view(torch.int16))
    # N = 1 goes to the GEMV (no partials at all) through both entries alike
    rc_ws, rc_na, y_ws, y_na, _ = _both(lib, 512, 1024, 1, 11, ws, ws_floats)
    assert rc_ws == 0 and rc_na == 0 and torch.equal(y_ws.view(torch.int16), y_na.view(torch.int16))


def test_noalloc_refuses_partials_beyond_its_array():
    lib = nf4._load_ext()
    ws_floats = int(lib.chr_nf4_gemm_noalloc_max_floats())
    ws = torch.empty(ws_floats, dtype=torch.float32, device="cuda")
    try:
        nf4.nf4_set_tuning(split_k=16)
        m, k, n = 13824, 5120, 32
        assert nf4.nf4_plan(m, k, n)["ws_floats"] > ws_floats
        rc_ws, rc_na, _, y_na, _ = _both(lib, m, k, n, 13, ws, ws_floats)
    finally:
        nf4.nf4_set_tuning()
    assert rc_ws == -7 and rc_na == -7
    assert bool((y_na == 1).all())          # nothing was launched


def test_noalloc_calls_recorded_into_a_graph():
    """What the entry point is for: its calls recorded during stream capture (after a first
    call on the device outside capture, which looks the array's address up) and replayed, with
    eager work between the replays; every replay gives the workspace entry's bits."""
    lib = nf4._load_ext()
    ws_floats = int(lib.chr_nf4_gemm_noalloc_max_floats())
    ws = torch.empty(ws_floats, dtype=torch.float32, device="cuda")
    shapes = [(5120, 13824, 32, 21), (640, 2048, 5, 22)]
    want, held = [], []
    for m, k, n, seed in shapes:
        rc_ws, rc_na, y_ws, y_na, (packed, scale, x) = _both(lib, m, k, n, seed, ws, ws_floats)
        assert rc_ws == 0 and rc_na == 0
        want.append(y_ws.clone())
        held.append((nf4._dev(packed, scale, m, k, oc.k_pad(k)), packed, scale, x,
                     torch.zeros((m, n), dtype=torch.bfloat16, device="cuda"), n))
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        graph.capture_begin()
        for dev, _, _, x, y, n in held:
            assert lib.chr_nf4_gemm_noalloc(ctypes.byref(dev), x.data_ptr(), y.data_ptr(), n, nf4._stream()) == 0
        graph.capture_end()
    torch.cuda.synchronize()
    for rep in range(3):
        for _, _, _, _, y, _ in held:
            y.fill_(1)
        graph.replay()
        torch.cuda.synchronize()
        for (_, _, _, _, y, _), w in zip(held, want):
            assert torch.equal(y.view(torch.int16), w.view(torch.int16)), rep
        # eager work of the same kind between the replays
        m, k, n, seed = shapes[1]
        rc_ws, rc_na, y_ws, y_na, _ = _both(lib, m, k, n, seed, ws, ws_floats)
        assert rc_ws == 0 and rc_na == 0 and torch.equal(y_ws.view(torch.int16), y_na.view(torch.int16))
