"""``CompressedLinear``: the ``nn.Linear``-shaped seat (``gpu/host/linear.py:84-220``).
Host logic on the CPU; the forward against ``F.linear`` on the decoded matrix on the GPU."""

from __future__ import annotations

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from deepfold_amd import nf4
from deepfold_amd.chr0.loader import ChrMatrix
from deepfold_amd.host import CompressedLinear, k_pad, nf4_linear
from deepfold_amd.ring import HostImage
from oracle import nf4_oracle as oc

from helpers import staged_gemv_model, takes_staged_gemv


def blobs(m, k, seed=0, sigma=0.05):
    w = np.random.default_rng(seed).standard_normal((m, k)).astype(np.float32) * sigma
    p, s = oc.c_encode(w)
    return torch.from_numpy(p), torch.from_numpy(np.ascontiguousarray(s).view(np.float16))


def test_no_dense_weight_is_ever_owned():
    lin = CompressedLinear(200, 48, bias=True)
    assert lin.K == 200 and lin.M == 48 and lin.K_pad == k_pad(200) == 256 and lin.n_groups == 4
    assert lin.home == "empty" and not lin.is_loaded and lin.nbytes == 0
    assert lin.weight.numel() == 0 and lin.weight.dtype == torch.bfloat16
    assert list(lin.parameters()) == [] and lin.state_dict() == {}
    with pytest.raises(AttributeError):
        lin.weight = torch.zeros(48, 200)          # a stray dense weight must fail loudly
    with pytest.raises(RuntimeError, match="no weights"):
        lin(torch.zeros(1, 200))
    with pytest.raises(ValueError):
        CompressedLinear(0, 4)


def test_attach_checks_and_shares():
    p, s = blobs(48, 200)
    mat = ChrMatrix("blk.0.q", 48, 200, 256, p, s)
    a, b = CompressedLinear(200, 48), CompressedLinear(200, 48)
    a.attach(mat)
    b.attach(mat)
    assert a.packed.data_ptr() == b.packed.data_ptr() == p.data_ptr()   # shared, not copied
    assert a.home == "device" and a.is_loaded and a.chr_name == "blk.0.q"
    assert a.nbytes == p.numel() + 2 * s.numel()
    with pytest.raises(ValueError):
        CompressedLinear(200, 47).attach(mat)
    with pytest.raises(ValueError):
        CompressedLinear(100, 48).attach(ChrMatrix("x", 48, 100, 256, p, s))
    with pytest.raises(TypeError):
        a.attach(ChrMatrix("x", 48, 200, 256, p.to(torch.int8), s))
    with pytest.raises(ValueError, match="bias=False"):
        a.set_bias(torch.zeros(48))
    c = CompressedLinear(200, 48, bias=True)
    with pytest.raises(ValueError):
        c.set_bias(torch.zeros(47))
    c.set_bias(torch.ones(48, dtype=torch.float32))
    assert c.bias.dtype == torch.bfloat16


def test_host_resident_forward_is_refused():
    p, s = blobs(16, 64)
    lin = CompressedLinear(64, 16)
    lin.attach(ChrMatrix("m", 16, 64, 64, p, s))
    lin.attach_host(HostImage.from_blobs(p, s, 64))
    assert lin.home == "host" and lin.is_loaded and lin.nbytes == 0 and lin.packed.numel() == 0
    with pytest.raises(RuntimeError, match="host-resident"):
        lin(torch.zeros(1, 64))
    with pytest.raises(ValueError):
        CompressedLinear(64, 15).attach_host(HostImage.from_blobs(p, s, 64))
    assert "home=host" in repr(lin)


@pytest.mark.gpu
@pytest.mark.parametrize("lead", [(1,), (1, 1), (5,), (2, 16), (3, 33), (70,)])
@pytest.mark.parametrize("bias", [False, True])
def test_forward_matches_linear_on_the_decoded_matrix(lead, bias):
    m, k = 328, 200
    p, s = blobs(m, k, seed=3)
    w = torch.from_numpy(oc.c_decode(p.numpy(), s.numpy().view(np.uint16), m, k).copy()).cuda()
    lin = CompressedLinear(k, m, bias=bias, device="cuda")
    lin.attach(ChrMatrix("t", m, k, k_pad(k), p.cuda(), s.cuda()))
    b = None
    if bias:
        b = torch.randn(m, device="cuda").to(torch.bfloat16)
        lin.set_bias(b)
    g = torch.Generator(device="cuda").manual_seed(7)
    x = torch.randn(*lead, k, generator=g, device="cuda").to(torch.bfloat16)
    y = lin(x)
    assert y.shape == (*lead, m) and y.dtype == torch.bfloat16
    # the split-K tiles multiply bf16-rounded weights (gpu/nf4/nf4_gemm.cu:312-323); whole
    # vectors of up to 32 tokens go to the tile that multiplies bf16(level) and scales each
    # group's sum; one token goes to the GEMV, which keeps the weights in fp32
    # (the module feeds the GEMM windows of at most 32 tokens: the expectation goes window by
    # window too)
    n = int(np.prod(lead))
    x2 = x.reshape(n, k)
    parts = []
    for t0 in range(0, n, 32):
        xw = x2[t0:t0 + 32]
        nw = xw.shape[0]
        if nw > 1 and nf4.nf4_plan(m, k, nw)["bm"] in (32, 64):
            model = staged_gemv_model(p.numpy(), s.numpy().view(np.uint16), m, k,
                                      xw.float().cpu().numpy().T, terms=1)
            parts.append(torch.from_numpy(model.T.copy()).cuda().to(torch.bfloat16))
        elif n == 1:
            # K = 200 is ragged, so the one-token launch stages x in LDS and multiplies the
            # levels as that kernel keeps them (tests/helpers.py staged_levels)
            assert takes_staged_gemv(m, k, fused=k % 64 != 0)
            model = staged_gemv_model(p.numpy(), s.numpy().view(np.uint16), m, k, xw.float().cpu().numpy().T)
            parts.append(torch.from_numpy(model.T.copy()).cuda().to(torch.bfloat16))
        else:
            wk = w.to(torch.bfloat16).float()
            parts.append((xw.double() @ wk.double().t()).to(torch.bfloat16))
    want0 = torch.cat(parts, dim=0)
    want = want0 + b if bias else want0
    want0, want = want0.reshape(*lead, m).double(), want.reshape(*lead, m).double()
    err = (y.double() - want).abs()
    # a step of the product before the bias is added may be larger than a step of the sum
    ulp = 2.0 ** (torch.floor(torch.log2(torch.maximum(want.abs(), want0.abs()).clamp_min(2.0 ** -126))) - 7)
    assert bool((err <= 2 * ulp + 1e-3 * want.pow(2).mean().sqrt()).all()), float((err / ulp).max())
    # the same through the functional form and torch's own linear on the decoded weight
    y2 = nf4_linear(x, lin.packed, lin.scale, m, k, k_pad(k), lin.bias if bias else None)
    assert torch.equal(y, y2)
    ref = F.linear(x.float(), w, None if b is None else b.float())
    assert float((y.float() - ref).abs().max()) <= 1e-2 * float(ref.abs().max()) + 1e-3
