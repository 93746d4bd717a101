"""The streaming ring: its host-visible protocol on CPU slots (no kernel launches), and on
the GPU the same results from a streamed matrix as from a resident one."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from deepfold_amd import ring as rg
from oracle import nf4_oracle as oc


def image(m, k, seed):
    p, s = oc.toy_blobs(m, k, seed)
    return rg.HostImage.from_blobs(torch.from_numpy(p), torch.from_numpy(np.ascontiguousarray(s).view(np.float16)), k)


def tape(n, m=8, k=128):
    return [rg.StreamedMatrix.on_host(f"L{i}", image(m, k, i)) for i in range(n)]


def cpu_ring(n_slots=2, nbytes=None, **kw):
    nbytes = rg.arena_nbytes(8, 128) if nbytes is None else nbytes
    return rg.CopyRing(rg.SlotPair(nbytes, "cpu", n_slots), **kw)


# ---- host image and slots -------------------------------------------------------------

def test_arena_is_packed_then_scale_and_views_share_storage():
    p, s = oc.toy_blobs(5, 200, 3)
    tp, ts = torch.from_numpy(p), torch.from_numpy(np.ascontiguousarray(s).view(np.float16))
    img = rg.HostImage.from_blobs(tp, ts, 200)
    assert img.K_pad == 256 and img.nbytes == 5 * 128 + 5 * 4 * 2 == rg.arena_nbytes(5, 200)
    assert (img.arena[: 5 * 128].numpy() == p.reshape(-1)).all()
    assert (img.arena[5 * 128:].numpy() == np.ascontiguousarray(s).view(np.uint8).reshape(-1)).all()
    assert torch.equal(img.packed, tp) and torch.equal(img.scale, ts)
    assert img.packed.data_ptr() == img.arena.data_ptr()
    assert img.scale.data_ptr() == img.arena.data_ptr() + 5 * 128
    assert rg.is_pinned(img.arena) == torch.cuda.is_available()


def test_pack_arena_rejects_wrong_inputs():
    p = torch.zeros((4, 32), dtype=torch.uint8)
    s = torch.zeros((4, 1), dtype=torch.float16)
    with pytest.raises(TypeError):
        rg.pack_arena(p.to(torch.int8), s)
    with pytest.raises(TypeError):
        rg.pack_arena(p, s.float())
    with pytest.raises(ValueError):
        rg.pack_arena(p, torch.zeros((3, 1), dtype=torch.float16))
    with pytest.raises(ValueError):
        rg.pack_arena(p, torch.zeros((4, 2), dtype=torch.float16))
    with pytest.raises(ValueError):
        rg.pack_arena(p.reshape(-1), s)
    with pytest.raises(ValueError):
        rg.HostImage.from_blobs(p, s, 200)
    with pytest.raises(ValueError):
        rg.unpack_arena(torch.zeros(7, dtype=torch.uint8), 4, 64)


def test_slot_views_and_limits():
    sp = rg.SlotPair(rg.arena_nbytes(8, 128), "cpu")
    assert sp.count == 2 and len(sp.arena) == 2
    packed, scale = sp.view(1, 8, 128, 128)
    assert packed.shape == (8, 64) and scale.shape == (8, 2) and scale.dtype == torch.float16
    assert packed.data_ptr() == sp.arena[1].data_ptr()
    small = sp.view(0, 2, 64, 64)[0]
    assert small.shape == (2, 32)
    with pytest.raises(ValueError):
        sp.view(0, 16, 128, 128)
    with pytest.raises(IndexError):
        sp.view(2, 8, 128, 128)
    with pytest.raises(ValueError):
        rg.SlotPair(16, "cpu", count=1)
    with pytest.raises(ValueError):
        rg.SlotPair(-1, "cpu")


# ---- protocol (gpu/loop/test_ring.py:143-845) -------------------------------------------

def test_issue_logs_wait_copy_record_in_that_order():
    r = cpu_ring()
    t = tape(1)
    r.arm(t)
    s = r.issue(t[0])
    assert s == 0
    assert r.ops == [("wait_gemm", 0), ("h2d", 0, t[0].host_image.nbytes), ("record_copy", 0)]
    assert r.ahead == 1 and r.issue_count == 1


def test_two_slots_allow_one_copy_ahead():
    r = cpu_ring()
    assert r.max_ahead == 1 and r.n_copy_streams == 1
    t = tape(2)
    r.arm(t)
    r.issue(t[0])
    with pytest.raises(RuntimeError, match="prefetch depth"):
        r.issue(t[1])


def test_bind_returns_slot_views_with_the_matrix_bytes():
    r = cpu_ring()
    t = tape(1)
    r.arm(t)
    r.prefetch()
    packed, scale = r.bind_for_gemm(t[0])
    assert packed.data_ptr() == r.slots.arena[0].data_ptr()
    assert packed.data_ptr() != t[0].host_image.arena.data_ptr()
    assert torch.equal(packed, t[0].host_image.packed) and torch.equal(scale, t[0].host_image.scale)
    r.record_gemm(t[0])


def test_bind_issues_the_next_copy_before_the_gemm_is_recorded():
    r = cpu_ring()
    t = tape(3)
    r.arm(t)
    r.prefetch()
    r.bind_for_gemm(t[0])
    kinds = [op[0] for op in r.ops]
    # copy 0, wait for it, then copy 1 goes out while matrix 0 is still bound
    assert kinds == ["wait_gemm", "h2d", "record_copy", "wait_copy", "wait_gemm", "h2d", "record_copy"]
    assert r.ops[3] == ("wait_copy", 0) and r.ops[5][1] == 1
    r.record_gemm(t[0])
    assert r.ops[-1] == ("record_gemm", 0)


def test_slot_order_over_a_tape():
    r = cpu_ring()
    t = tape(3)
    r.arm(t)
    r.prefetch()
    for g in t:
        r.bind_for_gemm(g)
        r.record_gemm(g)
    assert r.slot_order == [0, 1, 0]
    r3 = cpu_ring(3)
    assert r3.max_ahead == 2
    t4 = tape(4)
    r3.arm(t4)
    r3.prefetch()
    assert r3.ahead == 2
    for g in t4:
        r3.bind_for_gemm(g)
        r3.record_gemm(g)
    assert r3.slot_order == [0, 1, 2, 0]


def test_arm_resets_the_forward_and_keeps_the_totals():
    r = cpu_ring()
    t = tape(2)
    for fwd in range(2):
        r.arm(t)
        r.prefetch()
        for g in t:
            r.bind_for_gemm(g)
            r.record_gemm(g)
        assert r.issue_count == 2 and r.forward_bytes == 2 * t[0].host_image.nbytes
    snap = r.snapshot()
    assert snap["total_copies"] == 4 and snap["total_forwards"] == 2
    assert snap["total_bytes"] == 4 * t[0].host_image.nbytes and snap["cuda"] is False
    assert snap["forward_copy_ms"] is None
    r.arm(t)
    assert r.issue_count == 0 and r.forward_bytes == 0 and r.ops == [] and r.slot_order == []


def test_prefetch_next_is_not_copied_twice():
    r = cpu_ring()
    t = tape(3)
    r.arm(t)
    r.prefetch()
    for g in t:
        r.bind_for_gemm(g)
        r.record_gemm(g)
    before = r.total_copies
    r.prefetch_next()                       # head of the next forward, during lm_head
    assert r.total_copies == before + 1 and r.ahead == 1
    r.arm(t)
    r.prefetch()                            # nothing new: L0 is already in flight
    assert r.total_copies == before + 1
    packed, _ = r.bind_for_gemm(t[0])
    assert torch.equal(packed, t[0].host_image.packed)
    r.record_gemm(t[0])
    assert r.total_copies == before + 2     # bind issued L1
    # a different tape after prefetch_next drops the carried copy
    r2 = cpu_ring()
    r2.arm(t)
    r2.prefetch()
    for g in t:
        r2.bind_for_gemm(g)
        r2.record_gemm(g)
    r2.prefetch_next()
    other = tape(2, m=4, k=64)
    for i, g in enumerate(other):
        g.name = f"X{i}"
    r2.arm(other)
    assert r2.ahead == 0
    r2.prefetch()
    assert torch.equal(r2.bind_for_gemm(other[0])[0], other[0].host_image.packed)


def test_prefetch_next_waits_for_the_tape_to_finish():
    r = cpu_ring()
    t = tape(3)
    r.arm(t)
    r.prefetch()
    r.prefetch_next()
    assert r.total_copies == 1              # forward not finished: no-op
    r.bind_for_gemm(t[0])
    r.prefetch_next()
    assert r.total_copies == 2              # only the copy bind itself issued


def test_hold_is_one_copy_for_many_gemms():
    r = cpu_ring()
    t = tape(2)
    r.arm(t)
    r.prefetch()
    packed, _ = r.bind_hold(t[0])
    for _ in range(5):
        r.gemm_hold()
    assert r.total_copies == 1              # nothing prefetched during the hold
    with pytest.raises(RuntimeError, match="hold already active"):
        r.bind_hold(t[1])
    with pytest.raises(RuntimeError):
        r.bind_for_gemm(t[1])
    r.release_hold(t[0])
    assert r.total_copies == 2 and r.ops[-4:] == [("record_gemm", 0), ("wait_gemm", 1),
                                                  ("h2d", 1, t[1].host_image.nbytes), ("record_copy", 1)]
    with pytest.raises(RuntimeError, match="no active hold"):
        r.gemm_hold()


def test_misuse_is_refused():
    r = cpu_ring()
    t = tape(2)
    r.arm(t)
    with pytest.raises(RuntimeError, match="no active bind"):
        r.record_gemm()
    r.prefetch()
    with pytest.raises(RuntimeError, match="queue head"):
        r.bind_for_gemm(t[1])
    r.bind_for_gemm(t[0])
    with pytest.raises(RuntimeError, match="active is"):
        r.record_gemm(t[1])
    r.record_gemm(t[0])
    resident = rg.StreamedMatrix("res", 8, 128, 128, "device", None, torch.zeros(1), torch.ones(1))
    fresh = cpu_ring()
    with pytest.raises(RuntimeError, match="HOST"):
        fresh.issue(resident)
    with pytest.raises(RuntimeError, match="HOST"):
        fresh.bind_hold(resident)
    assert r.bind_for_gemm(resident)[1] is resident.scale          # resident: passes through
    big = rg.StreamedMatrix.on_host("big", image(64, 128, 1))
    r2 = cpu_ring()
    r2.arm([big])
    with pytest.raises(ValueError, match="exceeds slot"):
        r2.issue(big)
    with pytest.raises(ValueError):
        rg.CopyRing(rg.SlotPair(16, "cpu"), n_copy_streams=0)


def test_bind_without_prefetch_issues_the_copy_itself():
    r = cpu_ring()
    t = tape(2)
    r.arm(t)
    packed, _ = r.bind_for_gemm(t[0])       # no prefetch() before
    assert torch.equal(packed, t[0].host_image.packed)
    assert r.slot_order == [0, 1]           # and the next one followed
    r.record_gemm(t[0])
    assert torch.equal(r.bind_for_gemm(t[1])[0], t[1].host_image.packed)


def test_join_knob(monkeypatch):
    monkeypatch.delenv("DEEPFOLD_COPY_JOIN", raising=False)
    assert rg.default_join_copy() is False
    monkeypatch.setenv("DEEPFOLD_COPY_JOIN", "1")
    assert rg.default_join_copy() is True
    monkeypatch.setenv("DEEPFOLD_COPY_JOIN", "off")
    assert rg.default_join_copy() is False


# ---- GPU: streamed == resident -----------------------------------------------------------

@pytest.mark.gpu
def test_streamed_gemv_and_gemm_equal_resident():
    from deepfold_amd import nf4
    shapes = [(256, 512), (512, 256), (128, 1088), (256, 512)]
    images = [image(m, k, 10 + i) for i, (m, k) in enumerate(shapes)]
    t = [rg.StreamedMatrix.on_host(f"W{i}", im) for i, im in enumerate(images)]
    slots = rg.SlotPair(max(im.nbytes for im in images), "cuda")
    r = rg.CopyRing(slots, timing=True)
    rng = np.random.default_rng(0)
    for fwd in range(3):
        r.arm(t)
        r.prefetch()
        for g, im in zip(t, images):
            x1 = torch.from_numpy(rng.standard_normal(g.K).astype(np.float32)).to(torch.bfloat16).cuda()
            xn = torch.from_numpy(rng.standard_normal((g.K, 8)).astype(np.float32)).to(torch.bfloat16).cuda()
            dp, ds = im.packed.cuda(), im.scale.cuda()
            want1 = nf4.nf4_gemv(dp, ds, x1, g.M, g.K, g.K_pad).view(-1)
            wantn = nf4.nf4_gemm(dp, ds, xn, g.M, g.K, g.K_pad)
            packed, scale = r.bind_hold(g)
            assert packed.is_cuda and packed.data_ptr() in {a.data_ptr() for a in slots.arena}
            got1 = nf4.nf4_gemv(packed, scale, x1, g.M, g.K, g.K_pad).view(-1)
            gotn = nf4.nf4_gemm(packed, scale, xn, g.M, g.K, g.K_pad)
            r.release_hold(g)
            assert torch.equal(got1, want1) and torch.equal(gotn, wantn), (fwd, g.name)
        r.prefetch_next()
    torch.cuda.synchronize()
    snap = r.snapshot()
    assert snap["cuda"] and snap["total_copies"] == 3 * len(t) + 1
    assert snap["total_copy_ms"] > 0


@pytest.mark.gpu
def test_streamed_linear_over_many_forwards_never_reads_a_stale_slot():
    """Every matrix has its own bytes; a kernel launched on a slot that was overwritten too
    early, or read too early, would give another matrix's product."""
    from deepfold_amd import nf4
    m, k, n_mat = 1024, 2048, 6
    images = [image(m, k, 100 + i) for i in range(n_mat)]
    t = [rg.StreamedMatrix.on_host(f"F{i}", im) for i, im in enumerate(images)]
    r = rg.CopyRing(rg.SlotPair(images[0].nbytes, "cuda"))
    x = torch.from_numpy(np.random.default_rng(1).standard_normal(k).astype(np.float32)).to(torch.bfloat16).cuda()
    want = [nf4.nf4_gemv(im.packed.cuda(), im.scale.cuda(), x, m, k, k).view(-1).clone() for im in images]
    for fwd in range(5):
        r.arm(t)
        r.prefetch()
        outs = [rg.streamed_linear(r, g, x).clone() for g in t]
        r.prefetch_next()
        for i, (a, b) in enumerate(zip(outs, want)):
            assert torch.equal(a, b), (fwd, i)
    assert r.total_copies == 5 * n_mat + 1       # the head of each next forward is copied once
