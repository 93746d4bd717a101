"""The checker that reads the ring GEMV kernels' generated code back: it must pass on what
the build produced and must catch each kind of problem it exists for."""

from __future__ import annotations

import os

import pytest

from deepfold_amd import build_ext, ring_asm_check as chk

NAME = "_ZN3chr12_GLOBAL__N_114gemv_ring_rowsILi5ELi1ELb1EEEvNS0_10StreamArgsE"


def listing(body: str) -> str:
    return f"{NAME}:\n{body}\n.Lfunc_end0:\n"


GOOD = """
	v_mov_b32_e32 v1, 0
	;;#ASMSTART
	s_nop 4
	global_load_dwordx2 v[104:105], v1, s[4:5] offset:0 nt
	;;#ASMEND
	;;#ASMSTART
	global_load_dwordx4 v[8:11], v[2:3], off
	;;#ASMEND
	v_add_u32_e32 v1, 1, v1
	;;#ASMSTART
	s_waitcnt vmcnt(2) ; covers v[8:11]
	;;#ASMEND
	v_mov_b32_e32 v9, 0
	s_endpgm
"""


def test_a_sound_listing_passes():
    assert chk.check_assembly(listing(GOOD)) == []


def test_compiler_code_in_a_reserved_register_is_found():
    bad = GOOD.replace("v_add_u32_e32 v1, 1, v1", "v_add_u32_e32 v104, 1, v1")
    assert any("reserved registers [104]" in p for p in chk.check_assembly(listing(bad)))


def test_touching_a_register_in_flight_is_found_across_a_branch():
    bad = GOOD.replace("v_add_u32_e32 v1, 1, v1",
                       "s_cbranch_scc1 .LBB0_2\n\tv_add_u32_e32 v1, 1, v1\n.LBB0_2:\n\tv_mov_b32_e32 v12, v10")
    assert any("still being written: [10]" in p for p in chk.check_assembly(listing(bad)))


def test_a_restored_scalar_used_too_soon_by_an_asm_load_is_found():
    bad = GOOD.replace("\t;;#ASMSTART\n\ts_nop 4\n", "\tv_readlane_b32 s5, v78, 1\n\t;;#ASMSTART\n\ts_nop 1\n", 1)
    found = chk.check_assembly(listing(bad))
    assert any("reads s5 2 wait states after" in p for p in found), found
    ok = GOOD.replace("\t;;#ASMSTART\n\ts_nop 4\n", "\tv_readlane_b32 s5, v78, 1\n\t;;#ASMSTART\n\ts_nop 4\n", 1)
    assert chk.check_assembly(listing(ok)) == []


def test_spills_are_found():
    bad = GOOD.replace("v_add_u32_e32 v1, 1, v1", "scratch_store_dword off, v1, off offset:4")
    assert any("scratch instructions" in p for p in chk.check_assembly(listing(bad)))


def test_a_listing_without_ring_kernels_is_refused():
    assert chk.check_assembly("nothing here\n")


@pytest.mark.skipif(not build_ext.have_hipcc(), reason="needs hipcc")
def test_the_built_kernels_pass():
    chk.check_source(build_ext.hipcc(), build_ext.HIPCC_FLAGS, os.path.join(build_ext.CSRC, "nf4_gemv.hip"))
