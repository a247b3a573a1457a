"""The static checks of the generated code (yasakani_amd/isa_check.py) - registers touched while a hand-written load into
them is in flight, results of hand-written matrix instructions touched before their passes are through: the checker itself
on small hand-made listings, then the library's sources."""
import os
import shutil

import pytest

from yasakani_amd import isa_check
from yasakani_amd.isa_check import check_kernel


def test_checker_sees_a_copy_in_front_of_a_wait():
    good = """
	;;#ASMSTART
	global_load_dwordx4 v[10:13], v2, s[4:5] offset:0 nt
	;;#ASMEND
	v_add_u32_e32 v3, v4, v5
	;;#ASMSTART
	s_waitcnt vmcnt(0)
	;;#ASMEND
	v_mov_b32_e32 v20, v10
"""
    bad = good.replace("v_add_u32_e32 v3, v4, v5", "v_mov_b64_e32 v[60:61], v[10:11]")
    assert check_kernel(good.split("\n")) == []
    assert len(check_kernel(bad.split("\n"))) == 1
    # a wait that leaves the youngest load in flight retires only the older one
    two = """
	;;#ASMSTART
	global_load_dword v10, v2, s[4:5]
	;;#ASMEND
	;;#ASMSTART
	global_load_dword v11, v2, s[4:5] offset:64
	;;#ASMEND
	;;#ASMSTART
	s_waitcnt vmcnt(1)
	;;#ASMEND
	v_mov_b32_e32 v20, v10
	v_mov_b32_e32 v21, v11
"""
    v = check_kernel(two.split("\n"))
    assert len(v) == 1 and v[0][2] == [11]


def test_checker_sees_a_copy_of_matrix_results_that_comes_too_early():
    from yasakani_amd.isa_check import check_mfma_results
    listing = """
	;;#ASMSTART
	v_mfma_f32_32x32x16_f16 a[16:31], v[2:5], v[6:9], a[16:31]
	;;#ASMEND
	s_add_i32 s4, s4, s5
	s_cmp_lt_i32 s4, s6
	s_cbranch_scc1 .LBB0_2
	v_accvgpr_mov_b32 a40, a31
.LBB0_2:
	v_accvgpr_read_b32 v1, a16
	s_endpgm
"""
    count, bad = check_mfma_results(listing.split("\n"))
    assert count == 1 and len(bad) == 2                      # both the copy on the fall-through path and the read at the label
    drained = listing.replace("s_add_i32 s4, s4, s5", "s_nop 15")
    assert check_mfma_results(drained.split("\n")) == (1, [])
    # a matrix instruction that accumulates onto the same registers is interlocked by the hardware: not a finding
    chained = listing.replace("s_add_i32 s4, s4, s5", "v_mfma_f32_32x32x16_f16 a[16:31], v[10:13], v[6:9], a[16:31]\n\ts_nop 15")
    assert check_mfma_results(chained.split("\n"))[1] == []


def test_checker_sees_an_operand_written_right_in_front_of_a_matrix_instruction():
    from yasakani_amd.isa_check import check_mfma_operands
    listing = """
	v_cvt_pk_f16_f32 v9, v20, v21
	;;#ASMSTART
	v_mfma_f32_16x16x32_f16 a[0:3], v[2:5], v[6:9], a[0:3]
	;;#ASMEND
"""
    assert len(check_mfma_operands(listing.split("\n"))) == 1
    assert check_mfma_operands(listing.replace("v_cvt_pk_f16_f32 v9, v20, v21", "v_cvt_pk_f16_f32 v9, v20, v21\n\ts_nop 2").split("\n")) == []
    assert check_mfma_operands(listing.replace("v9, v20", "v30, v20").split("\n")) == []


@pytest.mark.skipif(shutil.which(isa_check.HIPCC) is None and not os.path.exists(isa_check.HIPCC), reason="hipcc not found")
def test_no_instruction_touches_a_register_with_a_load_in_flight(tmp_path):
    seen, problems = isa_check.check_sources(str(tmp_path))
    assert seen >= 5 * 2 * 14, "the hand-written loads were not found: the check looked at nothing"
    assert not problems, "\n".join(problems[:40])
