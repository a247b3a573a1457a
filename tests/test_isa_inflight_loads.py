"""The static check of the generated code for registers touched while a hand-written load into them is in flight
(yasakani_amd/isa_check.py): the checker itself on small hand-made listings, then the library's sources."""
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


@pytest.mark.skipif(shutil.which(isa_check.HIPCC) is None and not os.path.exists(isa_check.HIPCC), reason="hipcc not found")
def test_no_instruction_touches_a_register_with_a_load_in_flight(tmp_path):
    seen, problems = isa_check.check_sources(str(tmp_path))
    assert seen >= 5 * 2 * 14, "the hand-written loads were not found: the check looked at nothing"
    assert not problems, "\n".join(problems[:40])
