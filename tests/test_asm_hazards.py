"""The generated device code around the hand-written vector-memory instructions.

The compiler's hazard recognizer does not look into asm statements; a load issued from one must
not read a scalar register that a vector instruction wrote fewer than five wait states earlier
(a spilled buffer descriptor restored with v_readlane_b32 right in front of a hidden load made that
load return zeros).  ``cumm_amd.build.find_asm_hazards`` scans device assembly for that pattern:
checked here on hand-made snippets, then on the assembly of every translation unit of the library
(compiled on first use and after a source change; about a minute of hipcc on eight cores).
"""
import shutil

import pytest

from cumm_amd import build

BAD = """
kernel_a:
	v_readlane_b32 s4, v168, 38
	v_readlane_b32 s5, v168, 39
	v_readlane_b32 s6, v168, 40
	v_readlane_b32 s7, v168, 41
	;;#ASMSTART
	buffer_load_dword v9, v2, s[4:7], 0 offen
	;;#ASMEND
	s_endpgm
"""

GOOD_NOPS = """
kernel_b:
	v_readlane_b32 s7, v168, 41
	;;#ASMSTART
	s_nop 4
	buffer_load_dword v9, v2, s[4:7], 0 offen
	;;#ASMEND
"""

GOOD_DISTANCE = """
kernel_c:
	v_readfirstlane_b32 s34, v3
	v_add_u32_e32 v1, v2, v3
	v_add_u32_e32 v1, v2, v3
	v_add_u32_e32 v1, v2, v3
	;;#ASMSTART
	s_mov_b32 m0, s43
	s_nop 0
	buffer_load_dwordx4 v66, s[4:7], s34 offen lds
	;;#ASMEND
"""

BAD_OFFSET = """
kernel_d:
	v_readfirstlane_b32 s34, v3
	v_add_u32_e32 v1, v2, v3
	;;#ASMSTART
	s_mov_b32 m0, s43
	s_nop 0
	buffer_load_dwordx4 v66, s[4:7], s34 offen lds
	;;#ASMEND
"""

SCALAR_WRITER = """
kernel_e:
	s_mul_i32 s34, s2, s3
	;;#ASMSTART
	s_mov_b32 m0, s43
	s_nop 0
	buffer_load_dwordx4 v66, s[4:7], s34 offen lds
	;;#ASMEND
"""

COMPILER_LOAD = """
kernel_f:
	v_readlane_b32 s7, v168, 41
	buffer_load_dword v9, v2, s[4:7], 0 offen
"""


def test_finder_on_snippets():
    hits = build.find_asm_hazards(BAD)
    assert len(hits) == 1 and hits[0][0] == "kernel_a" and "v_readlane_b32 s7" in hits[0][3]
    assert build.find_asm_hazards(GOOD_NOPS) == []
    assert build.find_asm_hazards(GOOD_DISTANCE) == []
    hits = build.find_asm_hazards(BAD_OFFSET)
    assert len(hits) == 1 and "s34" in hits[0][3]
    # a scalar instruction's result is interlocked; loads the compiler emitted are its own business
    assert build.find_asm_hazards(SCALAR_WRITER) == []
    assert build.find_asm_hazards(COMPILER_LOAD) == []
    # a compare into a register pair that the descriptor overlaps
    assert len(build.find_asm_hazards(BAD.replace("v_readlane_b32 s7, v168, 41", "v_cmp_gt_i32_e64 s[6:7], v1, v2"))) == 1


@pytest.mark.skipif(shutil.which(build.HIPCC) is None, reason="hipcc not found")
def test_no_hazard_in_the_library():
    hits = build.check_asm_hazards()
    assert hits == [], "\n".join("%s: %s line %d: %s   <- %s" % h for h in hits)
