"""The build's scan for scalar-register hazards around memory instructions issued from asm statements."""
from eshkol_amd.build import sgpr_to_vmem_hazards

RELOAD_THEN_ATOMIC = """
	v_readlane_b32 s10, v233, 9
	v_mov_b32_e32 v3, s58
	v_readlane_b32 s11, v233, 10
	;;#ASMSTART
	global_atomic_add v182, v3, v2, s[10:11] sc0
	;;#ASMEND
"""

RELOAD_NOPS_ATOMIC = """
	v_readlane_b32 s10, v233, 9
	v_mov_b32_e32 v3, s58
	v_readlane_b32 s11, v233, 10
	;;#ASMSTART
	s_nop 4
	global_atomic_add v182, v3, v2, s[10:11] sc0
	;;#ASMEND
"""


def test_a_memory_instruction_right_behind_the_reload_of_its_address_is_found():
    found = sgpr_to_vmem_hazards(RELOAD_THEN_ATOMIC)
    assert [(f[0], f[2]) for f in found] == [(6, 2), (6, 0)]


def test_five_wait_states_clear_it():
    assert sgpr_to_vmem_hazards(RELOAD_NOPS_ATOMIC) == []


def test_other_scalar_registers_and_scalar_writers_do_not_count():
    asm = """
	v_readfirstlane_b32 s4, v0
	s_mov_b32 s20, s4
	buffer_load_dwordx4 v[0:3], v4, s[8:11], s20 offen
	v_cmp_eq_u32_e64 s[12:13], 0, v1
	s_nop 1
	s_nop 1
	global_load_dword v5, v6, s[12:13]
	v_readlane_b32 s30, v7, 1
	s_nop 4
	global_load_dword v5, v6, s[30:31]
"""
    found = sgpr_to_vmem_hazards(asm)
    assert [(f[0], f[2]) for f in found] == [(8, 4)]
