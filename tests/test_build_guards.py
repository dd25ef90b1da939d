"""The build's scans of the kernels that issue memory instructions from asm statements: scalar-register
hazards in front of them, and registers used while such a load may still be writing them."""
from eshkol_amd.build import hidden_load_violations, sgpr_to_vmem_hazards

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


RING = """
ring_kernel:
	buffer_load_dwordx4 v[0:3], v20, s[8:11], s20 offen
	buffer_load_dwordx4 v[4:7], v20, s[8:11], s20 offen offset:1024
	buffer_load_dwordx4 v20, s[12:15], s20 offen lds
.LBB0_1:
	s_waitcnt vmcnt(%d)
	v_mfma_i32_32x32x32_i8 a[0:15], v[8:11], v[0:3], a[0:15]
	buffer_load_dwordx4 v[0:3], v20, s[8:11], s20 offen
	s_waitcnt vmcnt(2)
	%s
	v_mfma_i32_32x32x32_i8 a[0:15], v[8:11], v[4:7], a[0:15]
	buffer_load_dwordx4 v[4:7], v20, s[8:11], s20 offen offset:1024
	buffer_load_dwordx4 v20, s[12:15], s20 offen lds
	s_cbranch_scc1 .LBB0_1
	s_waitcnt vmcnt(0)
	s_endpgm
	.end_amdhsa_kernel
other_kernel:
	global_load_dword v1, v2, s[0:1]
	v_add_u32 v1, v1, v1
	s_endpgm
"""


def test_a_ring_register_read_after_a_sufficient_wait_is_fine_on_every_path():
    # vmcnt(2): the first load has landed, at the loop's entry and on its back edge alike
    assert hidden_load_violations(RING % (2, "s_nop 0"), ["ring_kernel"]) == []


def test_a_wait_count_one_too_large_is_found():
    found = hidden_load_violations(RING % (3, "s_nop 0"), ["ring_kernel"])
    # the MFMA reads the register in flight, and the next load into it would overtake nothing but is flagged too
    assert [(f[0], f[1], f[3]) for f in found] == [("ring_kernel", 8, [0, 1, 2, 3]), ("ring_kernel", 9, [0, 1, 2, 3])]


def test_a_copy_of_a_ring_register_before_its_wait_is_found():
    # what a compiler that does not know about the hidden load might insert: a move out of a register in flight
    found = hidden_load_violations(RING % (2, "v_accvgpr_write_b32 a20, v0"), ["ring_kernel"])
    assert [(f[1], f[3]) for f in found] == [(11, [0])]
    # only the named kernels are scanned (other_kernel relies on the compiler's own waits)
    assert hidden_load_violations(RING % (2, "s_nop 0"), ["other_kernel"]) != []
