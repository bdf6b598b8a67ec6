"""The static check of the hand-placed waits (rknpu2_matmul_open_amd/audit_waits.py) on small
pieces of assembly: it must accept the patterns the kernels rely on and flag a register that is
touched between an inline-assembly load and the wait that covers it -- the failure a different
register allocation or schedule of the compiler would cause without any error at build time."""
from rknpu2_matmul_open_amd import audit_waits


def _kernel(body):
    return "_ZN1x14gemm_wk_kernelILi4EEEvv:\n" + body + "\n\ts_endpgm\n"


# a ring of two registers: A is requested ahead of the loop; an iteration requests B, waits for A,
# uses it, requests A again, waits for B, uses it
RING_OK = """
	;;#ASMSTART
	global_load_dwordx4 v[10:13], v1, s[2:3] offset:0
	;;#ASMEND
.LBB0_1:
	;;#ASMSTART
	global_load_dwordx4 v[14:17], v1, s[2:3] offset:0
	;;#ASMEND
	;;#ASMSTART
	s_waitcnt vmcnt(1)
	;;#ASMEND
	v_mfma_i32_32x32x32_i8 v[20:35], v[10:13], v[40:43], v[20:35]
	;;#ASMSTART
	global_load_dwordx4 v[10:13], v1, s[2:3] offset:0
	;;#ASMEND
	;;#ASMSTART
	s_waitcnt vmcnt(1)
	;;#ASMEND
	v_mfma_i32_32x32x32_i8 v[20:35], v[14:17], v[40:43], v[20:35]
	s_cbranch_scc1 .LBB0_1
	;;#ASMSTART
	s_waitcnt vmcnt(0)
	;;#ASMEND
	v_mov_b32_e32 v50, v10
"""


def test_in_order_ring_is_accepted():
    found, checked = audit_waits.audit_text(_kernel(RING_OK))
    assert checked == 1 and found == []


def test_use_before_the_covering_wait_is_flagged():
    # the consumer moved in front of the wait (vmcnt(1) with one younger load covers the older one only)
    bad = RING_OK.replace("""	;;#ASMSTART
	s_waitcnt vmcnt(1)
	;;#ASMEND
	v_mfma_i32_32x32x32_i8 v[20:35], v[10:13], v[40:43], v[20:35]""", """	v_mfma_i32_32x32x32_i8 v[20:35], v[10:13], v[40:43], v[20:35]
	;;#ASMSTART
	s_waitcnt vmcnt(1)
	;;#ASMEND""", 1)
    found, checked = audit_waits.audit_text(_kernel(bad))
    assert checked == 1 and len(found) >= 1 and "v[10:13]" in found[0] and "v_mfma" in found[0]


def test_a_copy_or_spill_of_a_register_in_flight_is_flagged():
    for touch in ("	v_mov_b32_e32 v60, v15", "	scratch_store_dword off, v16, s0 offset:8", "	v_accvgpr_write_b32 a3, v14"):
        bad = RING_OK.replace("	;;#ASMSTART\n	s_waitcnt vmcnt(1)", touch + "\n	;;#ASMSTART\n	s_waitcnt vmcnt(1)", 1)
        found, _ = audit_waits.audit_text(_kernel(bad))
        assert found and "v[14:17]" in found[0], touch


def test_too_loose_a_wait_is_flagged():
    # vmcnt(2) leaves the first load possibly in flight when its data is used
    bad = RING_OK.replace("s_waitcnt vmcnt(1)", "s_waitcnt vmcnt(2)", 1)
    found, _ = audit_waits.audit_text(_kernel(bad))
    assert found


def test_lds_reads_are_covered_by_lgkmcnt0_only():
    ok = """
	;;#ASMSTART
	ds_read_b128 v[4:7], v2 offset:0x800
	;;#ASMEND
	v_mfma_i32_32x32x32_i8 v[20:35], v[40:43], v[44:47], v[20:35]
	;;#ASMSTART
	s_waitcnt lgkmcnt(0)
	;;#ASMEND
	v_mfma_i32_32x32x32_i8 v[20:35], v[40:43], v[4:7], v[20:35]
"""
    assert audit_waits.audit_text(_kernel(ok))[0] == []
    bad = ok.replace("s_waitcnt lgkmcnt(0)", "s_waitcnt vmcnt(0)")
    found, _ = audit_waits.audit_text(_kernel(bad))
    assert found and "ds_read_b128" in found[0]


def test_paths_through_branches_are_followed():
    # the use sits in a block that is reached over a branch, before any wait
    bad = """
	;;#ASMSTART
	global_load_dwordx2 v[8:9], v1, s[2:3] offset:0
	;;#ASMEND
	s_cbranch_scc1 .LBB0_5
	;;#ASMSTART
	s_waitcnt vmcnt(0)
	;;#ASMEND
	s_branch .LBB0_6
.LBB0_5:
	v_add_u32_e32 v3, v8, v3
.LBB0_6:
	;;#ASMSTART
	s_waitcnt vmcnt(0)
	;;#ASMEND
"""
    found, _ = audit_waits.audit_text(_kernel(bad))
    assert len(found) == 1 and "v_add_u32" in found[0]


def test_other_kernels_and_compiler_loads_are_ignored():
    text = "_ZN1x11gemv_kernelILi1EEEvv:\n	global_load_dwordx4 v[10:13], v1, s[2:3]\n	v_mov_b32_e32 v1, v10\n	s_endpgm\n"
    assert audit_waits.audit_text(text) == ([], 0)
    # a load the compiler issued itself (outside an asm block) is the compiler's business
    body = "	global_load_dwordx4 v[10:13], v1, s[2:3]\n	s_waitcnt vmcnt(0)\n	v_mov_b32_e32 v1, v10"
    assert audit_waits.audit_text(_kernel(body)) == ([], 1)
