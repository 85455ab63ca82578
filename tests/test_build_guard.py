"""The compiler-dependent assumptions of the kernels that track their own loads (scan_px.h, and the
prefetch into accumulation registers of scan_bwd_xdl.h), checked on the assembly hipcc emits for them
(no GPU needed): no register touched while it is the destination of a load in flight, no vector register
spilled where loads land in vector registers.  Plus the scanner itself on hand-made listings."""
from aussm_amd import build


GOOD = """
	;;#ASMSTART
	global_load_dwordx4 v[2:5], v[8:9], off
	;;#ASMEND
	v_add_u32_e32 v10, v11, v12
	;;#ASMSTART
	s_waitcnt vmcnt(0)
	;;#ASMEND
	v_mov_b32_e32 v20, v2
"""
# the value is dead for the compiler, which reuses v[2:3] as the next address while the load is in flight
BAD = """
	;;#ASMSTART
	global_load_dwordx4 v[2:5], v[2:3], off
	;;#ASMEND
	v_lshl_add_u64 v[2:3], s[0:1], 0, v[130:131]
	global_store_dwordx4 v[2:3], v[62:65], off
	;;#ASMSTART
	s_waitcnt vmcnt(0)
	;;#ASMEND
"""
# a wait by count retires the oldest loads only
COUNTED = """
	;;#ASMSTART
	global_load_dwordx4 v[2:5], v[8:9], off
	;;#ASMEND
	;;#ASMSTART
	global_load_dwordx4 v[12:15], v[8:9], off
	;;#ASMEND
	;;#ASMSTART
	s_waitcnt vmcnt(1)
	;;#ASMEND
	v_mov_b32_e32 v20, v2
	v_mov_b32_e32 v21, v12
"""
# the same for a prefetch into accumulation registers: copied out before the wait
ACC_BAD = """
	;;#ASMSTART
	global_load_dwordx4 a[4:7], v[8:9], off
	;;#ASMEND
	v_accvgpr_read_b32 v30, a5
	;;#ASMSTART
	s_waitcnt vmcnt(0)
	;;#ASMEND
	v_accvgpr_read_b32 v31, a6
"""
# a load issued at the end of a loop body and retired at the top of the next iteration: the register is
# touched between the loop's label and the wait, which only the walk over the back-edge sees
LOOP_BAD = """
.LBB0_1:
	v_mov_b32_e32 v40, v2
	;;#ASMSTART
	s_waitcnt vmcnt(0)
	;;#ASMEND
	v_mov_b32_e32 v41, v3
	;;#ASMSTART
	global_load_dwordx4 v[2:5], v[8:9], off
	;;#ASMEND
	s_cbranch_scc1 .LBB0_1
	;;#ASMSTART
	s_waitcnt vmcnt(0)
	;;#ASMEND
"""
LOOP_GOOD = LOOP_BAD.replace("v_mov_b32_e32 v40, v2", "v_mov_b32_e32 v40, v9")


def test_scanner_on_hand_made_listings():
    found = build.scan_listing(LOOP_BAD)
    assert len(found) == 1 and "v40" in found[0][1]
    assert build.scan_listing(LOOP_GOOD) == []
    assert build.scan_listing(GOOD) == []
    assert [ln for ln, _ in build.scan_listing(BAD)] == [5, 6]
    found = build.scan_listing(COUNTED)
    assert len(found) == 1 and "v21" in found[0][1]
    found = build.scan_listing(ACC_BAD)
    assert len(found) == 1 and "a5" in found[0][1]


def test_kernels_keep_loads_in_flight_intact():
    build.check_px_listing(verbose=False)
