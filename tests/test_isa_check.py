"""The static check of hand-tracked loads (sten_amd/isa_check.py) on small synthetic kernels:
it must see a register touched while its load is in flight, honour counted waits, carry the state
of a loop into its next iteration, and tell spills inside a streaming loop from spills outside."""
from sten_amd import isa_check as C


def run(body):
    C.notes.clear()
    return C.check_kernel("_Zk", body.strip("\n").split("\n"))


def test_touch_before_wait_is_found():
    p = run("""
\tglobal_load_dwordx4 v[4:7], v1, s[2:3]
\tv_mov_b32_e32 v9, v5
\ts_waitcnt vmcnt(0)
""")
    assert len(p) == 1 and "v_mov_b32_e32 v9, v5" in p[0]


def test_wait_clears_and_counts_in_order():
    clean = run("""
\tglobal_load_dwordx4 v[4:7], v1, s[2:3]
\tglobal_load_dwordx4 v[8:11], v1, s[2:3] offset:1024
\ts_waitcnt vmcnt(1)
\tv_mov_b32_e32 v20, v5
\ts_waitcnt vmcnt(0)
\tv_mov_b32_e32 v21, v9
""")
    assert clean == []
    early = run("""
\tglobal_load_dwordx4 v[4:7], v1, s[2:3]
\tglobal_load_dwordx4 v[8:11], v1, s[2:3] offset:1024
\ts_waitcnt vmcnt(1)
\tv_mov_b32_e32 v21, v9
""")
    assert len(early) == 1


def test_dma_loads_count_but_write_no_register():
    p = run("""
\tglobal_load_dwordx4 v[4:7], v1, s[2:3]
\tglobal_load_lds_dwordx4 v2, s[4:5]
\ts_waitcnt vmcnt(1)
\tv_add_u32_e32 v2, 1, v2
\tv_mov_b32_e32 v20, v4
""")
    assert p == []


def test_state_carried_around_a_loop():
    # the load at the end of the body is consumed at its top: fine with a wait there, a hazard without
    good = run("""
\tglobal_load_dword v4, v1, s[2:3]
.LBB0_1:
\ts_waitcnt vmcnt(0)
\tv_mov_b32_e32 v9, v4
\tglobal_load_dword v4, v1, s[2:3]
\ts_cbranch_scc1 .LBB0_1
\ts_waitcnt vmcnt(0)
""")
    assert good == []
    bad = run("""
\tglobal_load_dword v4, v1, s[2:3]
\ts_waitcnt vmcnt(0)
.LBB0_1:
\tv_mov_b32_e32 v9, v4
\tglobal_load_dword v4, v1, s[2:3]
\ts_cbranch_scc1 .LBB0_1
\ts_waitcnt vmcnt(0)
""")
    assert len(bad) == 1 and "second iteration" in bad[0]


def test_spill_of_a_register_in_flight_and_spill_in_a_streaming_loop():
    p = run("""
\tglobal_load_dword v4, v1, s[2:3]
\tscratch_store_dword off, v4, off
\ts_waitcnt vmcnt(0)
""")
    assert len(p) == 1 and "scratch_store_dword" in p[0]
    p = run("""
.LBB0_1:
\tglobal_load_dword v4, v1, s[2:3]
\tscratch_store_dword off, v30, off
\ts_waitcnt vmcnt(0)
\ts_cbranch_scc1 .LBB0_1
""")
    assert len(p) == 1 and "inside a loop" in p[0]
    p = run("""
\tscratch_store_dword off, v30, off
.LBB0_1:
\tglobal_load_dword v4, v1, s[2:3]
\ts_waitcnt vmcnt(0)
\ts_cbranch_scc1 .LBB0_1
\tscratch_load_dword v30, off, off
\ts_waitcnt vmcnt(0)
""")
    assert p == [] and len(C.notes) == 2


def test_register_of_an_unused_load_reused_before_the_wait():
    # a load whose result nobody reads (a prefetch beyond the last step) still lands: its
    # destination must not be given to other values before the wait that covers it
    p = run("""
\tglobal_load_dwordx4 v[4:7], v1, s[2:3]
\tv_accvgpr_read_b32 v5, a32
\ts_waitcnt vmcnt(0)
\tv_cvt_f16_f32_e32 v9, v5
""")
    assert len(p) == 1 and "v_accvgpr_read_b32 v5, a32" in p[0]
    ok = run("""
\tglobal_load_dwordx4 v[4:7], v1, s[2:3]
\ts_waitcnt vmcnt(0)
\tv_accvgpr_read_b32 v5, a32
""")
    assert ok == []


def test_unconditional_forward_branch_is_followed():
    # a rotated loop: its body lies behind an unconditional branch to the header and is entered only
    # from there; falling into it after the prologue would report the refill of a set that is in
    # flight, which never runs in that order
    p = run("""
\tglobal_load_dword v4, v1, s[2:3]
\ts_branch .LBB0_2
.LBB0_1:
\tv_mov_b32_e32 v9, v4
\tglobal_load_dword v4, v1, s[2:3]
.LBB0_2:
\ts_waitcnt vmcnt(0)
\ts_cbranch_scc1 .LBB0_1
""")
    assert p == []
    # the same body without the wait in the header is a hazard on the way round
    p = run("""
\tglobal_load_dword v4, v1, s[2:3]
\ts_branch .LBB0_2
.LBB0_1:
\tv_mov_b32_e32 v9, v4
\tglobal_load_dword v4, v1, s[2:3]
.LBB0_2:
\ts_cbranch_scc1 .LBB0_1
\ts_waitcnt vmcnt(0)
""")
    assert len(p) == 1 and "v_mov_b32_e32 v9, v4" in p[0]


def test_only_loads_of_instruction_statements_are_tracked_by_register():
    # with the compiler's marks in the text, its own loads take their place in the queue but their
    # registers are its own business
    p = run("""
\tglobal_load_dword v7, v1, s[2:3]
\tv_mov_b32_e32 v8, v7
\t;;#ASMSTART
\tglobal_load_dword v4, v1, s[2:3]
\t;;#ASMEND
\tv_mov_b32_e32 v9, v4
\ts_waitcnt vmcnt(0)
""")
    assert len(p) == 1 and "v_mov_b32_e32 v9, v4" in p[0]


def test_scalar_register_written_by_the_vector_unit_needs_wait_states_before_a_hand_issued_load():
    p = run("""
\tv_readlane_b32 s2, v201, 27
\tv_readlane_b32 s3, v201, 28
\t;;#ASMSTART
\tglobal_load_dwordx2 v[4:5], v1, s[2:3]
\t;;#ASMEND
\ts_waitcnt vmcnt(0)
""")
    assert len(p) == 1 and "five wait states" in p[0]
    p = run("""
\tv_readlane_b32 s2, v201, 27
\tv_readlane_b32 s3, v201, 28
\t;;#ASMSTART
\ts_nop 4
\tglobal_load_dwordx2 v[4:5], v1, s[2:3]
\t;;#ASMEND
\ts_waitcnt vmcnt(0)
""")
    assert p == []



def test_spill_among_outstanding_hand_issued_loads_is_reported():
    # the compiler's wait for its scratch operation drains the loads that were meant to stay in flight
    p = run("""
\t;;#ASMSTART
\tglobal_load_dwordx4 v[10:13], v2, s[4:5]
\t;;#ASMEND
\tscratch_load_dword v40, off, off offset:4
\t;;#ASMSTART
\ts_waitcnt vmcnt(0)
\t;;#ASMEND
\tv_add_u32_e32 v1, v10, v11
""")
    assert any("scratch traffic while hand-issued loads are outstanding" in q for q in p)
    clean = run("""
\tscratch_store_dword off, v40, off offset:4
\t;;#ASMSTART
\tglobal_load_dwordx4 v[10:13], v2, s[4:5]
\t;;#ASMEND
\t;;#ASMSTART
\ts_waitcnt vmcnt(0)
\t;;#ASMEND
\tv_add_u32_e32 v1, v10, v11
""")
    assert clean == []
