"""The build-time assembly check must catch a register that is touched while an inline-assembly
load into it is still in flight, and must accept the same code once a counted wait covers it."""
from lmdeploy_amd.asm_lint import lint

HEAD = "_ZN5w4a164test_kernelEv:\n"
TAIL = "\ts_endpgm\n.Lfunc_end0:\n"


def load(reg):
    return "\t;;#ASMSTART\n\tglobal_load_dwordx4 v[%d:%d], v40, s[2:3] offset:0\n\t;;#ASMEND\n" % (reg, reg + 3)


def test_clean_counted_wait():
    asm = HEAD + load(0) + load(4) + "\ts_waitcnt vmcnt(1)\n\tv_mov_b32_e32 v20, v1\n" + TAIL
    assert lint(asm) == []


def test_copy_before_wait_is_reported():
    asm = HEAD + load(0) + load(4) + "\tv_mov_b32_e32 v20, v1\n\ts_waitcnt vmcnt(1)\n" + TAIL
    msgs = lint(asm)
    assert len(msgs) == 1 and "v1" in msgs[0]


def test_wait_too_weak_is_reported():
    # vmcnt(1) retires only the older load: v[4:7] may still be in flight
    asm = HEAD + load(0) + load(4) + "\ts_waitcnt vmcnt(1)\n\tv_add_u32_e32 v21, v5, v5\n" + TAIL
    assert len(lint(asm)) == 1


def test_loop_carried_load_is_tracked_across_the_back_edge():
    # the load at the end of the loop body is in flight at the top of the next trip
    asm = (HEAD + load(0) + ".LBB0_1:\n\ts_waitcnt vmcnt(0)\n\tv_mov_b32_e32 v20, v0\n" + load(0)
           + "\tv_mov_b32_e32 v21, v2\n\ts_cbranch_scc1 .LBB0_1\n" + TAIL)
    msgs = lint(asm)
    assert len(msgs) == 1 and "v_mov_b32_e32 v21, v2" in msgs[0]


def test_join_takes_the_younger_position():
    # one path issues a second load, so after the join vmcnt(1) no longer covers v[0:3]... it does:
    # v[0:3] is older on both paths; v[4:7] is only in flight on one of them and must stay flagged
    asm = (HEAD + load(0) + "\ts_cbranch_scc1 .LBB0_2\n" + load(4) + ".LBB0_2:\n\ts_waitcnt vmcnt(1)\n"
           "\tv_mov_b32_e32 v20, v4\n" + TAIL)
    assert len(lint(asm)) == 1


def test_other_functions_are_ignored():
    asm = "_ZN5w4a166helperEv:\n" + load(0) + "\tv_mov_b32_e32 v20, v1\n" + TAIL
    assert lint(asm) == []


def test_parking_an_in_flight_register_in_an_agpr_is_reported():
    # the register allocator saves a VGPR to an AGPR to reuse it, while a load into it is pending:
    # the saved value is stale and the load later lands on the register's new owner
    asm = HEAD + load(48) + "\tv_accvgpr_write_b32 a106, v51\n\ts_waitcnt vmcnt(0)\n" + TAIL
    msgs = lint(asm)
    assert len(msgs) == 1 and "v51" in msgs[0]


def test_parking_a_settled_register_is_accepted():
    asm = HEAD + load(48) + "\ts_waitcnt vmcnt(0)\n\tv_accvgpr_write_b32 a106, v51\n" + TAIL
    assert lint(asm) == []


def mfma(acc):
    return "\t;;#ASMSTART\n\tv_mfma_f32_16x16x32_f16 a[%d:%d], v[0:3], v[4:7], a[%d:%d]\n\t;;#ASMEND\n" % (acc, acc + 3, acc, acc + 3)


def test_accumulator_read_right_after_an_inline_mfma_is_reported():
    asm = HEAD + mfma(8) + "\tv_accvgpr_read_b32 v20, a9\n" + TAIL
    msgs = lint(asm)
    assert len(msgs) == 1 and "wait states" in msgs[0]


def test_accumulator_read_after_the_pipe_has_drained_is_accepted():
    asm = HEAD + mfma(8) + "\t;;#ASMSTART\n\ts_nop 15\n\ts_nop 15\n\t;;#ASMEND\n\tv_accvgpr_read_b32 v20, a9\n" + TAIL
    assert lint(asm) == []


def test_accumulator_move_inside_a_loop_of_inline_mfmas_is_reported():
    # at the top of the body, textually before the MFMA, but reached again across the back edge
    asm = (HEAD + ".LBB0_1:\n\tv_accvgpr_mov_b32 a8, a12\n" + mfma(8) + "\ts_cbranch_scc1 .LBB0_1\n" + TAIL)
    msgs = lint(asm)
    assert any("inside a loop" in m for m in msgs)
