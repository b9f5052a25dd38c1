"""check_asm proves, on device assembly, that nothing touches the destination of a hand-issued register load
before a covering s_waitcnt, and that the scalar registers such an instruction reads have settled (five wait
states after a VALU write, one after a write to M0).  Synthetic listings: the accepted patterns and each way
they can go wrong."""
import os

from llm_kernels_amd import check_asm

HEAD = "kern:\n"
LOAD = "\t;;#ASMSTART\n\tglobal_load_dwordx2 v[10:11], v20, s[2:3]\n\t;;#ASMEND\n"
DMA = "\t;;#ASMSTART\n\ts_mov_b32 m0, s5\n\ts_nop 0\n\tglobal_load_lds_dwordx4 v21, s[6:7]\n\t;;#ASMEND\n"


def _check(tmp_path, body):
    p = os.path.join(tmp_path, "k.s")
    with open(p, "w") as f:
        f.write(HEAD + body + "\ts_endpgm\n")
    return check_asm.check_file(p)


def test_accepts_wait_that_covers_the_load(tmp_path):
    n, bad = _check(tmp_path, LOAD + DMA + DMA + "\tv_add_u32_e32 v1, v2, v3\n\ts_waitcnt vmcnt(2)\n\tv_mov_b32_e32 v4, v10\n")
    assert n == 1 and bad == []


def test_rejects_copy_before_the_wait(tmp_path):
    n, bad = _check(tmp_path, LOAD + DMA + "\tv_mov_b64_e32 v[30:31], v[10:11]\n\ts_waitcnt vmcnt(1)\n")
    assert n == 1 and len(bad) == 1 and "touches" in bad[0]


def test_rejects_overwrite_and_range_overlap(tmp_path):
    _, bad = _check(tmp_path, LOAD + "\tv_mfma_f32_16x16x32_f16 v[8:11], v[40:43], v[44:47], v[8:11]\n\ts_waitcnt vmcnt(0)\n")
    assert len(bad) == 1


def test_wait_that_leaves_the_load_in_flight_does_not_count(tmp_path):
    # two younger loads, vmcnt(3): the hand-issued load may still be outstanding when v10 is read
    _, bad = _check(tmp_path, LOAD + DMA + DMA + "\ts_waitcnt vmcnt(3)\n\tv_mov_b32_e32 v4, v10\n\ts_waitcnt vmcnt(0)\n")
    assert len(bad) == 1


def test_follows_both_sides_of_a_branch_and_loops(tmp_path):
    ok = LOAD + DMA + "\ts_cbranch_scc1 .LBB0_2\n\tv_add_u32_e32 v1, v2, v3\n.LBB0_2:\n\ts_waitcnt vmcnt(1)\n\tv_mov_b32_e32 v4, v11\n"
    assert _check(tmp_path, ok)[1] == []
    bad_taken = LOAD + DMA + "\ts_cbranch_scc1 .LBB0_2\n\ts_waitcnt vmcnt(1)\n\ts_branch .LBB0_3\n.LBB0_2:\n\tv_mov_b32_e32 v4, v11\n.LBB0_3:\n\ts_waitcnt vmcnt(0)\n"
    assert len(_check(tmp_path, bad_taken)[1]) == 1
    # loop: request at the bottom, wait + use at the top of the next iteration
    loop = ".LBB0_1:\n\ts_waitcnt vmcnt(1)\n\tv_mov_b32_e32 v4, v10\n" + LOAD + DMA + "\ts_cbranch_scc1 .LBB0_1\n\ts_waitcnt vmcnt(0)\n"
    assert _check(tmp_path, loop)[1] == []


def test_rejects_spills_in_kernels_with_such_loads(tmp_path):
    p = os.path.join(tmp_path, "k.s")
    with open(p, "w") as f:
        f.write(HEAD + LOAD + "\ts_waitcnt vmcnt(0)\n\ts_endpgm\n"
                "amdhsa.kernels:\n  - .name:           kern\n    .private_segment_fixed_size: 64\n    .vgpr_spill_count: 3\n")
    n, bad = check_asm.check_file(p)
    assert n == 1 and len(bad) == 1 and "spilled" in bad[0]


def test_rejects_spills_in_any_kernel(tmp_path):
    p = os.path.join(tmp_path, "k.s")
    with open(p, "w") as f:
        f.write(HEAD + "\tv_mov_b32_e32 v4, v10\n\ts_endpgm\n"
                "amdhsa.kernels:\n  - .name:           kern\n    .private_segment_fixed_size: 472\n    .vgpr_spill_count: 0\n")
    n, bad = check_asm.check_file(p)
    assert n == 0 and len(bad) == 1 and "scratch" in bad[0]


WAIT = "\ts_waitcnt vmcnt(0)\n"


def test_rejects_base_read_too_soon_after_a_valu_write(tmp_path):
    # v_readfirstlane_b32 writes s3; the load that reads s[2:3] follows with two wait states in between
    body = "\tv_readfirstlane_b32 s3, v7\n\tv_add_u32_e32 v1, v2, v3\n\ts_mul_i32 s9, s8, s8\n" + LOAD + WAIT
    _, bad = _check(tmp_path, body)
    assert len(bad) == 1 and "wait states" in bad[0] and "s3" in bad[0]
    # a carry-out is a VALU write of scalar registers as well
    body = "\tv_mad_u64_u32 v[30:31], s[2:3], v5, s10, v[32:33]\n" + LOAD + WAIT
    assert len(_check(tmp_path, body)[1]) == 1
    # ... also across a branch
    body = "\tv_readfirstlane_b32 s2, v7\n\ts_cbranch_scc1 .LBB0_2\n\ts_nop 7\n.LBB0_2:\n" + LOAD + WAIT
    assert len(_check(tmp_path, body)[1]) == 1


def test_accepts_settled_base(tmp_path):
    body = "\tv_readfirstlane_b32 s2, v6\n\tv_readfirstlane_b32 s3, v7\n\t;;#ASMSTART\n\ts_nop 4 ; settled\n\t;;#ASMEND\n" + LOAD + WAIT
    assert _check(tmp_path, body)[1] == []
    # five ordinary instructions are five wait states
    body = "\tv_readfirstlane_b32 s3, v7\n" + "\tv_add_u32_e32 v1, v2, v3\n" * 5 + LOAD + WAIT
    assert _check(tmp_path, body)[1] == []
    # a scalar-ALU write replaces the VALU's value (interlocked), and a source operand is not a write
    body = "\tv_mad_u64_u32 v[30:31], s[2:3], v5, s10, v[32:33]\n\ts_add_u32 s2, s12, s14\n\ts_addc_u32 s3, s13, s15\n" + LOAD + WAIT
    assert _check(tmp_path, body)[1] == []
    body = "\tv_mul_f32_e32 v71, s2, v73\n" + LOAD + WAIT
    assert _check(tmp_path, body)[1] == []


def test_rejects_lds_load_right_after_the_write_to_m0(tmp_path):
    body = "\t;;#ASMSTART\n\ts_mov_b32 m0, s5\n\tglobal_load_lds_dwordx4 v21, s[6:7]\n\t;;#ASMEND\n" + WAIT
    _, bad = _check(tmp_path, body)
    assert len(bad) == 1 and "M0" in bad[0]
