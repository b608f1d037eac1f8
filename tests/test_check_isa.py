"""The build's check of asm-issued matrix-core instructions (co-rope_amd/check_isa.py), on small pieces of assembly."""
import importlib

check = importlib.import_module("co-rope_amd.check_isa").check_asm_mfma

ASM = "\t;;#ASMSTART\n\tv_mfma_f32_32x32x16_bf16 v[16:31], v[32:35], v[48:51], v[0:15]\n\t;;#ASMEND\n"
ACCUMULATE = "\tv_mfma_f32_32x32x16_bf16 v[16:31], v[36:39], v[52:55], v[16:31]\n"


def test_in_place_accumulate_is_accepted():
    assert check("kern:\n" + ASM + "\tds_read_b128 v[36:39], v40\n" + ACCUMULATE + "\tv_mov_b32 v63, v17\n") == []


def test_register_copy_right_behind_it_is_reported():
    # what a build with accumulators in the other half of the register file produced: the copy reads the old contents
    problems = check("kern:\n" + ASM + "\ts_nop 0\n\tv_accvgpr_write_b32 a0, v16\n" + ACCUMULATE)
    assert len(problems) == 1 and "kern" in problems[0] and "v_accvgpr_write_b32" in problems[0]


def test_overwrite_and_other_accumulator_are_reported():
    assert check("kern:\n" + ASM + "\tds_read_b128 v[28:31], v40\n" + ACCUMULATE)
    assert check("kern:\n" + ASM + "\tv_mfma_f32_32x32x16_bf16 v[64:79], v[36:39], v[52:55], v[16:31]\n")


def test_untouched_for_long_enough_is_accepted():
    assert check("kern:\n" + ASM + "\ts_nop 11\n\tv_mov_b32 v63, v17\n") == []
    assert check("kern:\n" + ASM + "\ts_nop 5\n\tv_mov_b32 v63, v17\n")


def test_both_sides_of_a_branch_are_followed():
    tail = "\ts_cbranch_scc1 .LBB0_1\n\tv_mov_b32 v61, v62\n.LBB0_1:                 ; %bb.1\n"
    assert check("kern:\n" + ASM + tail + ACCUMULATE) == []
    assert check("kern:\n" + ASM + tail + "\tv_mov_b32 v63, v17\n")
    # only the path that is not taken reads the result too early
    assert check("kern:\n" + ASM + "\ts_cbranch_scc1 .LBB0_1\n\tv_mov_b32 v63, v17\n.LBB0_1:\n" + ACCUMULATE)


def test_result_in_the_accumulation_half_and_operand_there_are_understood():
    asm = "\t;;#ASMSTART\n\tv_mfma_f32_32x32x16_bf16 v[16:31], v[32:35], a[48:51], v[16:31]\n\t;;#ASMEND\n"
    assert check("kern:\n" + asm + "\ts_nop 11\n\tv_exp_f32_e32 v3, v17\n") == []
    assert check("kern:\n" + asm + "\tv_exp_f32_e32 v3, v17\n")
    asm_a = "\t;;#ASMSTART\n\tv_mfma_f32_32x32x16_bf16 a[0:15], v[32:35], v[48:51], a[0:15]\n\t;;#ASMEND\n"
    assert check("kern:\n" + asm_a + "\tv_accvgpr_read_b32 v3, a4\n")
    assert check("kern:\n" + asm_a + "\tv_mov_b32 v4, v5\n" * 12 + "\tv_accvgpr_read_b32 v3, a4\n") == []


def test_addend_overwritten_while_it_may_still_be_read_is_reported():
    # the result lands beside the addend v[0:15]: a vector write to the addend right behind the instruction is too early
    assert check("kern:\n" + ASM + "\tv_mov_b32_e32 v3, v40\n" + ACCUMULATE)
    assert check("kern:\n" + ASM + "\tv_mov_b32_e32 v40, v41\n" * 8 + "\tv_mov_b32_e32 v3, v40\n") == []
    # reading the addend is fine
    assert check("kern:\n" + ASM + "\tv_mov_b32_e32 v40, v3\n" + ACCUMULATE) == []


def test_operand_written_right_in_front_is_reported():
    assert check("kern:\n\tv_cvt_pk_bf16_f32 v48, v60, v61\n" + ASM + ACCUMULATE)
    assert check("kern:\n\tv_cvt_pk_bf16_f32 v48, v60, v61\n\ts_nop 1\n" + ASM + ACCUMULATE) == []
    assert check("kern:\n\tds_read_b128 v[32:35], v40\n\ts_waitcnt lgkmcnt(0)\n" + ASM + ACCUMULATE) == []


def test_sources_with_asm_matrix_instructions_are_found():
    build = importlib.import_module("co-rope_amd.build")
    checked = {s for s in build.SOURCES if build.isa_checked(s)}
    assert {"rope_attn_fwd_pipe.hip", "rope_attn_fwd_pipe_acc.hip", "rope_attn_bwd.hip"} <= checked
    assert "rope_rotate.hip" not in checked and "abi.hip" not in checked
