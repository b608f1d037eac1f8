"""The build's check of asm-issued matrix-core instructions (co-rope_amd/check_isa.py), on small pieces of assembly."""
import importlib

check = importlib.import_module("co-rope_amd.check_isa").check_asm_mfma

ASM = "\t;;#ASMSTART\n\tv_mfma_f32_32x32x16_bf16 v[16:31], v[32:35], v[48:51], v[0:15]\n\t;;#ASMEND\n"
ACCUMULATE = "\tv_mfma_f32_32x32x16_bf16 v[16:31], v[36:39], v[52:55], v[16:31]\n"


def test_in_place_accumulate_is_accepted():
    assert check("kern:\n" + ASM + "\tds_read_b128 v[36:39], v40\n" + ACCUMULATE + "\tv_mov_b32 v3, v17\n") == []


def test_register_copy_right_behind_it_is_reported():
    # what a build with accumulators in the other half of the register file produced: the copy reads the old contents
    problems = check("kern:\n" + ASM + "\ts_nop 0\n\tv_accvgpr_write_b32 a0, v16\n" + ACCUMULATE)
    assert len(problems) == 1 and "kern" in problems[0] and "v_accvgpr_write_b32" in problems[0]


def test_overwrite_and_other_accumulator_are_reported():
    assert check("kern:\n" + ASM + "\tds_read_b128 v[28:31], v40\n" + ACCUMULATE)
    assert check("kern:\n" + ASM + "\tv_mfma_f32_32x32x16_bf16 v[64:79], v[36:39], v[52:55], v[16:31]\n")


def test_untouched_for_long_enough_is_accepted():
    assert check("kern:\n" + ASM + "\ts_nop 11\n\tv_mov_b32 v3, v17\n") == []
    assert check("kern:\n" + ASM + "\ts_nop 5\n\tv_mov_b32 v3, v17\n")


def test_both_sides_of_a_branch_are_followed():
    tail = "\ts_cbranch_scc1 .LBB0_1\n\tv_mov_b32 v1, v2\n.LBB0_1:                 ; %bb.1\n"
    assert check("kern:\n" + ASM + tail + ACCUMULATE) == []
    assert check("kern:\n" + ASM + tail + "\tv_mov_b32 v3, v17\n")
    # only the path that is not taken reads the result too early
    assert check("kern:\n" + ASM + "\ts_cbranch_scc1 .LBB0_1\n\tv_mov_b32 v3, v17\n.LBB0_1:\n" + ACCUMULATE)
