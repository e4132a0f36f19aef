"""The lint that checks the idle issue slots around inline-asm matrix instructions
(``jvp_flash_attention_amd/asm_lint.py``): it must flag the two patterns on hand-written ISA text and
find none in freshly compiled kernels."""
from jvp_flash_attention_amd import asm_lint

PARKED_OPERAND = """
_ZN5jvpfa4kernEv:
	v_accvgpr_read_b32 v19, a61
	;;#ASMSTART
	v_mfma_f32_32x32x16_bf16 v[32:47], v[64:67], v[16:19], v[32:47]
	;;#ASMEND
	s_nop 15
	s_nop 3
	v_mul_f32_e32 v1, v32, v2
"""

EARLY_READ = """
_ZN5jvpfa4kernEv:
	;;#ASMSTART
	v_mfma_f32_32x32x16_bf16 v[32:47], v[64:67], a[16:19], 0
	;;#ASMEND
	v_accvgpr_write_b32 a70, v33
	s_nop 15
	s_nop 3
"""


def test_a_parked_operand_restored_right_before_its_matrix_instruction_is_flagged():
    found = asm_lint.scan(PARKED_OPERAND, "unit")
    assert len(found) == 1 and "without idle slots" in found[0]
    guarded = PARKED_OPERAND.replace("\tv_mfma", "\ts_nop 1\n\tv_mfma")
    assert asm_lint.scan(guarded, "unit") == []


def test_a_resident_operand_rewritten_right_before_its_matrix_instruction_is_flagged():
    text = PARKED_OPERAND.replace("v_accvgpr_read_b32 v19, a61", "v_accvgpr_write_b32 a18, v7").replace("v[16:19]", "a[16:19]")
    found = asm_lint.scan(text, "unit")
    assert len(found) == 1 and "without idle slots" in found[0]


def test_a_result_read_before_the_wait_is_flagged():
    found = asm_lint.scan(EARLY_READ, "unit")
    assert len(found) == 1 and "before the wait" in found[0]
    assert asm_lint.scan(EARLY_READ.replace("\tv_accvgpr_write_b32 a70, v33\n", ""), "unit") == []


EARLY_ACCUMULATOR_READ = """
_ZN5jvpfa4kernEv:
	;;#ASMSTART
	v_mfma_f32_32x32x16_bf16 a[0:15], v[64:67], v[16:19], a[0:15]
	;;#ASMEND
	v_accvgpr_read_b32 v5, a3
	;;#ASMSTART
	s_nop 15
	s_nop 15
	;;#ASMEND
"""


def test_an_accumulator_read_back_before_the_wait_is_flagged():
    """What the compiler may do to an epilogue behind a wait that is not tied to the accumulators."""
    found = asm_lint.scan(EARLY_ACCUMULATOR_READ, "unit")
    assert len(found) == 1 and "before the wait" in found[0]
    lines = EARLY_ACCUMULATOR_READ.split("\n")
    moved = "\n".join(lines[:5] + lines[6:] + [lines[5]])  # the read behind the wait
    assert asm_lint.scan(moved, "unit") == []


def test_compiled_kernels_are_clean():
    """The ISA text that the build left behind for every kernel unit, or, without a build, two units
    compiled here (the D = 32 backward is where the allocator once parked a resident operand in the
    accumulation file and restored it in front of its matrix instruction)."""
    import os

    from jvp_flash_attention_amd import build

    names = [u[0] for u in build.units() if u[0].startswith(("fwd_", "bwd_"))]
    if all(os.path.exists(build.isa_path(n)) for n in names):
        for n in names:
            with open(build.isa_path(n)) as f:
                assert asm_lint.scan(f.read(), n) == []
    else:
        assert asm_lint.lint(["bwd_bf16_32", "fwd_bf16_64"]) == []


COPY_BEFORE_ARRIVAL = """
_ZN5jvpfa4kernEv:
	;;#ASMSTART
	ds_read_b64_tr_b16 v[64:65], v109 offset:4096
	;;#ASMEND
	;;#ASMSTART
	ds_read_b64_tr_b16 v[66:67], v110 offset:4096
	;;#ASMEND
	v_mov_b64_e32 v[104:105], v[66:67]
	;;#ASMSTART
	s_waitcnt lgkmcnt(0)
	;;#ASMEND
	v_mov_b64_e32 v[102:103], v[64:65]
"""


def test_a_copy_of_an_lds_fragment_made_before_it_has_arrived_is_flagged():
    found = asm_lint.scan(COPY_BEFORE_ARRIVAL, "unit")
    assert len(found) == 1 and "still in flight" in found[0] and "v[104:105]" in found[0]
    # a wait that leaves only the younger read in flight frees the older destination
    partly = COPY_BEFORE_ARRIVAL.replace("\tv_mov_b64_e32 v[104:105], v[66:67]\n",
                                         "\t;;#ASMSTART\n\ts_waitcnt lgkmcnt(1)\n\t;;#ASMEND\n\tv_mov_b64_e32 v[100:101], v[64:65]\n")
    assert asm_lint.scan(partly, "unit") == []
    assert len(asm_lint.scan(partly.replace("v[100:101], v[64:65]", "v[100:101], v[66:67]"), "unit")) == 1


TWO_YOUNGER = """
_ZN5jvpfa4kernEv:
	;;#ASMSTART
	v_mfma_f32_32x32x16_bf16 v[32:47], v[64:67], a[16:19], 0
	;;#ASMEND
	;;#ASMSTART
	v_mfma_f32_32x32x16_bf16 v[48:63], v[64:67], a[20:23], 0
	;;#ASMEND
	;;#ASMSTART
	global_atomic_add_f32 v1, v33, s[0:1] offset:512
	;;#ASMEND
	;;#ASMSTART
	v_mfma_f32_32x32x16_bf16 v[80:95], v[64:67], a[24:27], 0
	;;#ASMEND
	;;#ASMSTART
	global_atomic_add_f32 v1, v34, s[0:1] offset:1024
	;;#ASMEND
	s_nop 15
	s_nop 3
"""


def test_a_result_counts_as_written_behind_two_younger_matrix_instructions():
    """The matrix pipe takes 32x32 instructions one after another, so the second one behind a producer cannot
    start before the producer is through: a reader behind it is fine, one behind a single younger one is not."""
    found = asm_lint.scan(TWO_YOUNGER, "unit")
    assert len(found) == 1 and "before the wait" in found[0] and "v33" in found[0]


IN_PLACE_MOVE = """
_ZN5jvpfa4kernEv:
	v_accvgpr_write_b32 a0, 0
	v_accvgpr_mov_b32 a1, a0
	s_nop 1
	;;#ASMSTART
	v_mfma_f32_32x32x16_bf16 a[0:15], v[64:67], v[16:19], a[0:15]
	;;#ASMEND
	;;#ASMSTART
	v_mfma_f32_32x32x16_bf16 a[16:31], v[64:67], v[20:23], a[16:31]
	;;#ASMEND
	;;#ASMSTART
	s_nop 15
	s_nop 15
	;;#ASMEND
""" + "".join(f"""	;;#ASMSTART
	v_accvgpr_read_b32 v1, a{16 + e}
	v_accvgpr_read_b32 v2, a{e}
	v_fma_f32 v1, v2, v4, v1
	v_mul_f32 v2, v2, v3
	v_mul_f32 v1, v1, v3
	s_nop 1
	v_accvgpr_write_b32 a{e}, v2
	v_accvgpr_write_b32 a{16 + e}, v1
	s_nop 1
	;;#ASMEND
""" for e in range(16))


def test_in_place_accumulator_moves_must_meet_the_registers_the_matrix_instructions_accumulate_into():
    """acc_move_in_place names the accumulator elements as inputs and writes them: sound only on the very
    registers mfma_acc accumulates into, and only if the compiler holds no copy of them."""
    assert asm_lint.scan(IN_PLACE_MOVE, "unit") == []
    # the statement was handed a copy of one element (a40 instead of a3)
    other = IN_PLACE_MOVE.replace("v_accvgpr_read_b32 v2, a3\n", "v_accvgpr_read_b32 v2, a40\n").replace(
        "v_accvgpr_write_b32 a3, v2", "v_accvgpr_write_b32 a40, v2")
    found = asm_lint.scan(other, "unit")
    assert len(found) == 1 and "in-place accumulator moves" in found[0] and "[40]" in found[0] and "[3]" in found[0]
    # the compiler keeps a second home for an element behind the first accumulation
    copied = IN_PLACE_MOVE + "\tv_accvgpr_mov_b32 a100, a5\n"
    found = asm_lint.scan(copied, "unit")
    assert len(found) == 1 and "copies an accumulator" in found[0]
