"""The build's guard for kernels that keep state in accumulation registers behind the compiler's back
(hipml_amd/build.py: scan_hand_placed_acc), on canned assembly text: it must accept a kernel whose only uses
of those registers sit inside inline-assembly statements and refuse one where the compiler has placed a use
of its own, a text without the kernel, and a text in which it finds no such register at all."""
import pytest

from hipml_amd.build import scan_hand_placed_acc

GOOD = """
	.globl	_ZN5hipml9other_oneEv
_ZN5hipml9other_oneEv:
	v_accvgpr_write_b32 a0, v1
	s_endpgm
.Lfunc_end0:
_ZN5hipml20chunk_f16_t64_kernelENS_9ChunkArgsE:
	s_load_dwordx2 s[0:1], s[4:5], 0x0
	v_mov_b32_e32 v1, 0
	;;#ASMSTART
	v_accvgpr_write_b32 a[0], 0
	v_accvgpr_write_b32 a[1], 0
	;;#ASMEND
	v_add_f32_e32 v2, v1, v1 ; a comment that mentions a[3] is no use of it
	;;#ASMSTART
	v_mfma_f32_32x32x16_f16 a[16:31], v[2:5], v[6:9], a[16:31]
	;;#ASMEND
	s_endpgm
.Lfunc_end1:
_ZN5hipml10after_thatEv:
	v_accvgpr_read_b32 v0, a7
	s_endpgm
.Lfunc_end2:
""".split("\n")


def test_a_kernel_whose_accumulation_registers_stay_inside_its_statements_passes():
    assert scan_hand_placed_acc(GOOD, "canned.hip", "chunk_f16_t64_kernel") == 3


@pytest.mark.parametrize("stray", ["	v_accvgpr_write_b32 a4, v17", "	v_accvgpr_read_b32 v200, a[5]",
                                   "	v_mfma_f32_32x32x16_f16 a[0:15], v[2:5], v[6:9], a[0:15]",
                                   "	v_accvgpr_mov_b32 a9, a10"])
def test_a_use_the_compiler_placed_itself_is_refused(stray):
    text = list(GOOD)
    text.insert(text.index("	v_add_f32_e32 v2, v1, v1 ; a comment that mentions a[3] is no use of it"), stray)
    with pytest.raises(RuntimeError, match="accumulation registers of its own"):
        scan_hand_placed_acc(text, "canned.hip", "chunk_f16_t64_kernel")


def test_a_missing_kernel_and_a_text_without_such_registers_are_refused():
    with pytest.raises(RuntimeError, match="not found"):
        scan_hand_placed_acc(GOOD, "canned.hip", "no_such_kernel")
    bare = [l for l in GOOD if "a[" not in l.split(";")[0] or "hipml" in l]
    with pytest.raises(RuntimeError, match="wrong text"):
        scan_hand_placed_acc(bare, "canned.hip", "chunk_f16_t64_kernel")
