"""The build-time check of the compiler's assembly (csrc/asm_lint.py) on small hand-written listings: each rule fires on
the pattern it exists for and stays quiet on the corrected one."""

import importlib.util
import os
import textwrap

HERE = os.path.dirname(os.path.abspath(__file__))
_spec = importlib.util.spec_from_file_location("asm_lint", os.path.join(os.path.dirname(HERE), "jax-flash-attn2_amd", "csrc", "asm_lint.py"))
L = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(L)

# (first two boolean template arguments 0, 0: the strict variants of rule R4)
KERNEL = "_ZN3fa210fwd_kernelINS_4BF16ELi128ELi8ELi1ELi1ELb0ELb0ELb0ELb0ELb0EEEvNS_5KArgsE"
KERNEL_DROP = "_ZN3fa210fwd_kernelINS_4BF16ELi128ELi8ELi1ELi1ELb0ELb1ELb0ELb0ELb0EEEvNS_5KArgsE"


def _write(tmp_path, body, kernel=KERNEL):
	p = tmp_path / "k.s"
	p.write_text(f"{kernel}:\n" + textwrap.dedent(body) + "\n.Lfunc_end0:\n")
	return str(p)


def test_r1_c_operand_overwritten_while_the_product_runs(tmp_path):
	bad = _write(tmp_path, """
		;;#ASMSTART
		v_mfma_f32_32x32x16_bf16 v[0:15], v[16:19], a[0:3], v[32:47]
		;;#ASMEND
		v_mov_b32_e32 v32, 0
	""")
	assert any("R1" in x for x in L.lint(bad))
	good = _write(tmp_path, """
		;;#ASMSTART
		v_mfma_f32_32x32x16_bf16 v[0:15], v[16:19], a[0:3], v[32:47]
		;;#ASMEND
		;;#ASMSTART
		v_mfma_f32_32x32x16_bf16 v[48:63], v[16:19], a[0:3], v[48:63]
		;;#ASMEND
		v_mov_b32_e32 v32, 0
	""")
	assert not L.lint(good)


def test_r2_result_read_too_early(tmp_path):
	bad = _write(tmp_path, """
		;;#ASMSTART
		v_mfma_f32_32x32x16_bf16 v[0:15], v[16:19], a[0:3], v[0:15]
		;;#ASMEND
		v_mul_f32_e32 v20, v0, v1
	""")
	assert any("R2" in x for x in L.lint(bad))
	good = _write(tmp_path, """
		;;#ASMSTART
		v_mfma_f32_32x32x16_bf16 v[0:15], v[16:19], a[0:3], v[0:15]
		;;#ASMEND
		s_nop 15
		v_mul_f32_e32 v20, v0, v1
	""")
	assert not L.lint(good)


LOOP_WAIT = """
	.LBB0_1:                                ; =>This Loop Header: Depth=1
	s_nop 0
	.LBB0_2:                                ;   Parent Loop BB0_1 Depth=2
	ds_read_b128 v[4:7], v100
	s_waitcnt vmcnt(0)
	v_mfma_f32_32x32x16_bf16 v[0:15], v[4:7], v[16:19], v[0:15]
	s_cbranch_scc1 .LBB0_2
"""
LOOP_SPILL = """
	.LBB0_2:                                ;   Parent Loop BB0_1 Depth=2
	scratch_load_dword v9, off, off offset:4
	v_mfma_f32_32x32x16_bf16 v[0:15], v[4:7], v[16:19], v[0:15]
	s_cbranch_scc1 .LBB0_2
"""
LOOP_CLEAN = """
	s_waitcnt vmcnt(0)
	.LBB0_2:                                ;   Parent Loop BB0_1 Depth=2
	ds_read_b128 v[4:7], v100
	s_waitcnt lgkmcnt(0)
	v_mfma_f32_32x32x16_bf16 v[0:15], v[4:7], v[16:19], v[0:15]
	s_waitcnt vmcnt(0)
	s_barrier
	s_cbranch_scc1 .LBB0_2
"""
LOOP_BIAS_BY_VALUE = """
	.LBB0_2:                                ;   Parent Loop BB0_1 Depth=2
	global_load_ushort v9, v[10:11], off
	s_waitcnt vmcnt(0)
	v_mfma_f32_32x32x16_bf16 v[0:15], v[4:7], v[16:19], v[0:15]
	s_cbranch_scc1 .LBB0_2
"""


def test_r4_waits_and_spills_inside_tile_loops(tmp_path):
	for body in (LOOP_WAIT, LOOP_SPILL):
		problems, notes = L.lint_loops(_write(tmp_path, body))
		assert len(problems) == 1 and "R4" in problems[0] and not notes
		# the variants with bias or dropout: a note, not a failure
		problems, notes = L.lint_loops(_write(tmp_path, body, KERNEL_DROP))
		assert not problems and len(notes) == 1
	# a wait after the last product of the block (the end of a step), or outside the loop, is fine
	assert L.lint_loops(_write(tmp_path, LOOP_CLEAN)) == ([], [])
	# loops that load values from global memory into registers have waits of their own
	assert L.lint_loops(_write(tmp_path, LOOP_BIAS_BY_VALUE)) == ([], [])
