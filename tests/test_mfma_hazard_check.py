"""The build-time scanner for hand-written MFMAs (torchprime_amd/csrc/check_mfma_hazards.py) on small snippets of
gfx950 assembly: it must flag an operand written by a vector-ALU instruction right in front of an MFMA inside an
asm statement, and accept the same code once two wait states lie between them."""

import importlib.util
import os

_PATH = os.path.join(os.path.dirname(__file__), "..", "torchprime_amd", "csrc", "check_mfma_hazards.py")
_spec = importlib.util.spec_from_file_location("check_mfma_hazards", _PATH)
chk = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(chk)

KERNEL = "_ZN2tp6kernelEv: ; @_ZN2tp6kernelEv\n"


def _asm(body):
  return (KERNEL + body).splitlines(keepends=True)


def test_flags_operand_packed_right_before_the_mfma():
  found = chk.scan(_asm("""
	v_cvt_pk_bf16_f32 v8, v48, v49
	s_waitcnt lgkmcnt(0)
	;;#ASMSTART
	v_mfma_f32_32x32x16_bf16 a[112:127], v[12:15], v[8:11], a[112:127]
	;;#ASMEND
"""))
  assert len(found) == 1 and found[0][0] == "_ZN2tp6kernelEv" and "v_cvt_pk_bf16_f32 v8" in found[0][2]


def test_accepts_two_wait_states():
  for filler in ("\ts_nop 1\n", "\ts_nop 0\n\ts_waitcnt lgkmcnt(0)\n", "\tv_add_u32_e32 v40, 0, v41\n\tds_read_b128 v[20:23], v40\n"):
    found = chk.scan(_asm("\tv_cvt_pk_bf16_f32 v8, v48, v49\n" + filler +
                          "\t;;#ASMSTART\n\tv_mfma_f32_32x32x16_bf16 a[0:15], v[12:15], v[8:11], a[0:15]\n\t;;#ASMEND\n"))
    assert found == [], filler


def test_guard_inside_the_asm_statement_counts():
  found = chk.scan(_asm("""
	v_perm_b32 v13, v1, v2, v3
	;;#ASMSTART
	s_nop 1
	v_mfma_f32_32x32x16_f16 a[0:15], v[12:15], v[8:11], a[0:15]
	;;#ASMEND
"""))
  assert found == []


def test_compiler_emitted_mfma_and_unrelated_writes_are_ignored():
  found = chk.scan(_asm("""
	v_cvt_pk_bf16_f32 v8, v48, v49
	v_mfma_f32_32x32x16_bf16 v[16:31], v[12:15], v[8:11], v[16:31]
	v_cvt_pk_bf16_f32 v40, v48, v49
	;;#ASMSTART
	v_mfma_f32_32x32x16_bf16 a[0:15], v[12:15], v[8:11], a[0:15]
	;;#ASMEND
	ds_read_b128 v[12:15], v50
	s_waitcnt lgkmcnt(0)
	;;#ASMSTART
	v_mfma_f32_32x32x16_bf16 a[0:15], v[12:15], v[8:11], a[0:15]
	;;#ASMEND
"""))
  assert found == []


def test_main_exit_status(tmp_path, capsys):
  bad = tmp_path / "bad.s"
  bad.write_text(KERNEL + "\tv_mov_b32_e32 v9, v1\n\t;;#ASMSTART\n\tv_mfma_f32_32x32x16_bf16 a[0:15], v[12:15], v[8:11], a[0:15]\n\t;;#ASMEND\n")
  good = tmp_path / "good.s"
  good.write_text(KERNEL + "\ts_nop 3\n")
  assert chk.main([str(good)]) == 0
  assert chk.main([str(good), str(bad)]) == 1
  assert "less than 2 wait states" in capsys.readouterr().out


def test_flags_accumulator_copied_right_behind_the_mfma_that_writes_it():
  body = """
	;;#ASMSTART
	s_nop 1
	v_mfma_f32_32x32x16_bf16 a[48:63], v[2:5], v[14:17], a[48:63]
	;;#ASMEND
	v_accvgpr_mov_b32 a127, a63
"""
  found = chk.scan(_asm(body))
  assert len(found) == 1 and found[0][2].startswith("v_mfma") and "a127, a63" in found[0][3]
  # unrelated accumulation registers, and the same read behind enough wait states, are fine
  assert chk.scan(_asm(body.replace("a127, a63", "a127, a15"))) == []
  waited = body.replace("\tv_accvgpr_mov_b32", "\t;;#ASMSTART\n\ts_nop 15\n\ts_nop 3\n\t;;#ASMEND\n\tv_accvgpr_mov_b32")
  assert chk.scan(_asm(waited)) == []


def test_accumulating_into_the_same_registers_is_not_a_read_hazard():
  found = chk.scan(_asm("""
	;;#ASMSTART
	v_mfma_f32_32x32x16_bf16 a[0:15], v[2:5], v[14:17], a[0:15]
	;;#ASMEND
	ds_read_b128 v[2:5], v40
	s_waitcnt lgkmcnt(0)
	;;#ASMSTART
	v_mfma_f32_32x32x16_bf16 a[0:15], v[2:5], v[14:17], a[0:15]
	;;#ASMEND
"""))
  assert found == []
