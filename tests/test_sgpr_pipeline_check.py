"""The build-time checker of the scalar-load weight pipeline (dabnn_amd/csrc/check_sgpr_pipeline.py): it must flag an
SGPR of an inline-asm scalar load that is read before the load's wait, and pass the pattern the kernels rely on."""
import importlib.util
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def load_checker():
    spec = importlib.util.spec_from_file_location("check_sgpr_pipeline", os.path.join(ROOT, "dabnn_amd", "csrc", "check_sgpr_pipeline.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


GOOD = """
_Z6kernelv:
	;;#ASMSTART
	s_load_dwordx16 s[12:27], s[34:35], 0x80
	;;#ASMEND
	;;#ASMSTART
	v_xor_b32 v54, s36, v26
	;;#ASMEND
	v_readlane_b32 s10, v57, 17
	;;#ASMSTART
	s_waitcnt lgkmcnt(0)
	;;#ASMEND
	;;#ASMSTART
	v_xor_b32 v54, s12, v26
	;;#ASMEND
	v_writelane_b32 v57, s12, 21
	s_endpgm
"""

# what a register allocator under pressure produced once: the vector is spilled to VGPR lanes right behind its load
BAD = """
_Z6kernelv:
	;;#ASMSTART
	s_load_dwordx16 s[12:27], s[34:35], 0x80
	;;#ASMEND
	v_readlane_b32 s11, v57, 18
	v_writelane_b32 v57, s12, 21
	s_and_b64 vcc, exec, s[10:11]
	v_writelane_b32 v57, s13, 22
	;;#ASMSTART
	s_waitcnt lgkmcnt(0)
	;;#ASMEND
	s_endpgm
"""


def test_checker_passes_the_pipeline_and_flags_a_spill_in_flight(tmp_path):
    chk = load_checker()
    good, bad = tmp_path / "good.s", tmp_path / "bad.s"
    good.write_text(GOOD)
    bad.write_text(BAD)
    assert chk.check(str(good)) == []
    problems = chk.check(str(bad))
    assert len(problems) == 2 and "v_writelane_b32" in problems[0] and "line 4" in problems[0]
    # a copy to another SGPR or a use as a 64-bit pair operand is caught too
    bad.write_text(BAD.replace("v_writelane_b32 v57, s13, 22", "s_and_b64 vcc, exec, s[26:27]"))
    assert any("s_and_b64" in p for p in chk.check(str(bad)))


def test_checker_wants_wait_states_behind_a_wide_store_in_inline_asm(tmp_path):
    """A store of more than 8 bytes inside an inline-asm statement must carry its own `s_nop 1`: the compiler's hazard
    handling does not see it, and the next vector instruction could overwrite the data it still reads."""
    chk = load_checker()
    good = tmp_path / "good.s"
    good.write_text("""
_Z6kernelv:
	;;#ASMSTART
	global_store_dwordx4 v[154:155], v[144:147], off sc1
	s_nop 1
	;;#ASMEND
	v_mov_b32 v144, 1
	;;#ASMSTART
	global_store_dwordx2 v[154:155], v[144:145], off sc1
	;;#ASMEND
	global_store_dwordx4 v[2:3], v[4:7], off nt
	s_endpgm
""")
    assert chk.check(str(good)) == []
    for body in ("global_store_dwordx4 v[154:155], v[144:147], off sc1\n",
                 "global_store_dwordx4 v[154:155], v[144:147], off sc1\n\ts_nop 0\n",
                 "global_store_dwordx3 v[154:155], v[144:146], off\n\tv_mov_b32 v144, 1\n"):
        bad = tmp_path / "bad.s"
        bad.write_text("_Z6kernelv:\n\t;;#ASMSTART\n\t" + body + "\t;;#ASMEND\n\tv_mov_b32 v144, 1\n\ts_endpgm\n")
        problems = chk.check(str(bad))
        assert len(problems) == 1 and "more than 8 bytes" in problems[0], (body, problems)
