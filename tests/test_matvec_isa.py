"""A property of the kernels' compiled code that their source cannot express.

The mat-vec kernels issue LDS reads (and, in the chain's loop, global loads) from inline assembly.  The data of such a
request lands in its register some time after the instruction; until the wait, the register's contents are undefined,
and the compiler does not know that: between two `asm` statements it is free to copy or reuse the register.  So every
block of inline assembly must wait for what it requested before it ends.  `build.py` checks that on the assembly it
emits for every source with hand-written blocks (a build that breaks the rule fails); this test runs the same check
and shows that the checker sees a violation."""
import importlib.util
import os
import shutil

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "let-it-slide_amd")


def _build_module():
    spec = importlib.util.spec_from_file_location("rptc_build", os.path.join(PKG, "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
@pytest.mark.parametrize("source", ["matvec.hip", "matmul.hip"])
def test_every_asm_block_waits_for_its_requests(source):
    _build_module().check_assembly(os.path.join(PKG, "csrc", source))


def test_the_checker_sees_a_block_that_ends_with_reads_in_flight():
    check = _build_module().asm_blocks_left_waiting
    bad = """
	;;#ASMSTART
	ds_read_b32 v50, v14 offset:0
	;;#ASMEND
	;;#ASMSTART
	ds_read_b32 v51, v14 offset:128
	;;#ASMEND
	v_mov_b32_e32 v85, v50
	;;#ASMSTART
	s_waitcnt lgkmcnt(0)
	;;#ASMEND
"""
    assert [t for _, t in check(bad)] == ["ds_read_b32 v50, v14 offset:0", "ds_read_b32 v51, v14 offset:128"]
    good = """
	;;#ASMSTART
	ds_read_b32 v50, v14 offset:0
	ds_read_b32 v51, v14 offset:128
	global_load_dwordx4 v[4:7], v3, s[2:3]
	s_waitcnt lgkmcnt(1)
	v_mov_b32 v2, v50
	s_waitcnt vmcnt(0) lgkmcnt(0)
	;;#ASMEND
"""
    assert check(good) == []
    partial = """
	;;#ASMSTART
	ds_read_b32 v50, v14 offset:0
	ds_read_b32 v51, v14 offset:128
	s_waitcnt lgkmcnt(1)
	;;#ASMEND
"""
    assert [t for _, t in check(partial)] == ["ds_read_b32 v51, v14 offset:128"]


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
@pytest.mark.parametrize("source", ["matvec_t.hip", "decode_glue.hip"])
def test_handoffs_between_workgroups_are_what_the_source_says(source):
    """Partial results that one workgroup writes and another adds up (csrc/rptc_common.hpp: publishing / published /
    arrive / merging / merged): sc1 stores, the wait, a barrier in front of the arrival's atomic, sc1 loads."""
    _build_module().check_assembly(os.path.join(PKG, "csrc", source))


def test_the_handoff_checker_sees_a_plain_store_a_plain_load_and_a_missing_barrier():
    check = _build_module().handoff_violations
    good = """
	; rptc-handoff: publishing
	global_store_dword v2, v4, s[6:7] sc1
	; rptc-handoff: published
	s_waitcnt vmcnt(0)
	s_barrier
	global_atomic_add v1, v1, v3, s[6:7] sc0
	; rptc-handoff: merging
	global_load_dword v2, v[6:7], off sc1
	; rptc-handoff: merged
	global_load_dword v9, v[6:7], off
"""
    assert check(good) == []
    assert [w for _, _, w in check(good.replace("v4, s[6:7] sc1", "v4, s[6:7]"))] == ["a store of a publishing region without sc1"]
    assert [w for _, _, w in check(good.replace("off sc1", "off"))] == ["a load of a merging region without sc1"]
    assert [w for _, _, w in check(good.replace("\ts_barrier\n", ""))] == ["the arrival is counted without a barrier behind published()"]
    assert [w for _, _, w in check(good.replace("\ts_waitcnt vmcnt(0)\n", ""))] == ["no s_waitcnt vmcnt(0) behind published()"]


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
@pytest.mark.parametrize("source,switch", [("matvec.hip", "-DRPTC_MV_ONE"), ("matmul.hip", "-DRPTC_MM_ROWS"), ("matvec_steady.hip", "-DST_TUNED"),
                                           ("matvec_steady.hip", "-DST_MFMA"), ("matvec_steady.hip", "-DST_ROLL")])
def test_host_code_behind_the_build_switches_still_compiles(source, switch):
    """The untimed variants are off in the library's build; their host-side routing must not rot meanwhile (the device code
    of each is compiled and run by the wave-model tests)."""
    import subprocess
    r = subprocess.run(["hipcc", "-std=c++17", "--offload-arch=gfx950", "--cuda-host-only", "-fsyntax-only", "-Wall", "-Wno-unused-function",
                        switch, os.path.join(PKG, "csrc", source)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
