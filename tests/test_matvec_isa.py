"""A property of the mat-vec kernels' compiled code that their source cannot express.

`csrc/matvec.hip` and `csrc/matvec_chain.hip` reload a slab's 32 activation registers with `ds_read_b32` instructions
written as `asm` statements and wait for them in a further `asm` statement.  The data of such a read lands in its register some
time after the instruction; until the wait, the register's contents are undefined, and the compiler does not know
that.  It is free to place its own instructions between the statements, and a copy or a reuse of one of those
registers there reads or overwrites a value that has not arrived.  This test compiles the kernels to assembly with the
library's flags and checks that no compiler-generated instruction names a register of those reads between the first
read of a reload and its wait (every template instantiation of both files)."""
import importlib.util
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "let-it-slide_amd")


def _flags():
    spec = importlib.util.spec_from_file_location("rptc_build", os.path.join(PKG, "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod.FLAGS


def _vregs(text):
    regs = set()
    for a, b in re.findall(r"\bv\[(\d+):(\d+)\]", text):
        regs.update(range(int(a), int(b) + 1))
    for a in re.findall(r"\bv(\d+)\b", text):
        regs.add(int(a))
    return regs


def reload_sites(lines):
    """Yields (first line, wait line, offending instructions) for every run of asm LDS reads up to the asm wait."""
    i = 0
    while i < len(lines):
        if "#ASMSTART" in lines[i] and i + 1 < len(lines) and lines[i + 1].strip().startswith("ds_read_b32"):
            j, in_asm, pending, hits = i, False, set(), []
            while j < len(lines):
                t = lines[j].strip()
                if "#ASMSTART" in t:
                    in_asm = True
                elif "#ASMEND" in t:
                    in_asm = False
                elif in_asm and t.startswith("s_waitcnt") and "lgkmcnt(0)" in t:
                    break
                elif in_asm and t.startswith("ds_read_b32"):
                    pending.add(int(re.match(r"ds_read_b32 v(\d+),", t).group(1)))
                elif not in_asm and t and not t.startswith((";", ".")):
                    if re.match(r"s_waitcnt.*lgkmcnt\(0\)", t):
                        pending.clear()                  # a wait of the compiler's own covers them as well
                    elif _vregs(t) & pending:
                        hits.append((j + 1, t))
                j += 1
            assert j < len(lines), f"asm LDS reads from line {i + 1} on have no wait"
            yield i + 1, j + 1, hits
            i = j
        i += 1


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
@pytest.mark.parametrize("source", ["matvec_chain.hip", "matvec.hip"])
def test_no_compiler_instruction_touches_a_register_with_an_lds_read_in_flight(tmp_path, source):
    out = tmp_path / (source + ".s")
    cmd = ["hipcc", *_flags(), "--cuda-device-only", "-S", os.path.join(PKG, "csrc", source), "-o", str(out)]
    subprocess.run(cmd, check=True, capture_output=True)
    sites = list(reload_sites(out.read_text().split("\n")))
    assert len(sites) >= 4, "the reload of the activation registers was not found in the assembly"
    bad = [(first, wait, hits[:3]) for first, wait, hits in sites if hits]
    assert not bad, f"registers with LDS reads in flight are touched before the wait: {bad[:2]}"


def test_the_checker_sees_a_copy_between_read_and_wait():
    text = """
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
	v_mov_b32_e32 v86, v51
"""
    sites = list(reload_sites(text.split("\n")))
    assert len(sites) == 1 and [t for _, t in sites[0][2]] == ["v_mov_b32_e32 v85, v50"]
