"""Build the gfx950 libraries in-tree with hipcc.

librptc_hip.so        the C-ABI library of kernels (include/rptc_hip.h), from csrc/*.hip
../bench_aids/librptc_bench_aids.so
                      measurement aids bench.py times beside the mat-vec (an empty launch, kernels that only read,
                      instruction issue rates); beside bench.py, out of the product library, its header and its folder
"""
import glob
import os
import re
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "librptc_hip.so")
AIDS_DIR = os.path.join(os.path.dirname(HERE), "bench_aids")
AIDS_LIB = os.path.join(AIDS_DIR, "librptc_bench_aids.so")

FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC",
    # hipcc must not form packed-fp32 instructions on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # kernel arguments arrive in SGPRs at wave start instead of through a scalar load
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
    "-Wall", "-Wno-unused-function",
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)


def asm_blocks_left_waiting(assembly):
    """The rule the hand-written blocks follow, checked on the assembly the compiler emits: a block of inline assembly
    that issues LDS reads or global loads waits for them before it ends.  The data of such a request lands in its
    register some time after the instruction; the compiler does not know that, and between two `asm` statements it is
    free to copy or reuse that register, so a request and its wait must never sit in different statements.
    Returns [(line number, instruction)] for every request that its own block does not wait for (empty = good)."""
    bad = []
    lgkm, vm, in_asm = [], [], False
    for no, line in enumerate(assembly.split("\n"), 1):
        t = line.strip()
        if "#ASMSTART" in t:
            in_asm, lgkm, vm = True, [], []
        elif "#ASMEND" in t:
            bad += lgkm + vm
            in_asm = False
        elif in_asm:
            if re.match(r"ds_(read|bpermute|permute)", t):
                lgkm.append((no, t))
            elif re.match(r"(global|buffer|flat)_load", t):
                vm.append((no, t))
            elif t.startswith("s_waitcnt"):
                k = re.search(r"lgkmcnt\((\d+)\)", t)
                if k:
                    lgkm = lgkm[len(lgkm) - int(k.group(1)):] if int(k.group(1)) else []
                v = re.search(r"vmcnt\((\d+)\)", t)
                if v:
                    vm = vm[len(vm) - int(v.group(1)):] if int(v.group(1)) else []
    return bad


def handoff_violations(assembly):
    """The hand-off of partial results between workgroups (`publishing()` .. `published()`, `arrive()`, `merging()` ..
    `merged()` in csrc/rptc_common.hpp) replaces release / acquire fences by three properties of the emitted code, checked
    here on the markers those functions leave in the assembly: every global store of a publishing region and every global
    load of a merging region is an sc1 one (written through to / read from the level all XCDs share); `published()`'s
    `s_waitcnt vmcnt(0)` is there; and a workgroup barrier stands between it and the arrival's atomic add.
    Returns [(line number, text, what is wrong)] (empty = good)."""
    bad = []
    state = None                  # None, "publishing", "waiting" (published, barrier not yet seen), "merging"
    lines = assembly.split("\n")
    for no, line in enumerate(lines, 1):
        t = line.strip()
        if t.startswith("; rptc-handoff: publishing"):
            state = "publishing"
        elif t.startswith("; rptc-handoff: published"):
            nxt = next((x.strip() for x in lines[no:no + 3] if x.strip() and not x.strip().startswith(";")), "")
            if not (nxt.startswith("s_waitcnt") and "vmcnt(0)" in nxt):
                bad.append((no, t, "no s_waitcnt vmcnt(0) behind published()"))
            state = "waiting"
        elif t.startswith("; rptc-handoff: merging"):
            state = "merging"
        elif t.startswith("; rptc-handoff: merged"):
            state = None
        elif t.startswith(".Lfunc_end"):
            state = None
        elif state == "publishing" and re.match(r"(global|flat|buffer)_store", t) and " sc1" not in t:
            bad.append((no, t, "a store of a publishing region without sc1"))
        elif state == "merging" and re.match(r"(global|flat|buffer)_load", t) and " sc1" not in t:
            bad.append((no, t, "a load of a merging region without sc1"))
        elif state == "waiting":
            if t.startswith("s_barrier"):
                state = None
            elif re.match(r"(global|flat|buffer)_atomic", t):
                bad.append((no, t, "the arrival is counted without a barrier behind published()"))
                state = None
    return bad


def check_assembly(src, verbose=False, extra=()):
    """Compiles `src` to assembly with the library's flags and applies `asm_blocks_left_waiting` and
    `handoff_violations`; raises on a hit."""
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, os.path.basename(src) + ".s")
        _run(["hipcc", *FLAGS, *extra, "--cuda-device-only", "-S", src, "-o", out], verbose)
        text = open(out).read()
    bad = asm_blocks_left_waiting(text)
    if bad:
        raise RuntimeError(f"{os.path.basename(src)}: an inline-assembly block ends with requests in flight: {bad[:3]}")
    bad = handoff_violations(text)
    if bad:
        raise RuntimeError(f"{os.path.basename(src)}: the hand-off between workgroups is not what rptc_common.hpp says: {bad[:3]}")
    if "arrive(" in open(src).read() and "rptc-handoff: published" not in text:
        raise RuntimeError(f"{os.path.basename(src)}: arrive() without the markers of a hand-off in the assembly")


def build(verbose=False, extra=()):
    """Compiles every source (one hipcc per file, in parallel), checks the emitted assembly of the sources that hold
    hand-written request/wait sequences, and links the two libraries."""
    os.makedirs(OBJ, exist_ok=True)
    srcs = sources()
    objs = [os.path.join(OBJ, os.path.basename(s)[:-4] + ".o") for s in srcs]
    jobs = min(len(srcs), max(1, min(8, os.cpu_count() or 1)))
    with ThreadPoolExecutor(jobs) as pool:
        list(pool.map(lambda so: _run(["hipcc", *FLAGS, *extra, "-c", so[0], "-o", so[1]], verbose), zip(srcs, objs)))
        with_asm = [s for s in srcs if re.search(r"\basm\b", open(s).read()) or "decode_asm.hpp" in open(s).read()]
        list(pool.map(lambda s: check_assembly(s, verbose, extra), with_asm))
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs], verbose)
    _run(["hipcc", *FLAGS, *extra, "-shared", "-o", AIDS_LIB, os.path.join(AIDS_DIR, "probe.hip")], verbose)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True, extra=sys.argv[1:]))
