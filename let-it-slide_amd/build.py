"""Build the gfx950 libraries in-tree with hipcc.

librptc_hip.so        the C-ABI library of kernels (include/rptc_hip.h), from csrc/*.hip
librptc_bench_aids.so two measurement aids bench.py times beside the mat-vec (an empty launch, a
                      kernel that only reads); kept out of the product library and its header
"""
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "librptc_hip.so")
AIDS_LIB = os.path.join(HERE, "librptc_bench_aids.so")

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


def build(verbose=False, extra=()):
    """Compiles every source (one hipcc per file, in parallel) and links the two libraries."""
    os.makedirs(OBJ, exist_ok=True)
    srcs = sources()
    objs = [os.path.join(OBJ, os.path.basename(s)[:-4] + ".o") for s in srcs]
    jobs = min(len(srcs), max(1, min(8, os.cpu_count() or 1)))
    with ThreadPoolExecutor(jobs) as pool:
        list(pool.map(lambda so: _run(["hipcc", *FLAGS, *extra, "-c", so[0], "-o", so[1]], verbose), zip(srcs, objs)))
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs], verbose)
    _run(["hipcc", *FLAGS, *extra, "-shared", "-o", AIDS_LIB, os.path.join(HERE, "bench_aids", "probe.hip")], verbose)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True, extra=sys.argv[1:]))
