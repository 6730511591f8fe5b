"""Build librptc_hip.so (the C-ABI library of gfx950 kernels) in-tree with hipcc."""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "librptc_hip.so")

FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-shared", "-fPIC",
    # hipcc must not form packed-fp32 instructions on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # kernel arguments arrive in SGPRs at wave start instead of through a scalar load
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
    "-Wall", "-Wno-unused-function",
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def build(verbose=False, extra=()):
    cmd = ["hipcc", *FLAGS, *extra, "-o", LIB, *sources()]
    if verbose:
        print(" ".join(cmd))
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True, extra=sys.argv[1:]))
