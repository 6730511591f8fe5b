"""Build the CPU oracle (oracle/_build/librptc_oracle.so) with gcc.

The oracle is the checker used by tests/, the smoke check and the benchmark's
CPU-baseline leg.  The reference's own hot path is CUDA C++ with inline PTX
(rptc_kernels/csrc/rptc_kernels/inference.cu:1-6,254) and cannot be compiled
with the tools in this image, so no oracle/_ref build exists.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
OUT_DIR = os.path.join(HERE, "_build")
LIB = os.path.join(OUT_DIR, "librptc_oracle.so")


def build(verbose=False):
    os.makedirs(OUT_DIR, exist_ok=True)
    cmd = ["gcc", "-O3", "-march=x86-64-v2", "-ffp-contract=off", "-fopenmp", "-shared", "-fPIC", "-Wall", "-Wextra",
           "-o", LIB, os.path.join(HERE, "rptc_oracle.c"), "-lm"]
    if verbose:
        print(" ".join(cmd))
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
    sys.exit(0)
