"""Build the CPU oracle (test infrastructure) into oracle/libqlinear_oracle.so with gcc.

The reference's own implementation of this path is CUDA + CUTLASS behind a Windows/MSVC build script, so there is
nothing under the reference tree that gcc could compile: no oracle/_ref is produced.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "qlinear_oracle.c")
OUT = os.path.join(HERE, "libqlinear_oracle.so")


def build(force: bool = True) -> str:
    if not force and os.path.exists(OUT) and os.path.getmtime(OUT) >= os.path.getmtime(SRC):
        return OUT
    cmd = ["gcc", "-O3", "-march=x86-64-v3", "-fopenmp", "-ffp-contract=off", "-fno-fast-math", "-fvisibility=hidden",
           "-shared", "-fPIC", "-o", OUT, SRC, "-lm"]
    subprocess.check_call(cmd)
    return OUT


if __name__ == "__main__":
    print(build(force="--if-stale" not in sys.argv))
