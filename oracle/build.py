"""Build the CPU oracle (test infrastructure) into oracle/libhs_oracle.so.

Usage: python oracle/build.py
Strict IEEE flags: no fast-math, no FMA contraction, so that the fp32
quantizer arithmetic is exactly the sequence of operations written in the C.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "hs_oracle.c")
OUT = os.path.join(HERE, "libhs_oracle.so")


def build(verbose: bool = False) -> str:
    cmd = ["gcc", "-O2", "-std=c11", "-fPIC", "-shared", "-fvisibility=hidden",
           "-ffp-contract=off", "-fno-fast-math", "-msse2", "-mfpmath=sse",
           "-Wall", "-Wextra", "-o", OUT, SRC, "-lm"]
    if verbose:
        print(" ".join(cmd))
    subprocess.check_call(cmd)
    return OUT


if __name__ == "__main__":
    print(build(verbose=True))
    sys.exit(0)
