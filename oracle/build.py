"""Build the CPU oracle (test infrastructure) into oracle/liborc.so with gcc.

No contraction and no fast-math: every rounding step in tf_oracle.c is written out, and the parity tests rely on it.
tf_oracle_simd.c (the vectorised projection loops the CPU baseline times) is built with the same flags; its AVX2 + FMA
functions carry their own target attribute and are only called where orc_simd_available() says the host has both.
"""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "liborc.so")
SOURCES = [os.path.join(HERE, "tf_oracle.c"), os.path.join(HERE, "tf_oracle_simd.c")]
FLAGS = ["-O2", "-fPIC", "-shared", "-std=c11", "-ffp-contract=off", "-fno-fast-math", "-fopenmp", "-Wall", "-Wextra"]


def build(force=True):
    newest = max(os.path.getmtime(p) for p in SOURCES + [os.path.join(HERE, "tf_oracle.h")])
    if not force and os.path.exists(LIB) and os.path.getmtime(LIB) >= newest:
        return LIB
    subprocess.run(["gcc", *FLAGS, *SOURCES, "-o", LIB, "-lm"], check=True)
    return LIB


if __name__ == "__main__":
    print(build())
