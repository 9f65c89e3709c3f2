"""Build the oracle's C twin (oracle/libuv_oracle.so) with gcc.  The reference is pure Python (its only native code is
a CUDA source string compiled at run time by NVRTC), so there is no oracle/_ref build: nothing in the reference
compiles with gcc/g++ here.

    python -m oracle.build
"""
from __future__ import annotations

import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "uv_oracle.c")
LIB = os.path.join(HERE, "libuv_oracle.so")


def build(force: bool = False) -> str:
    if force or not os.path.exists(LIB) or os.path.getmtime(LIB) < os.path.getmtime(SRC):
        # no -ffast-math: the quantizer relies on IEEE division and round-half-even
        subprocess.run(["gcc", "-O2", "-fPIC", "-shared", "-std=c11", "-fno-fast-math", "-ffp-contract=off",
                        "-o", LIB, SRC, "-lm"], check=True)
    return LIB


if __name__ == "__main__":
    print(build(force=True))
