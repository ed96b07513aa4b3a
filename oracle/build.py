"""Compile the C oracle (test infrastructure) into ``oracle/libpqhsa_oracle.so``.

The reference is pure Python, so there is no ``oracle/_ref`` build: nothing of the
reference compiles from C/C++ sources.
"""

from __future__ import annotations

import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "pqhsa_oracle.c")
LIB = os.path.join(HERE, "libpqhsa_oracle.so")


def build(force: bool = True) -> str:
    if not force and os.path.exists(LIB) and os.path.getmtime(LIB) >= os.path.getmtime(SRC):
        return LIB
    cmd = [
        "gcc", "-O2", "-std=c11", "-fPIC", "-shared", "-mfma", "-ffp-contract=off",
        "-fno-fast-math", "-Wall", "-Wextra", "-o", LIB, SRC, "-lm",
    ]
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    print(build())
