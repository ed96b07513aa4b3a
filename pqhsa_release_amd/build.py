"""Compile the HIP kernels and the C ABI into ``pqhsa_release_amd/lib/libpqhsa.so`` (gfx950)."""

from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libpqhsa.so")
SOURCES = ["api.hip", "lut_build.hip", "scan_select.hip", "attend.hip", "encode.hip", "decode.hip"]

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # fixed-order fp32 parity with the CPU oracle: no implicit contraction, IEEE sqrt/div
    "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    # packed fp32 VALU forms stay off
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def build(verbose: bool = False, extra: list[str] | None = None, out: str | None = None) -> str:
    """Compile the library; ``extra`` adds compiler flags and ``out`` names another output file
    (a tuning build next to the shipped one, loaded through the PQHSA_LIBRARY variable)."""
    os.makedirs(LIBDIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    out = out or LIB
    cmd = [hipcc, *FLAGS, *(extra or []), *[os.path.join(CSRC, s) for s in SOURCES], "-o", out]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return out


if __name__ == "__main__":
    print(build(verbose=True, extra=sys.argv[1:]))
