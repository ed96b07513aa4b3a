"""Compile the HIP kernels and the C ABI into ``pqhsa_release_amd/lib/libpqhsa.so`` (gfx950)."""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libpqhsa.so")
SOURCES = ["api.hip", "lut_build.hip", "scan_select.hip", "scan_emit.hip", "scan_stats.hip", "attend.hip", "encode.hip", "encode_prefilter.hip", "nearest.hip", "decode.hip", "probe.hip", "fused.hip"]

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # fixed-order fp32 parity with the CPU oracle: no implicit contraction, IEEE sqrt/div
    "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    # packed fp32 VALU forms stay off
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def build(verbose: bool = False, extra: list[str] | None = None, out: str | None = None,
          incremental: bool = False) -> str:
    """Compile the library: one object per source file (in parallel), then one link.  ``extra``
    adds compiler flags and ``out`` names another output file (a tuning build next to the shipped
    one, loaded through the PQHSA_LIBRARY variable).  ``incremental`` keeps objects that are newer
    than every source and header (a convenience while editing; the default compiles everything)."""
    os.makedirs(LIBDIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    out = out or LIB
    tag = os.path.splitext(os.path.basename(out))[0]
    objdir = os.path.join(LIBDIR, "obj_" + tag)
    os.makedirs(objdir, exist_ok=True)
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    headers.append(os.path.join(os.path.dirname(HERE), "include", "pqhsa.h"))
    newest_header = max(os.path.getmtime(h) for h in headers)

    def compile_one(src: str) -> str:
        path = os.path.join(CSRC, src)
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        if incremental and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(path), newest_header):
            return obj
        cmd = [hipcc, *FLAGS, *(extra or []), "-c", path, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True)
        return obj

    with ThreadPoolExecutor(max_workers=min(len(SOURCES), os.cpu_count() or 1)) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", out]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return out


if __name__ == "__main__":
    args = sys.argv[1:]
    inc = "--incremental" in args
    print(build(verbose=True, extra=[a for a in args if a != "--incremental"], incremental=inc))
