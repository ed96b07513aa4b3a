"""Per-workgroup phase clocks of the decode step's kernels.

A build of the library with ``-DPQHSA_TRACE`` makes every workgroup of the five kernels store the
wall clock (100 MHz) at a few marks; this tool builds that variant next to the shipped library
(``lib/libpqhsa_trace.so``, never loaded by anything else), runs decode steps of one of the
benchmark's configurations with it and prints, per kernel, when the workgroups pass each mark
(microseconds from the kernel's first workgroup) and how long the phases between marks take.

    python -m pqhsa_release_amd.trace_clocks --build          # compile the variant (hipcc, no GPU needed)
    python -m pqhsa_release_amd.trace_clocks --config 2       # on a GPU: the tables

The marks (slot numbers as printed):
  lut     0 start, 1 query rows loaded, 2 rows normalised, 3 centroid tile staged (tables written
          for the table block), 4 end
  sample  0 start, 1 tables and first sampled keys loaded, 2 sampled keys scored, 3 smallest and
          largest key known, 4 threshold found (end); where the launch also builds the tables (no
          lut launch then): 5 query row normalised, 6 first half of every centroid staged, 7 list scores and
          PQ table done
  scan    0 start, 1 tables staged, 2 last window scored, 3 candidates and per-list sums flushed (end)
  select  0 start, 1 candidates requested and LDS cleared, 2 histogram of the keys built, 3 k-th key
          found and ties ranked, 4 output slots assigned, 5 winners and losers' weights written, 6 end
  attend  0 start, 1 chunk consumed and partial stored, 2 hand-over (and fold, for the row's last) done
"""
import argparse
import ctypes
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
TRACE_LIB = os.path.join(HERE, "lib", "libpqhsa_trace.so")
KERNELS = ["lut", "sample", "scan", "select", "attend"]
SLOTS, MAX_WGS = 8, 8192


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--build", action="store_true", help="compile the tracing variant of the library and exit")
    ap.add_argument("--config", type=int, default=2, help="benchmark configuration (bench.py CONFIGS)")
    ap.add_argument("--kernels", default=",".join(KERNELS))
    args = ap.parse_args()
    if args.build:
        from pqhsa_release_amd import build
        print(build.build(extra=["-DPQHSA_TRACE"], out=TRACE_LIB))
        return
    if not os.path.exists(TRACE_LIB):
        sys.exit(f"{TRACE_LIB} is missing: run this tool with --build first")
    os.environ["PQHSA_LIBRARY"] = TRACE_LIB
    sys.path.insert(0, ROOT)
    import numpy as np
    import torch
    import bench
    from pqhsa_release_amd import _lib

    lib = _lib.load()
    dev = torch.device("cuda:0")
    layers = [bench.Layer(args.config, 100 + 7919 * i, dev) for i in range(2)]
    stream = torch.cuda.current_stream().cuda_stream
    # the traced step follows others without a pause, as in a timed run (a kernel that starts on an
    # idle GPU sees its workgroups dispatched over several microseconds)
    for i in range(7):
        layers[i % 2].call.run(stream)
    torch.cuda.synchronize()
    for name in args.kernels.split(","):
        fn = getattr(lib, "pqhsa_trace_read_trace_" + name)
        buf = (ctypes.c_uint64 * (MAX_WGS * SLOTS))()
        if fn(buf) != 0:
            sys.exit("reading the trace of " + name + " failed")
        a = np.frombuffer(buf, dtype=np.uint64).reshape(MAX_WGS, SLOTS).astype(np.int64)
        a = a[a[:, 0] != 0]
        if len(a) == 0:
            print(f"== {name}: no marks (the kernel did not run at this configuration)")
            continue
        used = [s for s in range(SLOTS) if (a[:, s] != 0).any()]
        used.sort(key=lambda s: np.median(a[:, s][a[:, s] != 0]))  # (in the order the workgroups pass them)
        rel = (a - a[:, 0].min()) / 100.0
        print(f"== {name} (cfg {args.config}): {len(a)} workgroups; first start to last end {rel[:, used].max():.2f} us")
        print("| mark | workgroups | earliest | 10 % | median | 90 % | latest |")
        print("|---|---|---|---|---|---|---|")
        for s in used:
            x = rel[:, s][a[:, s] != 0]
            print(f"| {s} | {len(x)} | {x.min():.2f} | {np.percentile(x, 10):.2f} | {np.percentile(x, 50):.2f} | "
                  f"{np.percentile(x, 90):.2f} | {x.max():.2f} |")
        full = (a[:, used] != 0).all(axis=1)
        if full.any() and len(used) > 1:
            d = np.diff(rel[full][:, used], axis=1)
            print("| phase | mean us | 90 % | longest |")
            print("|---|---|---|---|")
            for i in range(d.shape[1]):
                print(f"| {used[i]} -> {used[i + 1]} | {d[:, i].mean():.2f} | {np.percentile(d[:, i], 90):.2f} | {d[:, i].max():.2f} |")


if __name__ == "__main__":
    main()
