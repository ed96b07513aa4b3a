#!/usr/bin/env python3
"""PQ-HSA decode-attention benchmark: one step = one layer's single-token decode attention
over one batch of synthetic sequences resident in HBM.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2]

Prints ONE JSON line: decode-attention microseconds per layer on the headline configuration
(Llama-3-8B-shape layer, 131 072-token context, batch 4, bf16 paged K/V), the HBM roofline of
the dominant kernel from HIP-event timings taken on the launch stream, and the torch-CPU
restatement of the reference path timed on this box's host cores.
"""

from __future__ import annotations

import argparse
import ctypes
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
MODEL_LAYERS = 32  # Llama-3-8B depth, for the tokens/s figure

CONFIGS = {
    # name: (description, batch, kv_heads, groups, ctx or (lo, hi), dtype, paged, shuffled blocks)
    0: ("cfg0: single KV head, single query, ctx 8192, fp32", 1, 1, 1, 8192, torch.float32, False, False),
    1: ("cfg1: Llama-3-8B-shape layer, batch 1, ctx 32768, bf16 paged (block 16)", 1, 8, 4, 32768,
        torch.bfloat16, True, True),
    2: ("cfg2: Llama-3-8B-shape layer, batch 4, ctx 131072, bf16 paged (block 16)", 4, 8, 4, 131072,
        torch.bfloat16, True, True),
    3: ("cfg3: ragged batch 16, ctx U[16K,64K], bf16 paged, shuffled blocks", 16, 8, 4, (16384, 65536),
        torch.bfloat16, True, True),
    4: ("cfg4: GQA-7 layer, batch 1, ctx 262144, bf16 paged", 1, 4, 7, 262144, torch.bfloat16, True, True),
}
SINK, LOCAL, FRACTION, LISTS, BLOCK = 4, 64, 0.02, 512, 16
KERNELS = ["lut_build", "sample_thresh", "scan_emit", "select_final", "attend_partial", "attend_reduce"]

# HBM bytes per launch (read + written) of each kernel, from two rocprofv3 counter runs of this
# script (FETCH_SIZE, then WRITE_SIZE), each scaled by what the same counter reads for a plain
# 256 MiB device copy (factor 2.0 for FETCH_SIZE, 1.0 for WRITE_SIZE, KiB per dispatch).  Counters
# cannot be read from inside the timed run, so the figure is carried here per workload; it is
# reported only for the configuration it was measured on.
MEASURED_TRAFFIC_BYTES = {
    2: {"lut_build": 9_637_000, "sample_thresh": 6_699_000, "scan_emit": 69_658_000, "select_final": 14_521_000,
        "attend_partial": 183_694_000, "attend_reduce": 1_693_000},
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def make_stream(ctx, groups, seed, device, dtype):
    """Seeded keys/values/queries of one (sequence, KV head), drawn on the device generator."""
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    dim = 128
    centres = torch.randn(512, dim, generator=gen, device=device)
    member = torch.randint(0, 512, (ctx,), generator=gen, device=device)
    keys = centres[member] + 0.3 * torch.randn(ctx, dim, generator=gen, device=device)
    scale = torch.exp(0.5 * torch.randn(dim, generator=gen, device=device))
    outliers = torch.randperm(dim, generator=gen, device=device)[:4]
    scale[outliers] *= 8.0
    keys = keys * scale
    values = torch.randn(ctx, dim, generator=gen, device=device)
    needle = torch.randint(8, max(9, ctx - 128), (groups,), generator=gen, device=device)
    queries = keys[needle] + 0.2 * torch.randn(groups, dim, generator=gen, device=device)
    return keys.to(dtype), values.to(dtype), queries.to(dtype)


class Layer:
    """One layer's resident state: K/V (paged or dense), trained + encoded index, queries."""

    def __init__(self, cfg_id, seed0, device, room=0):
        """``room`` > 0 prepares the layer for that many append + decode steps: the cache holds
        ``room`` more tokens per sequence (already written, as a serving engine writes a token's K/V
        before attention runs), and each step makes one of them visible."""
        from pqhsa_release_amd import ops
        from pqhsa_release_amd.index.train import train_ivfpq_batched

        desc, B, H, G, ctx, dtype, paged, shuffled = CONFIGS[cfg_id]
        self.B, self.H, self.G, self.dtype = B, H, G, dtype
        gen = torch.Generator().manual_seed(seed0)
        if isinstance(ctx, tuple):
            self.lens = [int(x) for x in torch.randint(ctx[0], ctx[1] + 1, (B,), generator=gen)]
        else:
            self.lens = [ctx] * B
        self.n = [max(SINK, ln - LOCAL) - SINK for ln in self.lens]
        n_max = max(self.n)
        self.index = ops.DeviceIndex(B, H, LISTS, n_max + room + 256, device)
        self.room, self.t = room, 0
        if paged:
            blocks_per = [(ln + room + BLOCK - 1) // BLOCK for ln in self.lens]
            total = sum(blocks_per)
            order = torch.randperm(total, generator=gen) if shuffled else torch.arange(total)
            table = torch.zeros(B, max(blocks_per), dtype=torch.int32)
            at = 0
            for b, nb in enumerate(blocks_per):
                table[b, :nb] = order[at : at + nb].to(torch.int32)
                at += nb
            self.block_table = table.to(device)
            self.cache = torch.zeros(2, total, BLOCK, H, 128, dtype=dtype, device=device)
            self.kv = ops.kv_paged(self.cache, self.block_table)
        else:
            self.keys = torch.zeros(B, H, max(self.lens) + room, 128, dtype=dtype, device=device)
            self.values = torch.zeros_like(self.keys)
            self.kv = ops.kv_contiguous(self.keys, self.values)
        q = torch.empty(B, H * G, 128, dtype=dtype, device=device)
        for b, ln0 in enumerate(self.lens):
            ln = ln0 + room
            pos = torch.arange(ln, device=device)
            head_keys = []
            for h in range(H):
                k, v, qq = make_stream(ln, G, seed0 + 1000 * b + h, device, dtype)
                if paged:
                    blk = self.block_table[b, pos // BLOCK].long()
                    self.cache[0, blk, pos % BLOCK, h] = k
                    self.cache[1, blk, pos % BLOCK, h] = v
                else:
                    self.keys[b, h, :ln] = k
                    self.values[b, h, :ln] = v
                q[b, h * G : (h + 1) * G] = qq
                head_keys.append(k[SINK : SINK + self.n[b]])
                del k, v
            # the sequence's KV heads have one length: their indexes train together
            coarse, books = train_ivfpq_batched(torch.stack(head_keys), num_lists=LISTS, coarse_iter=1, pq_iter=2,
                                                seed=0)
            self.index.coarse[b * H : (b + 1) * H, : coarse.shape[1]] = coarse
            self.index.codebooks[b * H : (b + 1) * H] = books
            del head_keys
        self.q = q
        self.out = torch.empty_like(q)
        self.index.set_counts(self.n)
        ops.encode(self.kv, self.index, SINK, [0] * B, self.n)
        self.index.finalize_layout()
        ops.value_summaries(self.kv, self.index, SINK)
        self.seq_lens = torch.tensor(self.lens, dtype=torch.int32, device=device)
        k_cap = ops.resolve_topk(n_max + room, FRACTION, 0)
        self.ws = ops.DecodeWorkspace(self.index, G, k_cap)
        self.call = ops.DecodeCall(self.q, self.out, self.kv, self.index, G, self.seq_lens, sink=SINK,
                                   full_max=SINK + LOCAL, fraction=FRACTION, topk=0, scale=1.0 / math.sqrt(128),
                                   workspace=self.ws)
        if room:
            # step t sees lens + t tokens; the key that leaves the local window is appended by the step
            steps = torch.arange(room + 1, dtype=torch.int32).unsqueeze(1)
            self.seq_steps = (torch.tensor(self.lens, dtype=torch.int32).unsqueeze(0) + steps).to(device).contiguous()
            self.ones = torch.ones(B, dtype=torch.int32, device=device)
            self.append_call = ops.DecodeCall(self.q, self.out, self.kv, self.index, G, self.seq_lens, sink=SINK,
                                              full_max=SINK + LOCAL, fraction=FRACTION, topk=0,
                                              scale=1.0 / math.sqrt(128), workspace=self.ws, append_count=self.ones)
        torch.cuda.synchronize()

    def append_step(self, stream):
        """One serving step: the next token becomes visible, its predecessor that leaves the local
        window is encoded into the index, then attention runs (one fused call)."""
        if self.t >= self.room:
            raise RuntimeError("bench layer: no room left for another append step")
        self.t += 1
        self.append_call.n_max = max(self.n) + self.t
        self.append_call.run(stream, seq_lens_ptr=self.seq_steps[self.t].data_ptr())
        self.index.note_appended([1] * self.B)

    def algorithmic_bytes(self):
        """Bytes each kernel must touch per launch (10 B per indexed key-head, tables, selected and
        full K/V rows, list means)."""
        e = 4 if self.dtype == torch.float32 else 2
        scan = sum(self.H * n * 10 for n in self.n)
        tables = self.B * self.H * (LISTS * 128 + 8 * 16 * 16) * 4
        exact = sum(self.H * self.G * math.ceil(n * FRACTION) * 2 * 128 * e for n in self.n)
        full = sum(self.H * (min(SINK, ln) + ln - (SINK + n)) * 2 * 128 * e for ln, n in zip(self.lens, self.n))
        bg = self.B * self.H * LISTS * 128 * 4
        sample = self.B * self.H * self.index.s_cap * 10
        return {"scan": scan, "sample": sample, "tables": tables, "exact": exact, "full": full, "bg": bg,
                "total": scan + tables + exact + full + bg}


def copy_bandwidth(device, mib=1024, reps=10):
    """HBM bandwidth a plain device-to-device copy reaches on this box (bytes read + written per
    second), the practical ceiling the roofline fraction can also be read against."""
    src = torch.empty(mib * 262144, dtype=torch.float32, device=device).normal_()
    dst = torch.empty_like(src)
    dst.copy_(src)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        dst.copy_(src)
    e1.record()
    torch.cuda.synchronize()
    return 2.0 * src.numel() * 4 * reps / (e0.elapsed_time(e1) * 1e-3) / 1e9


def standalone_kernels(layer, reps=20):
    """The stand-alone entry points on the same layer, buffers allocated once: the LUT scan that
    writes every logit (pqhsa_lut_scan) and the exact top-k of that logit matrix
    (pqhsa_topk_radix, two passes over the logits).  Times by torch events on the current stream."""
    from pqhsa_release_amd import _lib, ops

    lib, idx, G = _lib.load(), layer.index, layer.G
    bh, rows = idx.batch * idx.kv_heads, idx.batch * idx.kv_heads * layer.G
    qnorm, lut, ls = ops.lut_build(layer.q, idx, G)
    logits = torch.zeros(bh, G, idx.n_cap, dtype=torch.float32, device=idx.device)
    n = [layer.n[r // (idx.kv_heads * G)] for r in range(rows)]
    k = [math.ceil(x * FRACTION) for x in n]
    n_t = torch.tensor(n, dtype=torch.int32, device=idx.device)
    k_t = torch.tensor(k, dtype=torch.int32, device=idx.device)
    n_max, k_cap = max(n), max(max(k), 1)
    ws_bytes = lib.pqhsa_topk_workspace_bytes(rows, n_max)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=idx.device)
    tidx = torch.empty(rows, k_cap, dtype=torch.int32, device=idx.device)
    tval = torch.empty(rows, k_cap, dtype=torch.float32, device=idx.device)
    stream = torch.cuda.current_stream().cuda_stream

    # the layer's index is sorted by list, so logits are scattered to their retrieval-local columns;
    # with an identity position map the same kernel writes them in stored order, as for an index
    # that was never regrouped (same bytes, coalesced)
    arrival = type(idx.struct()).from_buffer_copy(idx.struct())
    ident = torch.arange(idx.n_cap, dtype=torch.int32, device=idx.device).repeat(bh, 1)
    arrival.pos = ident.data_ptr()
    which = {"ref": idx.ref()}

    def scan():
        _lib.check(lib.pqhsa_lut_scan(which["ref"], G, int(idx.n_max), qnorm.data_ptr(), lut.data_ptr(), ls.data_ptr(),
                                      1.0 / math.sqrt(128), logits.data_ptr(), idx.n_cap, stream), "pqhsa_lut_scan")

    def topk():
        _lib.check(lib.pqhsa_topk_radix(logits.data_ptr(), idx.n_cap, rows, n_t.data_ptr(), k_t.data_ptr(), n_max,
                                        tidx.data_ptr(), tval.data_ptr(), k_cap, ws.data_ptr(), ws_bytes, stream),
                   "pqhsa_topk_radix")

    out = {}
    keys = sum(layer.n) * idx.kv_heads
    for name, fn, nbytes in (("lut_scan_sorted_index", scan, keys * 14 + keys * G * 4),
                             ("lut_scan_arrival_order", scan, keys * 14 + keys * G * 4),
                             ("topk_radix", topk, 2 * keys * G * 4)):
        which["ref"] = ctypes.byref(arrival) if name == "lut_scan_arrival_order" else idx.ref()
        for _ in range(3):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1000.0 / reps
        out[name] = {"us": round(us, 2), "MB": round(nbytes / 1e6, 2), "GBps": round(nbytes / 1e3 / us, 1),
                     "frac_of_peak": round(nbytes / 1e3 / us / HBM_PEAK_GBPS, 4)}
    return out


def cpu_baseline(layer, seconds=12.0):
    """Time the torch-CPU restatement of the reference path on one (sequence, KV head) stream of
    the same inputs and trained index, and scale to the whole layer."""
    from oracle import torch_ref as tr
    from pqhsa_release_amd import ops

    b = h = 0
    bh, n, ln, G = 0, layer.n[0], layer.lens[0], layer.G
    kk, vv = ops.paged_gather_range(layer.kv, b, 0, ln) if layer.kv.view.paged else (layer.keys[b], layer.values[b])
    keys, values = kk[h].float().cpu(), vv[h].float().cpu()
    idx = layer.index
    _, lists_by_key, norms_by_key = idx.by_key(bh, n)
    ref = tr.RefIndex(idx.coarse[bh].cpu(), idx.codebooks[bh].cpu(), (lists_by_key.to(torch.int64) & 0xFFFF).cpu(),
                      idx.packed_bytes(bh, n).cpu().clone(), norms_by_key.cpu())
    vbar = idx.vbar[bh].cpu()
    q = layer.q[b, h * G : (h + 1) * G].float().cpu()
    cores = os.cpu_count() or 1
    cores = min(cores, 16)
    torch.set_num_threads(cores)
    args = dict(sink_end=SINK, retrieval_end=SINK + n, index=ref, vbar=vbar, fraction=FRACTION,
                scale=1.0 / math.sqrt(128))
    out = tr.hybrid_forward_many(q, keys, values, **args)
    t0, reps = time.perf_counter(), 0
    while True:
        tr.hybrid_forward_many(q, keys, values, **args)
        reps += 1
        if time.perf_counter() - t0 > seconds and reps >= 3:
            break
    per_stream = (time.perf_counter() - t0) / reps
    torch.set_num_threads(1)  # the same sample on one core, for a quarter of the time budget
    t1, reps1 = time.perf_counter(), 0
    while True:
        tr.hybrid_forward_many(q, keys, values, **args)
        reps1 += 1
        if time.perf_counter() - t1 > seconds / 4 and reps1 >= 2:
            break
    per_stream_1 = (time.perf_counter() - t1) / reps1
    torch.set_num_threads(cores)
    got = layer.out[b, h * G : (h + 1) * G].float().cpu()
    err = None if layer.t else float((got - out).abs().max())  # after append steps the device result is for a longer context
    streams = sum(1 for _ in range(layer.B * layer.H))
    scale_factor = sum(layer.n) * layer.H / max(n, 1)  # streams weighted by their indexed length
    return {
        "value": per_stream * scale_factor * 1e6,
        "unit": "us/layer",
        "cores": cores,
        "kind": "port",
        "sample": f"torch-CPU restatement of forward_many on 1 of {streams} (sequence, KV head) streams "
                  f"(n={n}, G={G}), {reps} reps, scaled by indexed keys to the whole layer",
        "single_core_value": per_stream_1 * scale_factor * 1e6,
        "max_abs_diff_vs_gpu": err,
        "gpu_out_dtype": str(layer.out.dtype).replace("torch.", ""),  # a bf16 output carries 2^-9 relative rounding
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=2)
    ap.add_argument("--layers", type=int, default=3, help="distinct resident layers rotated through (defeats cache reuse)")
    ap.add_argument("--event-every", type=int, default=8,
                    help="in the timed region the dominant kernel is bracketed by HIP events on one step in this many")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--append", action="store_true",
                    help="every step appends one key per sequence before it attends (always on for config 4)")
    ap.add_argument("--standalone", action="store_true",
                    help="also time the stand-alone entry points (pqhsa_lut_scan writing all logits, "
                         "pqhsa_topk_radix on that matrix) and report their HBM rates")
    ap.add_argument("--calibrate-copy-mib", type=int, default=0,
                    help="also run one device copy of this many MiB after the warm-up (a kernel of known HBM "
                         "traffic, the yardstick for FETCH_SIZE / WRITE_SIZE counter runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU (every sequence and KV head of the layer is on it); "
                 "--gpus must be 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the PQ-HSA kernels have no CPU path")

    from pqhsa_release_amd import _lib

    lib = _lib.load()
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    t_setup = time.perf_counter()
    appending = args.append or args.config == 4
    nl = max(1, args.layers)
    room = (3 * args.steps + 4 * args.warmup + 60 + nl - 1) // nl + 8 if appending else 0
    layers = [Layer(args.config, 100 + 7919 * i, device, room=room) for i in range(nl)]
    log(f"setup {time.perf_counter() - t_setup:.1f}s: {CONFIGS[args.config][0]}, {len(layers)} resident layers")
    stream = torch.cuda.current_stream().cuda_stream

    def run_steps(count, offset=0):
        for i in range(count):
            layer = layers[(i + offset) % len(layers)]
            if appending:
                layer.append_step(stream)
            else:
                layer.call.run(stream)

    run_steps(args.warmup)
    torch.cuda.synchronize()
    if args.calibrate_copy_mib > 0:
        src = torch.empty(args.calibrate_copy_mib * 262144, dtype=torch.float32, device=device).normal_()
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    def logged_run(count, only, every=1):
        """count steps with the HIP-event log on the stream, one step in `every` carrying the
        records; returns (ms per step, per-kernel ms averaged over the logged steps)."""
        _lib.check(lib.pqhsa_profile_enable(count), "pqhsa_profile_enable")
        _lib.check(lib.pqhsa_profile_only(only), "pqhsa_profile_only")
        _lib.check(lib.pqhsa_profile_every(every), "pqhsa_profile_every")
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run_steps(count)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        kms = (ctypes.c_float * len(KERNELS))()
        seen = ctypes.c_int32(0)
        _lib.check(lib.pqhsa_profile_collect(kms, ctypes.byref(seen)), "pqhsa_profile_collect")
        assert seen.value == (count + every - 1) // every, (seen.value, count, every)
        return (t1 - t0) * 1000.0 / count, [float(v) for v in kms]

    # untimed survey with every kernel bracketed by events: finds the dominant kernel
    _, survey = logged_run(max(args.warmup, 20), -1)
    dominant_i = max(range(len(KERNELS)), key=lambda i: survey[i])
    dominant = KERNELS[dominant_i]
    # timed region: exactly --steps steps; the dominant kernel carries two event records on one
    # step in --event-every, spread over the whole region: what its roofline figure is measured from
    ms_per_step, dom_ms = logged_run(args.steps, dominant_i, max(1, args.event_every))
    # the same steps with no event at all, to show what the records cost
    run_steps(args.warmup)
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    run_steps(args.steps)
    torch.cuda.synchronize()
    ms_plain = (time.perf_counter() - t2) * 1000.0 / args.steps

    # the same steps replayed from HIP graphs (one per resident layer): what a serving loop that
    # captures its steady state would see
    ms_graph = None
    if not appending:  # (a captured graph has the key count of its capture baked into its launch shapes)
        for l in layers:
            l.call.capture()
        for i in range(args.warmup):
            layers[i % len(layers)].call.replay()
        torch.cuda.synchronize()
        t3 = time.perf_counter()
        for i in range(args.steps):
            layers[i % len(layers)].call.replay()
        torch.cuda.synchronize()
        ms_graph = (time.perf_counter() - t3) * 1000.0 / args.steps

    layer = layers[0]
    ab = layer.algorithmic_bytes()
    kus = {name: survey[i] * 1000.0 for i, name in enumerate(KERNELS)}
    algo = {"lut_build": ab["tables"], "sample_thresh": ab["sample"], "scan_emit": ab["scan"],
            "select_final": 0, "attend_partial": ab["exact"] + ab["full"], "attend_reduce": ab["bg"]}
    kernels = {}
    for name in KERNELS:
        us = kus[name]
        kernels[name] = {"us": round(us, 3), "algo_MB": round(algo[name] / 1e6, 3),
                         "GBps": round(algo[name] / 1e3 / us, 1) if us > 0 else None}
    dom_us = dom_ms[dominant_i] * 1000.0
    dom_bytes = algo[dominant]
    roofline = {
        "kernel": dominant,
        "bound": "hbm",
        "achieved": round(dom_bytes / 1e3 / dom_us, 1),
        "peak": HBM_PEAK_GBPS,
        "unit": "GB/s",
        "frac": round(dom_bytes / 1e3 / dom_us / HBM_PEAK_GBPS, 4),
        "traffic": MEASURED_TRAFFIC_BYTES.get(args.config, {}).get(dominant),
        "algorithmic_bytes": dom_bytes,
        "launch_us": round(dom_us, 3),
        "launches_timed": (args.steps + max(1, args.event_every) - 1) // max(1, args.event_every),
    }
    scan_us = kus["scan_emit"]
    result = {
        "metric": "decode attn us/layer at 128K ctx (8 KV heads); LUT-scan HBM GB/s vs peak",
        "value": round(ms_per_step * 1000.0, 3),
        "unit": "us/layer",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": CONFIGS[args.config][0], "batch": layer.B, "kv_heads": layer.H,
                   "gqa_group": layer.G, "context": layer.lens if len(set(layer.lens)) > 1 else layer.lens[0],
                   "num_lists": LISTS, "top_fraction": FRACTION, "sink": SINK, "local_window": LOCAL,
                   "kv_dtype": str(layer.dtype).replace("torch.", ""), "resident_layers": len(layers)},
        "roofline": roofline,
        "tokens_per_s": round(layer.B / (MODEL_LAYERS * ms_per_step / 1000.0), 1),
        "step_bytes_MB": round(ab["total"] / 1e6, 2),
        "step_roofline_frac": round(ab["total"] / 1e3 / (ms_per_step * 1000.0) / HBM_PEAK_GBPS, 4),
        "lut_scan": {"us": round(scan_us, 3), "algo_MB": round(ab["scan"] / 1e6, 3),
                     "GBps": round(ab["scan"] / 1e3 / scan_us, 1) if scan_us > 0 else None,
                     "frac_of_peak": round(ab["scan"] / 1e3 / scan_us / HBM_PEAK_GBPS, 4) if scan_us > 0 else None},
        "kernels": kernels,
        "kernel_sum_us": round(sum(kus.values()), 3),
        "ms_per_step_without_event_log": round(ms_plain, 6),
        "ms_per_step_graph_replay": None if ms_graph is None else round(ms_graph, 6),
        "append_per_step": appending,
        "selection": {"k": math.ceil(layer.n[0] * FRACTION), "rescanned_rows": sum(l.ws.rescans() for l in layers),
                      "candidates_mean": round(float(layer.ws.candidate_counts().float().mean()), 1),
                      "candidates_max": int(layer.ws.candidate_counts().max())},
    }
    if args.standalone:
        result["standalone"] = standalone_kernels(layer)
    copy_gbps = copy_bandwidth(device)
    result["hbm_copy_GBps"] = round(copy_gbps, 1)
    result["roofline"]["frac_of_copy"] = round(result["roofline"]["achieved"] / copy_gbps, 4)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(layer, args.cpu_seconds)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
