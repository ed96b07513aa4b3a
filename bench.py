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
KERNELS = ["lut_build", "sample_thresh", "scan_emit", "select_final", "attend"]

# HBM bytes per launch (read + written) of each kernel come from two rocprofv3 counter runs of this
# script (FETCH_SIZE, then WRITE_SIZE), each scaled by what the same counter reads for a plain
# device copy of known size.  Counters cannot be read from inside the timed run, so the figures
# are kept in a small JSON file per workload beside the profile summaries, stamped with the git
# commit of the kernels they were measured on, and are reported together with that stamp.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "decode_step_cfg{cfg}_hbm_traffic.json")


def kernel_sources_digest():
    """SHA-256 over the library's kernel sources (file names and contents, in name order): the stamp a
    counter measurement carries, so that a figure measured on other kernels is not passed on as today's."""
    import hashlib

    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "pqhsa_release_amd", "csrc")
    for name in sorted(os.listdir(csrc)):
        if name.endswith((".hip", ".h")):
            h.update(name.encode())
            with open(os.path.join(csrc, name), "rb") as f:
                h.update(f.read())
    return h.hexdigest()


def measured_traffic(cfg_id, kernel):
    """(HBM bytes per launch from the committed counter runs, the commit they were taken at); the bytes
    are None when there is no measurement of this kernel or the kernel sources have changed since."""
    try:
        with open(TRAFFIC_FILE.format(cfg=cfg_id)) as f:
            rec = json.load(f)
        nbytes = int(rec["bytes_per_launch"][kernel])
        if rec.get("sources_sha256") != kernel_sources_digest():
            return None, rec.get("commit")
        return nbytes, rec.get("commit")
    except (OSError, KeyError, ValueError):
        return None, None


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

    @staticmethod
    def _now(device):
        torch.cuda.synchronize(device)
        return time.perf_counter()

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
        train_s, seq_keys = 0.0, []
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
            seq_keys.append(torch.stack(head_keys))
            del head_keys
        # sequences of one length train together, all their KV heads at once (about 2 GB of fp32 keys per call)
        by_n = {}
        for b, nb in enumerate(self.n):
            by_n.setdefault(nb, []).append(b)
        for nb, seqs in by_n.items():
            step = max(1, ((1 << 31) // (nb * 128 * 4)) // H)
            for i in range(0, len(seqs), step):
                part = seqs[i : i + step]
                t0 = self._now(device)
                coarse, books = train_ivfpq_batched(torch.cat([seq_keys[b] for b in part]), num_lists=LISTS,
                                                    coarse_iter=1, pq_iter=2, seed=0)
                train_s += self._now(device) - t0
                for j, b in enumerate(part):
                    self.index.coarse[b * H : (b + 1) * H, : coarse.shape[1]] = coarse[j * H : (j + 1) * H]
                    self.index.codebooks[b * H : (b + 1) * H] = books[j * H : (j + 1) * H]
        del seq_keys
        self.q = q
        self.out = torch.empty_like(q)
        self.index.set_counts(self.n)
        t0 = self._now(device)
        ops.encode(self.kv, self.index, SINK, [0] * B, self.n)
        t1 = self._now(device)
        self.index.finalize_layout()
        t2 = self._now(device)
        ops.value_summaries(self.kv, self.index, SINK)
        t3 = self._now(device)
        # wall-clock of the index build's parts for this layer (the device drained around each)
        self.build_ms = {"train": round(train_s * 1e3, 2), "encode": round((t1 - t0) * 1e3, 2),
                         "layout": round((t2 - t1) * 1e3, 2), "value_summaries": round((t3 - t2) * 1e3, 2)}
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


def _cpu_stream(layer, b, h):
    """One (sequence, KV head) stream of the layer on the host, in the form the torch restatement takes."""
    from oracle import torch_ref as tr
    from pqhsa_release_amd import ops

    bh, n, ln, G = b * layer.H + h, layer.n[b], layer.lens[b] + layer.t, layer.G
    n += layer.t
    kk, vv = ops.paged_gather_range(layer.kv, b, 0, ln) if layer.kv.view.paged else (layer.keys[b], layer.values[b])
    keys, values = kk[h, :ln].float().cpu(), vv[h, :ln].float().cpu()
    idx = layer.index
    _, lists_by_key, norms_by_key = idx.by_key(bh, n)
    ref = tr.RefIndex(idx.coarse[bh].cpu(), idx.codebooks[bh].cpu(), (lists_by_key.to(torch.int64) & 0xFFFF).cpu(),
                      idx.packed_bytes(bh, n).cpu().clone(), norms_by_key.cpu())
    q = layer.q[b, h * G : (h + 1) * G].float().cpu()
    args = dict(sink_end=SINK, retrieval_end=SINK + n, index=ref, vbar=idx.vbar[bh].cpu(), fraction=FRACTION,
                scale=1.0 / math.sqrt(128))
    return q, keys, values, args


def float64_forward(q, keys, values, args):
    """The same restatement evaluated in float64 on the same stream.  The reference forms the
    background as (all keys' approximate weights) - (the selected keys' approximate weights), both
    relative to the largest approximate logit; where a row's exact logits lie far below that, the
    softmax denominator is a small difference of sums near 1 and the fp32 evaluation keeps few of
    its digits (how few depends on the host's summation order).  The float64 evaluation is what
    both the fp32 restatement and the GPU are held against."""
    import dataclasses

    from oracle import torch_ref as tr

    ix = args["index"]
    ix64 = dataclasses.replace(ix, coarse=ix.coarse.double(), codebooks=ix.codebooks.double(), norms=ix.norms.double())
    a64 = dict(args, index=ix64, vbar=args["vbar"].double())
    return tr.hybrid_forward_many(q.double(), keys.double(), values.double(), **a64)


def host_cores():
    return min(os.cpu_count() or 1, 16)


def fp32_output_step(layer):
    """One more step of the layer with the same query values held in fp32 and an fp32 output (the
    K/V cache stays as it is): what the step computes before the output row is rounded to the
    query dtype.  Only for layers that have taken no append step (the step sees the same index)."""
    from pqhsa_release_amd import ops

    q32 = layer.q.float().contiguous()
    out32 = torch.empty_like(q32)
    ops.decode_step(q32, out32, layer.kv, layer.index, layer.G, layer.seq_lens, sink=SINK, full_max=SINK + LOCAL,
                    fraction=FRACTION, topk=0, scale=1.0 / math.sqrt(128), workspace=layer.ws)
    torch.cuda.synchronize()
    return out32


def index_maintenance(device, batch=4, kv_heads=8, groups=4, ctx=131072, appended=256):
    """Wall-clock of the index work around the decode step, through the adapter a serving engine
    drives (the device drained around each part): the build after prefill (training + encode +
    layout + summaries of all streams), ``appended`` one-token appends with the deferred strategy,
    and the flush that follows them (table moves, re-encode of every key, layout, summaries)."""
    from pqhsa_release_amd.attention import GQAIVFPQDecodeAttentionAdapter
    from pqhsa_release_amd.config import IVFPQConfig, SparseAttentionConfig

    ic = IVFPQConfig(num_lists=LISTS, nprobe=8, num_subspaces=8, num_bits=4, residual=True, coarse_max_iter=1,
                     pq_max_iter=2, kernel_backend="mi355x", direction_normalize=True, seed=0)
    ac = SparseAttentionConfig(sink_tokens=SINK, local_window=LOCAL, retrieval_top_fraction=FRACTION,
                               exact_rerank=True, mode="hybrid", hybrid_value_mode="centroid",
                               index_update_interval=appended, index_update_strategy="deferred",
                               collect_attention_details=False)
    gen = torch.Generator(device=device).manual_seed(1)
    centres = torch.randn(LISTS, 128, device=device, generator=gen)

    def rows(n):
        pick = torch.randint(0, LISTS, (batch, kv_heads, n), device=device, generator=gen)
        k = (centres[pick] + 0.3 * torch.randn(batch, kv_heads, n, 128, device=device, generator=gen)).to(torch.bfloat16)
        return k, torch.randn(batch, kv_heads, n, 128, device=device, generator=gen).to(torch.bfloat16)

    def clock():
        torch.cuda.synchronize(device)
        return time.perf_counter()

    keys, values = rows(ctx)
    adapter = GQAIVFPQDecodeAttentionAdapter(ic, ac, num_query_heads=kv_heads * groups, num_key_value_heads=kv_heads)
    adapter.build_cache(keys, values)                     # first call: allocations, kernel loading
    q = torch.randn(batch, kv_heads * groups, 128, device=device, generator=gen)
    out = {"shape": f"batch {batch} x {kv_heads} KV heads x {ctx} tokens, bf16", "appended_keys_per_flush": appended}
    for rep in range(2):                                  # the second round is the one reported
        nk, nv = rows(appended)
        t0 = clock()
        for s in range(appended):
            adapter.append(nk[:, :, s], nv[:, :, s])
        t1 = clock()
        adapter.forward(q)
        t2 = clock()
        flushed = adapter.apply_pending_index_update()
        t3 = clock()
        out.update(append_us_per_key=round((t1 - t0) / appended * 1e6, 1), flush_ms=round((t3 - t2) * 1e3, 2),
                   flushed=bool(flushed))
    t0 = clock()
    adapter.build_cache(keys, values)
    out["build_ms"] = round((clock() - t0) * 1e3, 2)
    out["flush_us_per_step"] = round(out["flush_ms"] * 1e3 / appended, 1)
    return out


def cpu_baseline(layer, seconds=12.0):
    """Time the torch-CPU restatement of the reference path on one (sequence, KV head) stream of
    the same inputs and trained index, and scale to the whole layer."""
    from oracle import torch_ref as tr

    b = h = 0
    n, G = layer.n[0] + layer.t, layer.G
    q, keys, values, args = _cpu_stream(layer, b, h)
    cores = host_cores()
    torch.set_num_threads(cores)
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
    gpu32 = None if layer.t else fp32_output_step(layer)[b, h * G : (h + 1) * G].cpu()
    err32 = None if layer.t else float((gpu32 - out).abs().max())
    out64 = float64_forward(q, keys, values, args)
    streams = layer.B * layer.H
    scale_factor = sum(layer.n) * layer.H / max(layer.n[0], 1)  # streams weighted by their indexed length
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
        # the same step with fp32 queries and an fp32 output row (no rounding of the result): the
        # figure the 2e-3 bound is stated for; and the largest output magnitude of the compared rows
        # (half an ulp of bf16 at that magnitude is what the rounded output may add)
        "max_abs_diff_vs_gpu_fp32_out": err32,
        "max_abs_out": float(out.abs().max()),
        # both against the float64 evaluation of the same formula (see float64_forward): the GPU's
        # figure is the one the 2e-3 bound is about, the other is the fp32 baseline's own error
        "max_abs_diff_gpu_fp32_out_vs_float64": None if layer.t else float((gpu32.double() - out64).abs().max()),
        "max_abs_diff_cpu_vs_float64": float((out.double() - out64).abs().max()),
    }


def cpu_full_layer(layer, reps=3):
    """The torch-CPU restatement over EVERY stream of the layer, nothing scaled: the layer's
    time is the sum over its streams (best of ``reps`` passes), and every stream's output is
    compared with what the GPU wrote for it."""
    from oracle import torch_ref as tr

    cores = host_cores()
    torch.set_num_threads(cores)
    streams = [_cpu_stream(layer, b, h) for b in range(layer.B) for h in range(layer.H)]
    best, worst, worst32, biggest, gpu64, cpu64 = None, 0.0, 0.0, 0.0, 0.0, 0.0
    out32 = fp32_output_step(layer)
    for rep in range(reps + 1):                       # the first pass warms up and checks
        t0 = time.perf_counter()
        outs = [tr.hybrid_forward_many(q, k, v, **a) for q, k, v, a in streams]
        dt = time.perf_counter() - t0
        if rep == 0:
            G = layer.G
            for i, o in enumerate(outs):
                b, h = divmod(i, layer.H)
                worst = max(worst, float((layer.out[b, h * G : (h + 1) * G].float().cpu() - o).abs().max()))
                worst32 = max(worst32, float((out32[b, h * G : (h + 1) * G].cpu() - o).abs().max()))
                biggest = max(biggest, float(o.abs().max()))
                o64 = float64_forward(*streams[i])
                gpu64 = max(gpu64, float((out32[b, h * G : (h + 1) * G].cpu().double() - o64).abs().max()))
                cpu64 = max(cpu64, float((o.double() - o64).abs().max()))
        else:
            best = dt if best is None else min(best, dt)
    return {"value": best * 1e6, "unit": "us/layer", "cores": cores, "kind": "port",
            "sample": f"all {len(streams)} streams of the layer, best of {reps} passes",
            "max_abs_diff_vs_gpu": worst, "max_abs_diff_vs_gpu_fp32_out": worst32, "max_abs_out": biggest,
            "max_abs_diff_gpu_fp32_out_vs_float64": gpu64, "max_abs_diff_cpu_vs_float64": cpu64}


class Timed:
    """The resident layers of one configuration and the timing passes over them."""

    def __init__(self, lib, device, cfg_id, *, layers, steps, warmup, appending):
        self.lib, self.device, self.cfg_id, self.steps, self.warmup = lib, device, cfg_id, steps, warmup
        self.appending = appending or cfg_id == 4
        nl = max(1, layers)
        room = (3 * steps + 4 * warmup + 60 + nl - 1) // nl + 8 if self.appending else 0
        t0 = time.perf_counter()
        self.layers = [Layer(cfg_id, 100 + 7919 * i, device, room=room) for i in range(nl)]
        log(f"setup {time.perf_counter() - t0:.1f}s: {CONFIGS[cfg_id][0]}, {nl} resident layers")
        self.stream = torch.cuda.current_stream().cuda_stream

    def run_steps(self, count):
        for i in range(count):
            layer = self.layers[i % len(self.layers)]
            if self.appending:
                layer.append_step(self.stream)
            else:
                layer.call.run(self.stream)

    def logged_run(self, count, only, every=1):
        """count steps with the HIP-event log on the stream, one step in `every` carrying the
        records; returns (ms per step, per-kernel ms averaged over the logged steps)."""
        from pqhsa_release_amd import _lib

        lib = self.lib
        _lib.check(lib.pqhsa_profile_enable(count), "pqhsa_profile_enable")
        _lib.check(lib.pqhsa_profile_only(only), "pqhsa_profile_only")
        _lib.check(lib.pqhsa_profile_every(every), "pqhsa_profile_every")
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        self.run_steps(count)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        kms = (ctypes.c_float * len(KERNELS))()
        seen = ctypes.c_int32(0)
        _lib.check(lib.pqhsa_profile_collect(kms, ctypes.byref(seen)), "pqhsa_profile_collect")
        assert seen.value == (count + every - 1) // every, (seen.value, count, every)
        return (t1 - t0) * 1000.0 / count, [float(v) for v in kms]

    def measure(self, event_every):
        self.run_steps(self.warmup)
        torch.cuda.synchronize()
        # untimed survey with every kernel bracketed by events: finds the dominant kernel
        _, survey = self.logged_run(max(self.warmup, 20), -1)
        self.survey_us = {name: survey[i] * 1000.0 for i, name in enumerate(KERNELS)}
        self.dominant_i = max(range(len(KERNELS)), key=lambda i: survey[i])
        self.dominant = KERNELS[self.dominant_i]
        # a short context is one launch (decode_small_kernel): the log books it under its last slot
        # and the other slots hold only the cost of recording an event
        from pqhsa_release_amd import ops
        l0 = self.layers[0]
        self.launches = ops.decode_step_launches(l0.index, l0.G, l0.ws, appending=self.appending)
        # timed region: exactly `steps` steps; the dominant kernel carries two event records on one
        # step in `event_every`, spread over the whole region: what its roofline figure is measured from
        self.event_every = max(1, event_every)
        self.ms_per_step, dom_ms = self.logged_run(self.steps, self.dominant_i, self.event_every)
        self.dominant_us = dom_ms[self.dominant_i] * 1000.0
        # the candidate scan measured the same way, in a pass of its own (the second half of the metric)
        self.scan_us = None
        scan_i = KERNELS.index("scan_emit")
        if self.launches != 1 and scan_i != self.dominant_i:
            _, scan_ms = self.logged_run(self.steps, scan_i, self.event_every)
            self.scan_us = scan_ms[scan_i] * 1000.0
        elif self.launches != 1:
            self.scan_us = self.dominant_us
        layer = self.layers[0]
        ab = self.bytes = layer.algorithmic_bytes()
        self.algo = {"lut_build": ab["tables"], "sample_thresh": ab["sample"], "scan_emit": ab["scan"],
                     "select_final": 0, "attend": ab["exact"] + ab["full"] + ab["bg"]}
        if self.launches == 4:  # tables and threshold estimate share the first launch (booked under its slot)
            self.algo["lut_build"] += self.algo["sample_thresh"]
            self.algo["sample_thresh"] = 0
        if self.launches == 1:
            self.survey_us = {name: (us if name == self.dominant else 0.0) for name, us in self.survey_us.items()}
            self.algo = {name: (ab["total"] if name == self.dominant else 0) for name in KERNELS}

    def plain_ms(self):
        """The same steps with no event at all, to show what the records cost."""
        self.run_steps(self.warmup)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        self.run_steps(self.steps)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1000.0 / self.steps

    def graph_ms(self):
        """The same steps replayed from HIP graphs (one per resident layer), or None for steps that
        append (a captured graph has the key count of its capture in its launch shapes)."""
        if self.appending:
            return None
        for l in self.layers:
            l.call.capture()
        for i in range(self.warmup):
            self.layers[i % len(self.layers)].call.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(self.steps):
            self.layers[i % len(self.layers)].call.replay()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1000.0 / self.steps

    def roofline(self):
        nbytes = self.algo[self.dominant]
        traffic, commit = measured_traffic(self.cfg_id, self.dominant)
        return {
            "kernel": self.label(self.dominant),
            "bound": "hbm",
            "achieved": round(nbytes / 1e3 / self.dominant_us, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(nbytes / 1e3 / self.dominant_us / HBM_PEAK_GBPS, 4),
            "traffic": traffic,
            "traffic_measured_at_commit": commit,
            "algorithmic_bytes": nbytes,
            "launch_us": round(self.dominant_us, 3),
            "launches_timed": (self.steps + self.event_every - 1) // self.event_every,
        }

    def roofline_scan(self):
        """The candidate scan against the HBM roofline (None for a step served by the one-kernel path)."""
        if self.scan_us is None or self.scan_us <= 0:
            return None
        nbytes = self.algo["scan_emit"]
        traffic, commit = measured_traffic(self.cfg_id, "scan_emit")
        return {
            "kernel": "scan_emit",
            "bound": "hbm",
            "achieved": round(nbytes / 1e3 / self.scan_us, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(nbytes / 1e3 / self.scan_us / HBM_PEAK_GBPS, 4),
            "traffic": traffic,
            "traffic_measured_at_commit": commit,
            "algorithmic_bytes": nbytes,
            "launch_us": round(self.scan_us, 3),
            "launches_timed": (self.steps + self.event_every - 1) // self.event_every,
        }

    def label(self, name):
        if self.launches == 4 and name == "lut_build":
            return "tables_thresh (tables + threshold estimate)"
        return "decode_small (whole step)" if self.launches == 1 and name == self.dominant else name

    def hidden(self, name):
        """Slots of the event log that hold no launch of their own in this step's form."""
        return (self.launches == 1 and name != self.dominant) or (self.launches == 4 and name == "sample_thresh")

    def kernels(self):
        out = {}
        for name in KERNELS:
            if self.hidden(name):
                continue
            us = self.survey_us[name]
            out[self.label(name)] = {"us": round(us, 3), "algo_MB": round(self.algo[name] / 1e6, 3),
                         "GBps": round(self.algo[name] / 1e3 / us, 1) if us > 0 else None}
        return out

    def step_frac(self):
        return round(self.bytes["total"] / 1e3 / (self.ms_per_step * 1000.0) / HBM_PEAK_GBPS, 4)

    def summary(self):
        """The short per-configuration record of the default run's "configs" object."""
        r = self.roofline()
        return {"workload": CONFIGS[self.cfg_id][0], "us_per_layer": round(self.ms_per_step * 1000.0, 3),
                "steps": self.steps, "resident_layers": len(self.layers), "append_per_step": self.appending,
                "step_bytes_MB": round(self.bytes["total"] / 1e6, 2), "step_roofline_frac": self.step_frac(),
                "launches_per_step": self.launches,
                "dominant": {"kernel": r["kernel"], "launch_us": r["launch_us"], "GBps": r["achieved"], "frac": r["frac"]},
                "kernels_us": {self.label(k): round(v, 2) for k, v in self.survey_us.items() if not self.hidden(k)},
                "rescanned_rows": sum(l.ws.rescans() for l in self.layers)}

    def gather_ceiling(self, reps=30):
        """Rate at which this GPU delivers the very rows the last steps selected (K and V rows of the
        selected keys of every query row, read through the same addressing as the attention kernel by a
        kernel that does nothing else), rotating through the resident layers like the timed steps."""
        from pqhsa_release_amd import ops

        cases = []
        for l in self.layers:
            rows = l.B * l.H * l.G
            idx = l.ws.topk_idx.reshape(rows, -1).clone()
            cnt = l.ws.topk_cnt.reshape(rows, 1)
            col = torch.arange(idx.shape[1], device=idx.device).unsqueeze(0)
            idx = torch.where(col < cnt, idx, idx[:, :1])          # unused tail entries: a valid row again
            pos = (idx + SINK).reshape(l.B * l.H, -1).to(torch.int32).contiguous()
            cases.append((l.kv, pos, torch.zeros(ops.PROBE_SLOTS, dtype=torch.int32, device=idx.device)))
        for kv, pos, checks in cases:
            ops.gather_probe(kv, pos, checks)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for i in range(reps):
            ops.gather_probe(*cases[i % len(cases)])
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1000.0 / reps
        esz = 4 if self.layers[0].dtype == torch.float32 else 2
        nbytes = cases[0][1].numel() * 2 * 128 * esz
        return {"us": round(us, 2), "MB": round(nbytes / 1e6, 2), "GBps": round(nbytes / 1e3 / us, 1)}

    def close(self):
        self.layers = []
        torch.cuda.empty_cache()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=2)
    ap.add_argument("--layers", type=int, default=3, help="distinct resident layers rotated through (defeats cache reuse)")
    ap.add_argument("--event-every", type=int, default=10,
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
    ap.add_argument("--calibrate-gather", action=argparse.BooleanOptionalAction, default=True,
                    help="time a kernel that only reads the selected K/V rows and report its rate as "
                         "roofline.random_row_ceiling_GBps (the practical ceiling of the attention kernel)")
    ap.add_argument("--other-configs", action=argparse.BooleanOptionalAction, default=None,
                    help="after the main configuration, run short passes over the other configurations and "
                         "report them under \"configs\" (default: only when --config is the headline one)")
    ap.add_argument("--other-steps", type=int, default=60)
    ap.add_argument("--index-maintenance", action=argparse.BooleanOptionalAction, default=None,
                    help="also time the index build and the deferred flush at the cfg 2 shape through the adapter "
                         "(default: with the default configuration)")
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
    run = Timed(lib, device, args.config, layers=args.layers, steps=args.steps, warmup=args.warmup, appending=args.append)
    if args.calibrate_copy_mib > 0:
        run.run_steps(args.warmup)
        src = torch.empty(args.calibrate_copy_mib * 262144, dtype=torch.float32, device=device).normal_()
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    run.measure(args.event_every)
    ms_per_step = run.ms_per_step
    ms_plain = run.plain_ms()
    ms_graph = run.graph_ms()

    layer = run.layers[0]
    ab = run.bytes
    scan_us = run.survey_us["scan_emit"]
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
                   "kv_dtype": str(layer.dtype).replace("torch.", ""), "resident_layers": len(run.layers)},
        "roofline": run.roofline(),
        "roofline_scan": run.roofline_scan(),
        "tokens_per_s": round(layer.B / (MODEL_LAYERS * ms_per_step / 1000.0), 1),
        "step_bytes_MB": round(ab["total"] / 1e6, 2),
        "step_roofline_frac": run.step_frac(),
        "lut_scan": {"us": round(scan_us, 3), "algo_MB": round(ab["scan"] / 1e6, 3),
                     "GBps": round(ab["scan"] / 1e3 / scan_us, 1) if scan_us > 0 else None,
                     "frac_of_peak": round(ab["scan"] / 1e3 / scan_us / HBM_PEAK_GBPS, 4) if scan_us > 0 else None},
        "kernels": run.kernels(),
        "kernel_sum_us": round(sum(run.survey_us.values()), 3),
        "ms_per_step_without_event_log": round(ms_plain, 6),
        "ms_per_step_graph_replay": None if ms_graph is None else round(ms_graph, 6),
        "append_per_step": run.appending,
        "selection": {"k": math.ceil(layer.n[0] * FRACTION), "rescanned_rows": sum(l.ws.rescans() for l in run.layers),
                      "candidates_mean": round(float(layer.ws.candidate_counts().float().mean()), 1),
                      "candidates_max": int(layer.ws.candidate_counts().max())},
        "decode_workspace_MB": round(layer.ws.bytes / 1e6, 2),
        "index_build_ms": run.layers[-1].build_ms,   # of the layer built last (kernels and allocator warm)
    }
    if args.standalone:
        result["standalone"] = standalone_kernels(layer)
    if args.calibrate_gather:
        g = run.gather_ceiling()
        result["roofline"]["random_row_ceiling_GBps"] = g["GBps"]
        result["roofline"]["random_row_probe"] = g
        # (the attention's time from the timed region where it is the dominant kernel, else from the survey)
        att_us = run.dominant_us if run.dominant == "attend" else result["kernels"]["attend"]["us"]
        if att_us > 0:   # the rows alone (the attention kernel's figure also counts the list means)
            result["roofline"]["attend_frac_of_random_row_ceiling"] = round(
                (ab["exact"] + ab["full"]) / 1e3 / att_us / g["GBps"], 4)
    copy_gbps = copy_bandwidth(device)
    result["hbm_copy_GBps"] = round(copy_gbps, 1)
    result["roofline"]["frac_of_copy"] = round(result["roofline"]["achieved"] / copy_gbps, 4)
    if result["roofline_scan"]:
        result["roofline_scan"]["frac_of_copy"] = round(result["roofline_scan"]["achieved"] / copy_gbps, 4)
    # the whole step against the same ceiling: its algorithmic bytes over the timed step
    result["step_frac_of_copy"] = round(ab["total"] / 1e3 / (ms_per_step * 1000.0) / copy_gbps, 4)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(layer, args.cpu_seconds)
    others = args.other_configs if args.other_configs is not None else args.config == 2
    if others:
        del layer
        run.close()
        result["configs"] = {}
        for cfg in (c for c in sorted(CONFIGS) if c != args.config):
            side = Timed(lib, device, cfg, layers=2, steps=args.other_steps, warmup=10, appending=False)
            side.measure(args.event_every)
            rec = side.summary()
            if not args.no_cpu and cfg in (0, 1) and not side.appending:
                side.layers[0].call.run(side.stream)           # the output the CPU pass is compared with
                torch.cuda.synchronize()
                rec["cpu_baseline"] = cpu_full_layer(side.layers[0])
                result["cpu_baseline"].setdefault("full_layers", {})[f"cfg{cfg}"] = rec["cpu_baseline"]
            result["configs"][f"cfg{cfg}"] = rec
            log(f"cfg{cfg}: {rec['us_per_layer']} us/layer, step roofline {rec['step_roofline_frac']}")
            side.close()
            del side
    maintain = args.index_maintenance if args.index_maintenance is not None else (args.config == 2 and others)
    if maintain:
        if not others:
            del layer
            run.close()
        torch.cuda.empty_cache()
        result["index_maintenance"] = index_maintenance(device)
        log(f"index maintenance: {result['index_maintenance']}")
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
