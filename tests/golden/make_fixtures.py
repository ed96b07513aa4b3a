"""Write golden input/output vectors from the real reference implementation.

Run ONCE in the build container (the reference tree is not present anywhere else):

    python tests/golden/make_fixtures.py

It imports the reference's CPU torch path (``kernel_backend="torch"``) from
``/root/reference`` and records, for two small seeded cases, what the reference produces
for the parts of the decode path whose bit-level behaviour no closed form pins: the list
assignment and PQ codes chosen by its ``cdist``/``argmin`` encode, the key norms, the
approximate scores, the ``torch.topk`` selection and the hybrid attention output, before and
after incremental appends.  Only data (inputs and outputs) is written, as ``.npz`` files next
to this script.
"""

from __future__ import annotations

import math
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, REPO)
sys.path.insert(0, "/root/reference")

from pqhsa_release_amd.synth import make_head  # noqa: E402

from pq_hsa.attention.sparse_attention import (  # noqa: E402
    IVFPQSparseAttention,
    SparseAttentionConfig,
)
from pq_hsa.index.ivfpq import IVFPQConfig, IVFPQIndex  # noqa: E402
from benchmarks.vllm_backend.gqa_sidecar import GQASidecar  # noqa: E402


def index_config(num_lists: int) -> IVFPQConfig:
    return IVFPQConfig(
        num_lists=num_lists,
        nprobe=8,
        num_subspaces=8,
        num_bits=4,
        residual=True,
        coarse_max_iter=1,
        pq_max_iter=2,
        pack_codes=True,
        kernel_backend="torch",
        rotation="none",
        direction_normalize=True,
        seed=0,
    )


def attention_config(fraction: float, *, sink: int = 4, local: int = 64, strategy: str = "incremental",
                     interval: int = 1) -> SparseAttentionConfig:
    return SparseAttentionConfig(
        sink_tokens=sink,
        local_window=local,
        retrieval_top_fraction=fraction,
        exact_rerank=True,
        scale=None,
        mode="hybrid",
        hybrid_value_mode="centroid",
        hybrid_topk_source="all_pq",
        hybrid_denominator_source="all_pq",
        index_update_interval=interval,
        index_update_strategy=strategy,
        collect_attention_details=False,
    )


def np32(t: torch.Tensor) -> np.ndarray:
    return t.detach().to(torch.float32).cpu().numpy()


def snapshot(stream: IVFPQSparseAttention) -> dict[str, np.ndarray]:
    cache = stream.cache
    index = cache.index
    return {
        "list_ids": index.list_ids.to(torch.int32).numpy().astype(np.uint16),
        "packed": index.packed_codes.numpy().copy(),
        "norms": np32(index.key_norms),
        "vbar": np32(cache.retrieval_value_centroids),
    }


def make_case(name: str, *, ctx: int, heads: int, groups: int, num_lists: int, fraction: float,
              bf16: bool, steps: int, seed0: int) -> None:
    out: dict[str, np.ndarray] = {}
    dim = 128
    icfg = index_config(num_lists)
    acfg = attention_config(fraction)
    keys, values, queries = [], [], []
    for h in range(heads):
        k, v, q = make_head(ctx + steps, dim=dim, groups=groups * (steps + 1), seed=seed0 + h,
                            num_clusters=num_lists)
        if bf16:
            k = k.to(torch.bfloat16).float()
            v = v.to(torch.bfloat16).float()
            q = q.to(torch.bfloat16).float()
        keys.append(k)
        values.append(v)
        queries.append(q.reshape(steps + 1, groups, dim))
    keys_t = torch.stack(keys)            # [H, ctx+steps, D]
    values_t = torch.stack(values)
    queries_t = torch.stack(queries)      # [H, steps+1, G, D]
    out["keys"] = np32(keys_t)
    out["values"] = np32(values_t)
    out["queries"] = np32(queries_t)
    out["meta"] = np.array([ctx, heads, groups, num_lists, steps, acfg.sink_tokens,
                            acfg.local_window], dtype=np.int64)
    out["fraction"] = np.array([fraction], dtype=np.float64)

    sidecar = GQASidecar(icfg, acfg, num_query_heads=heads * groups, num_kv_heads=heads)
    sidecar.build_cache(keys_t[None, :, :ctx], values_t[None, :, :ctx])

    coarse, books = [], []
    for h, stream in enumerate(sidecar.streams):
        index = stream.cache.index
        coarse.append(np32(index.coarse_centroids))
        books.append(np32(index.pq.codebooks))
    out["coarse"] = np.stack(coarse)
    out["codebooks"] = np.stack(books)

    def record(tag: str, step: int) -> None:
        snaps = [snapshot(s) for s in sidecar.streams]
        for key in snaps[0]:
            out[f"{tag}_{key}"] = np.stack([s[key] for s in snaps])
        raw, top_idx, top_val = [], [], []
        for h, stream in enumerate(sidecar.streams):
            q = queries_t[h, step]
            scores = stream.cache.index.approximate_scores(q)        # [G, N]
            raw.append(np32(scores))
            n = scores.shape[1]
            k = min(max(int(math.ceil(n * fraction)), 0), n)
            logits = scores * (1.0 / math.sqrt(dim))
            vals, idx = torch.topk(logits, k=k, dim=1, sorted=True)
            top_idx.append(idx.numpy().astype(np.int32))
            top_val.append(np32(vals))
        out[f"{tag}_scores"] = np.stack(raw)
        out[f"{tag}_topk_idx"] = np.stack(top_idx)
        out[f"{tag}_topk_logit"] = np.stack(top_val)
        q_all = queries_t[:, step].reshape(1, heads * groups, dim)
        out[f"{tag}_output"] = np32(sidecar.forward(q_all))[0]      # [H*G, D]
        # the single-query path of the reference must agree with forward_many
        single = sidecar.streams[0].forward(queries_t[0, step, 0]).output
        out[f"{tag}_output_single_h0g0"] = np32(single)

    record("build", 0)
    for step in range(1, steps + 1):
        pos = ctx + step - 1
        sidecar.append(keys_t[None, :, pos], values_t[None, :, pos])
    if steps > 0:
        record("append", steps)

    # the "identical trained index" entry point: encode other keys with the same codebooks
    other, _, _ = make_head(300, dim=dim, groups=1, seed=seed0 + 77, num_clusters=num_lists)
    if bf16:
        other = other.to(torch.bfloat16).float()
    shared = IVFPQIndex(icfg).build_with_codebooks(
        other,
        coarse_centroids=torch.from_numpy(out["coarse"][0]),
        pq_codebooks=torch.from_numpy(out["codebooks"][0]),
    )
    out["shared_keys"] = np32(other)
    out["shared_list_ids"] = shared.list_ids.to(torch.int32).numpy().astype(np.uint16)
    out["shared_packed"] = shared.packed_codes.numpy().copy()
    out["shared_norms"] = np32(shared.key_norms)

    path = os.path.join(HERE, f"{name}.npz")
    np.savez_compressed(path, **out)
    print(name, {k: v.shape for k, v in out.items()}, os.path.getsize(path), "bytes")


def make_deferred_case(name: str, *, ctx: int, heads: int, groups: int, num_lists: int, fraction: float,
                       added: int, seed0: int) -> None:
    """The deferred update strategy: ``added`` keys are appended without touching the index, then
    ``apply_pending_index_update`` runs the reference's online refresh (EMA move of the coarse
    centroids and PQ codewords, full re-encode, rebuilt value means).  Recorded: the trained index
    before, everything the flush produces, and the attention output before and after it."""
    out: dict[str, np.ndarray] = {}
    dim = 128
    icfg = index_config(num_lists)
    acfg = attention_config(fraction, strategy="deferred", interval=8)
    keys, values, queries = [], [], []
    for h in range(heads):
        k, v, q = make_head(ctx + added, dim=dim, groups=groups, seed=seed0 + h, num_clusters=num_lists)
        k, v, q = k.to(torch.bfloat16).float(), v.to(torch.bfloat16).float(), q.to(torch.bfloat16).float()
        keys.append(k)
        values.append(v)
        queries.append(q)
    keys_t, values_t, queries_t = torch.stack(keys), torch.stack(values), torch.stack(queries)
    out["keys"], out["values"], out["queries"] = np32(keys_t), np32(values_t), np32(queries_t)
    out["meta"] = np.array([ctx, heads, groups, num_lists, added, acfg.sink_tokens, acfg.local_window],
                           dtype=np.int64)
    out["fraction"] = np.array([fraction], dtype=np.float64)
    out["lr"] = np.array([icfg.online_codebook_lr], dtype=np.float64)
    sidecar = GQASidecar(icfg, acfg, num_query_heads=heads * groups, num_kv_heads=heads)
    sidecar.build_cache(keys_t[None, :, :ctx], values_t[None, :, :ctx])

    def tables(tag: str) -> None:
        out[f"{tag}_coarse"] = np.stack([np32(s.cache.index.coarse_centroids) for s in sidecar.streams])
        out[f"{tag}_codebooks"] = np.stack([np32(s.cache.index.pq.codebooks) for s in sidecar.streams])
        snaps = [snapshot(s) for s in sidecar.streams]
        for key in snaps[0]:
            out[f"{tag}_{key}"] = np.stack([s[key] for s in snaps])

    tables("build")
    for i in range(added):
        sidecar.append(keys_t[None, :, ctx + i], values_t[None, :, ctx + i])
    q_all = queries_t.reshape(1, heads * groups, dim)
    assert all(s.cache.index.num_vectors == ctx - 4 - 64 for s in sidecar.streams)   # nothing indexed yet
    out["pending_output"] = np32(sidecar.forward(q_all))[0]
    flushed = [s.cache.apply_pending_index_update() for s in sidecar.streams]
    assert all(flushed)
    tables("flush")
    out["flush_output"] = np32(sidecar.forward(q_all))[0]
    path = os.path.join(HERE, f"{name}.npz")
    np.savez_compressed(path, **out)
    print(name, {k: v.shape for k, v in out.items()}, os.path.getsize(path), "bytes")


def main() -> None:
    torch.manual_seed(0)
    torch.set_num_threads(4)
    make_case("ref_fp32_h1", ctx=768, heads=1, groups=1, num_lists=64, fraction=0.02,
              bf16=False, steps=6, seed0=11)
    make_case("ref_bf16_gqa", ctx=640, heads=2, groups=4, num_lists=48, fraction=0.05,
              bf16=True, steps=4, seed0=23)
    make_deferred_case("ref_deferred_flush", ctx=900, heads=2, groups=2, num_lists=32, fraction=0.03,
                       added=24, seed0=41)


if __name__ == "__main__":
    main()
