"""Single-token-decode replacement hook for vLLM's FlashAttention backend.

The state machine of the reference's benchmarks/vllm_backend/pq_hsa_decode_runtime.py, with the
same function names, environment switches, STATS keys and error conventions: ``pq_or_dense_forward``
(:790-822) gates on ``pq_enabled`` / ``should_pq_decode`` (:302-341, 356-361), and
``run_pq_decode`` (:492-716) builds a sidecar from the paged cache on the first or a
non-sequential step, appends + attends on sequential steps, restores a checkpointed prefix when
the same prompt returns (or, with ``PQ_HSA_PREFIX_EXTEND=1``, extends it when the prompt continues
it), and flushes the deferred index update every ``PQ_HSA_FLUSH_INTERVAL``
appends.  The sidecar is the MI355X batched engine (``GQASidecar``).
"""

from __future__ import annotations

import hashlib
import os
import time
from array import array
from typing import Any, Callable, Optional

import torch

from ..config import IVFPQConfig, SparseAttentionConfig
from .paged_kv_fa import flashattn_seq_len, gather_flashattn_kv

STATS: dict[str, Any] = {
    "installed": False,
    "backend": None,
    "sidecar": None,
    "pq_decode_calls": 0,
    "pq_build_calls": 0,
    "pq_append_calls": 0,
    "pq_build_s_total": 0.0,
    "pq_forward_s_total": 0.0,
    "pq_forward_only_s_total": 0.0,
    "pq_append_s_total": 0.0,
    "pq_restore_s_total": 0.0,
    "pq_cache_write_s_total": 0.0,
    "pq_gather_s_total": 0.0,
    "pq_flush_s_total": 0.0,
    "pq_flush_calls": 0,
    "pq_copy_ctx_s_total": 0.0,
    "dense_fa_s_total": 0.0,
    "dense_fa_calls": 0,
    "batched_heads_active": None,
    "cuda_graph_active": None,
    "dense_fallback_calls": 0,
    "last_error": None,
    "layers_built": 0,
    "prefix_persist_hits": 0,
    "prefix_persist_misses": 0,
    "prefix_miss_reasons": {},
    "prefix_extend_hits": 0,
    "prefix_extend_rejects": {},
    "pq_extend_s_total": 0.0,
    "pq_extend_delta_tokens_total": 0,
    "pq_extend_last": None,
    "reject": {},
    "pq_batch_steps": 0,
    "pq_batch_reqs_total": 0,
    "pq_batch_fused_steps": 0,
    "pq_batch_group_builds": 0,
    "pq_batch_regroups": 0,
    "batch_mode": False,
}

_PRESERVE_ON_RESET = ("installed", "backend", "sidecar", "batched_heads_active", "cuda_graph_active", "batch_mode")

# layer name (or impl id) -> sidecar state; survives reset_pq_hsa_runtime_stats
_LAYER_STATE: dict[Any, dict[str, Any]] = {}


def pq_hsa_runtime_stats() -> dict[str, Any]:
    return dict(STATS)


def reset_pq_hsa_runtime_stats() -> None:
    for k, v in list(STATS.items()):
        if k in _PRESERVE_ON_RESET:
            continue
        if isinstance(v, dict):
            STATS[k] = {}
        elif isinstance(v, float):
            STATS[k] = 0.0
        elif isinstance(v, (bool, int)):
            STATS[k] = 0
        else:
            STATS[k] = None


def reset_pq_hsa_layer_state() -> None:
    _LAYER_STATE.clear()


def layer_state_key(impl, layer) -> Any:
    if layer is not None:
        name = getattr(layer, "layer_name", None)
        if name is not None:
            return name
    return id(impl)


def state_for(impl, layer) -> dict[str, Any]:
    key = layer_state_key(impl, layer)
    st = _LAYER_STATE.get(key)
    if st is None:
        st = {"sidecar": None, "seq_len": None, "prefix_key": None, "appends": 0}
        _LAYER_STATE[key] = st
    return st


def sidecar_cls():
    # PQ_HSA_SIDECAR=loop|fast select two classes in the reference; both are the batched engine here
    from .gqa_sidecar import GQASidecar

    return GQASidecar


def paper_index_config() -> IVFPQConfig:
    return IVFPQConfig(
        num_lists=int(os.environ.get("PQ_HSA_NUM_LISTS", "512")),
        nprobe=int(os.environ.get("PQ_HSA_NPROBE", "64")),
        num_subspaces=int(os.environ.get("PQ_HSA_SUBSPACES", "8")),
        num_bits=int(os.environ.get("PQ_HSA_BITS", "4")),
        residual=True,
        coarse_max_iter=int(os.environ.get("PQ_HSA_COARSE_ITER", "1")),
        pq_max_iter=int(os.environ.get("PQ_HSA_PQ_ITER", "2")),
        pack_codes=True,
        topk_block_size=int(os.environ.get("PQ_HSA_TOPK_BLOCK", "1024")),
        kernel_backend=os.environ.get("PQ_HSA_KERNEL", "mi355x"),
        rotation="none",
        direction_normalize=os.environ.get("PQ_HSA_DIR_NORM", "1") == "1",
        seed=0,
    )


def paper_attention_config(scale: float) -> SparseAttentionConfig:
    return SparseAttentionConfig(
        sink_tokens=int(os.environ.get("PQ_HSA_SINK", "4")),
        local_window=int(os.environ.get("PQ_HSA_LOCAL", "128")),
        retrieval_topk=100,
        retrieval_top_fraction=float(os.environ.get("PQ_HSA_TOP_FRAC", "0.01")),
        nprobe=int(os.environ.get("PQ_HSA_NPROBE", "64")),
        candidate_budget=int(os.environ.get("PQ_HSA_CAND_BUDGET", "4096")),
        exact_rerank=True,
        scale=float(scale),
        mode="hybrid",
        hybrid_value_mode="centroid",
        hybrid_topk_source="all_pq",
        hybrid_denominator_source="all_pq",
        index_update_interval=int(os.environ.get("PQ_HSA_UPD_INTERVAL", "256")),
        index_update_strategy="deferred",
        kv_storage="device",
        collect_attention_details=False,
        profile_attention_components=False,
    )


def batch_enabled() -> bool:
    on = os.environ.get("PQ_HSA_BATCH", "0") == "1"
    STATS["batch_mode"] = on
    return on


def min_pq_seq() -> int:
    return int(os.environ.get("PQ_HSA_SINK", "4")) + int(os.environ.get("PQ_HSA_LOCAL", "128")) + 16


def reject(reason: str) -> bool:
    STATS["reject"][reason] = STATS["reject"].get(reason, 0) + 1
    return False


def host_seq_lens(attn_metadata) -> list[int]:
    """The batch's sequence lengths as host integers.  Reading them from the device waits for the
    GPU, so the list is taken from a host copy when the metadata carries one and is kept on the
    metadata object: every layer of a step gets the same object."""
    cached = getattr(attn_metadata, "_pq_host_seq_lens", None)
    if cached is not None:
        return cached
    src = getattr(attn_metadata, "seq_lens_cpu", None)
    if src is None:
        src = attn_metadata.seq_lens
    lens = [int(x) for x in src.tolist()]
    try:
        attn_metadata._pq_host_seq_lens = lens
    except Exception:
        pass
    return lens


def host_first_blocks(attn_metadata) -> list[int]:
    """First physical block of every request of the batch, as host integers: what tells one
    request from another while it lives (vLLM moves requests between batch rows when one
    finishes).  Read once per step and kept on the metadata object, like the lengths."""
    cached = getattr(attn_metadata, "_pq_host_first_blocks", None)
    if cached is not None:
        return cached
    first = [int(x) for x in attn_metadata.block_table[:, 0].tolist()]
    try:
        attn_metadata._pq_host_first_blocks = first
    except Exception:
        pass
    return first


def should_pq_decode(attn_metadata) -> bool:
    if attn_metadata is None:
        return reject("no_metadata")
    if getattr(attn_metadata, "use_cascade", False):
        return reject("cascade")
    if int(getattr(attn_metadata, "max_query_len", 0)) != 1:
        return reject("max_query_len!=1")
    seq_lens = getattr(attn_metadata, "seq_lens", None)
    if batch_enabled():
        if seq_lens is None or int(seq_lens.shape[0]) < 1:
            return reject("num_reqs<1")
        if int(getattr(attn_metadata, "num_actual_tokens", 0)) != int(seq_lens.shape[0]):
            return reject("num_actual_tokens!=num_reqs")
        if min(host_seq_lens(attn_metadata)) < min_pq_seq():
            return reject("seq_too_short")
        return True
    if int(getattr(attn_metadata, "num_actual_tokens", 0)) != 1:
        return reject("num_actual_tokens!=1")
    if seq_lens is None or int(seq_lens.shape[0]) != 1:
        return reject("num_reqs!=1")
    if flashattn_seq_len(attn_metadata, 0) < min_pq_seq():
        return reject("seq_too_short")
    return True


def flush_interval() -> int:
    return int(os.environ.get("PQ_HSA_FLUSH_INTERVAL", "256"))


def pq_enabled() -> bool:
    return os.environ.get("PQ_HSA_ENABLE", "0") == "1"


def flush_sidecar(adapter) -> None:
    fn = getattr(adapter, "apply_pending_index_update", None)
    if fn is not None:
        fn()


def as_decode_qkv(t: torch.Tensor) -> torch.Tensor:
    if t.ndim == 3:
        return t[:1]
    if t.ndim == 2:
        return t[:1].unsqueeze(0)
    raise ValueError(f"expected [T,H,D] or [T,D], got {tuple(t.shape)}")


def copy_ctx(output: torch.Tensor, ctx: torch.Tensor, num_actual: int) -> None:
    dst = output[:num_actual]
    if ctx.shape != dst.shape:
        ctx = ctx.reshape(dst.shape)
    if ctx.dtype != dst.dtype:
        ctx = ctx.to(dtype=dst.dtype)
    dst.copy_(ctx)


def prefix_cache_key(attn_metadata, seq_len: int):
    cached = getattr(attn_metadata, "_pq_prefix_cache_key", None)
    if cached is not None:
        return cached
    runner = getattr(attn_metadata, "_pq_runner", None)
    if runner is None:
        return None
    req_ids = runner.input_batch.req_ids
    if not req_ids:
        return None
    request = runner.requests.get(req_ids[0])
    prompt_ids = None if request is None else request.prompt_token_ids
    if prompt_ids is None:
        return None
    context_len = int(seq_len) - int(attn_metadata.max_query_len)
    digest = hashlib.blake2b(array("I", prompt_ids).tobytes(), digest_size=16).digest()
    key = (context_len, digest)
    try:
        attn_metadata._pq_prefix_cache_key = key
    except Exception:
        pass
    return key


def _prefix_extend_enabled() -> bool:
    """``PQ_HSA_PREFIX_EXTEND=1``: when a request's prompt continues the checkpointed one, restore the
    index and take in only the added tokens instead of rebuilding (runtime.py:425-428).  Off by default."""
    return os.environ.get("PQ_HSA_PREFIX_EXTEND", "0") == "1"


def _prefix_extend_max_frac() -> float:
    try:
        return float(os.environ.get("PQ_HSA_PREFIX_EXTEND_MAX_FRAC", "0.5"))
    except ValueError:
        return 0.5


def prefix_extend_match(attn_metadata, old_key, checkpoint_len, seq_len: int):
    """Does the current request's prompt strictly extend the checkpointed prompt?  ``old_key`` is the
    ``(context_len, digest)`` stored with the checkpoint, ``checkpoint_len`` the sidecar's length at
    that time (prompt + the first decode token).  Returns ``(ok, reason, new_key, delta_tokens)``
    with the reference's reasons (runtime.py:438-488).  The digest of the new prompt's first
    ``context_len`` ids is kept on the metadata object, so the layers of one step hash it once."""
    if old_key is None or checkpoint_len is None:
        return False, "no_checkpoint", None, 0
    old_ctx, old_digest = int(old_key[0]), old_key[1]
    checkpoint_len = int(checkpoint_len)
    if checkpoint_len != old_ctx + 1:
        return False, "checkpoint_inconsistent", None, 0
    context_len = int(seq_len) - int(attn_metadata.max_query_len)
    delta = int(seq_len) - checkpoint_len
    if context_len <= old_ctx or delta <= 0:
        return False, "not_longer", None, 0
    if float(delta) / float(seq_len) > _prefix_extend_max_frac():
        return False, "delta_too_large", None, delta
    digests = getattr(attn_metadata, "_pq_prefix_ext_digests", None)
    if digests is None:
        digests = {}
        try:
            attn_metadata._pq_prefix_ext_digests = digests
        except Exception:
            pass
    d = digests.get(old_ctx)
    if d is None:
        runner = getattr(attn_metadata, "_pq_runner", None)
        if runner is None:
            return False, "no_runner", None, delta
        req_ids = runner.input_batch.req_ids
        if not req_ids:
            return False, "no_request", None, delta
        request = runner.requests.get(req_ids[0])
        prompt_ids = None if request is None else request.prompt_token_ids
        if prompt_ids is None or len(prompt_ids) != context_len:
            return False, "prompt_len_mismatch", None, delta
        d = hashlib.blake2b(array("I", prompt_ids[:old_ctx]).tobytes(), digest_size=16).digest()
        digests[old_ctx] = d
    if d != old_digest:
        return False, "prefix_digest_mismatch", None, delta
    new_key = prefix_cache_key(attn_metadata, seq_len)
    if new_key is None:
        return False, "no_prefix_key", None, delta
    return True, "ok", new_key, delta


def _build_sidecar(impl, kv_cache, attn_metadata, seq_idx: int):
    t_g = time.perf_counter()
    keys, values, gathered = gather_flashattn_kv(kv_cache, attn_metadata, seq_idx)
    STATS["pq_gather_s_total"] += time.perf_counter() - t_g
    t0 = time.perf_counter()
    adapter = sidecar_cls()(paper_index_config(), paper_attention_config(impl.scale),
                            num_query_heads=impl.num_heads, num_kv_heads=impl.num_kv_heads).build_cache(keys, values)
    adapter.set_paged_kv_context(kv_cache, attn_metadata, seq_idx)
    STATS["pq_build_s_total"] += time.perf_counter() - t0
    STATS["pq_build_calls"] += 1
    STATS["layers_built"] = int(STATS["layers_built"]) + 1
    STATS["batched_heads_active"] = getattr(adapter, "batched_heads_active", None)
    STATS["sidecar"] = type(adapter).__name__
    return adapter, gathered


def run_pq_decode(impl, layer, query, key, value, kv_cache, attn_metadata) -> torch.Tensor:
    """Build / append / restore / flush the layer's sidecar and return the context ``[1, Hq, D]``."""
    st = state_for(impl, layer)
    seq_len = flashattn_seq_len(attn_metadata, 0)
    prev, adapter = st["seq_len"], st["sidecar"]
    sequential = adapter is not None and prev is not None and seq_len == int(prev) + 1
    q = as_decode_qkv(query)
    if not sequential:
        pkey = prefix_cache_key(attn_metadata, seq_len)
        checkpoint_len = getattr(adapter, "prefix_checkpoint_length", None)
        can_restore = (adapter is not None and pkey is not None and pkey == st["prefix_key"]
                       and checkpoint_len is not None and int(checkpoint_len) == seq_len)
        if can_restore:
            t_restore = time.perf_counter()
            restored = adapter.restore_prefix(as_decode_qkv(key), as_decode_qkv(value), kv_cache=kv_cache,
                                              attn_metadata=attn_metadata, seq_idx=0)
            if not restored:
                raise RuntimeError("prefix sidecar checkpoint disappeared during restore")
            STATS["pq_restore_s_total"] += time.perf_counter() - t_restore
            STATS["prefix_persist_hits"] += 1
            st["seq_len"], st["appends"] = seq_len, 0
            t_forward = time.perf_counter()
            ctx = adapter.forward(q)
            STATS["pq_forward_only_s_total"] += time.perf_counter() - t_forward
            STATS["pq_decode_calls"] += 1
            return ctx
        if _prefix_extend_enabled() and adapter is not None and hasattr(adapter, "extend_prefix"):
            ok, why, new_key, delta = prefix_extend_match(attn_metadata, st["prefix_key"], checkpoint_len, seq_len)
            if ok:
                t_ext = time.perf_counter()
                info = adapter.extend_prefix(as_decode_qkv(key), as_decode_qkv(value), kv_cache=kv_cache,
                                             attn_metadata=attn_metadata, seq_idx=0, new_length=seq_len)
                ext_s = time.perf_counter() - t_ext
                if info is None:
                    why = "adapter_declined"
                else:
                    STATS["pq_extend_s_total"] += ext_s
                    STATS["prefix_extend_hits"] += 1
                    STATS["pq_extend_delta_tokens_total"] = int(STATS["pq_extend_delta_tokens_total"]) + int(delta)
                    STATS["pq_extend_last"] = dict(info, wall_s=ext_s)
                    st.update(prefix_key=new_key, seq_len=seq_len, appends=0)
                    t_forward = time.perf_counter()
                    ctx = adapter.forward(q)
                    forward_s = time.perf_counter() - t_forward
                    STATS["pq_forward_only_s_total"] += forward_s
                    STATS["pq_forward_s_total"] += ext_s + forward_s
                    adapter.checkpoint_prefix()          # the next turn may extend this one
                    STATS["pq_decode_calls"] += 1
                    return ctx
            rej = STATS["prefix_extend_rejects"]
            rej[why] = rej.get(why, 0) + 1
        STATS["prefix_persist_misses"] += 1
        if adapter is None:
            reason = "no_adapter"
        elif pkey is None:
            reason = "no_prefix_key"
        elif pkey != st["prefix_key"]:
            reason = "prefix_key_mismatch"
        else:
            reason = "checkpoint_length_mismatch"
        STATS["prefix_miss_reasons"][reason] = STATS["prefix_miss_reasons"].get(reason, 0) + 1
        adapter, gathered = _build_sidecar(impl, kv_cache, attn_metadata, 0)
        if gathered != seq_len:
            raise RuntimeError(f"gather seq {gathered} != metadata seq {seq_len}")
        st.update(sidecar=adapter, prefix_key=pkey, seq_len=seq_len, appends=0)
        t1 = time.perf_counter()
        ctx = adapter.forward(q)
        dt = time.perf_counter() - t1
        STATS["pq_forward_s_total"] += dt
        STATS["pq_forward_only_s_total"] += dt
        adapter.checkpoint_prefix()
        STATS["cuda_graph_active"] = getattr(adapter, "cuda_graph_active", None)
    else:
        adapter.set_paged_kv_context(kv_cache, attn_metadata, 0)
        t_append = time.perf_counter()
        adapter.append(as_decode_qkv(key), as_decode_qkv(value))
        append_s = time.perf_counter() - t_append
        t_forward = time.perf_counter()
        ctx = adapter.forward(q)
        forward_s = time.perf_counter() - t_forward
        STATS["pq_append_s_total"] += append_s
        STATS["pq_forward_only_s_total"] += forward_s
        STATS["pq_forward_s_total"] += append_s + forward_s
        STATS["pq_append_calls"] += 1
        st["seq_len"] = seq_len
        st["appends"] = int(st["appends"]) + 1
        interval = flush_interval()
        if interval > 0 and st["appends"] % interval == 0:
            t2 = time.perf_counter()
            flush_sidecar(adapter)
            STATS["pq_flush_s_total"] += time.perf_counter() - t2
            STATS["pq_flush_calls"] += 1
    STATS["pq_decode_calls"] += 1
    return ctx


def batch_fused() -> bool:
    """``PQ_HSA_BATCH_FUSED`` (default on): the requests of a decode batch share one engine and one
    kernel sequence per layer; ``0`` keeps one sidecar per request, as the reference does."""
    return os.environ.get("PQ_HSA_BATCH_FUSED", "1") == "1"


def _int32_table(attn_metadata, num_reqs: int) -> torch.Tensor:
    table = attn_metadata.block_table[:num_reqs]
    if table.dtype != torch.int32 or not table.is_contiguous():
        table = table.to(torch.int32).contiguous()
    return table


def run_pq_decode_group(impl, layer, query, key, value, kv_cache, attn_metadata, output) -> torch.Tensor:
    """All requests of the decode batch through one engine: the step's appends ride on the decode
    launches and every sequence, KV head and query row is served by the same six kernels.
    Requests are told apart by their first physical block.  When the batch is the previous one
    advanced by one token each, the step is one call; when requests left, joined or changed rows,
    the index rows of those that continue are copied into a new group (nothing is re-encoded)
    and only the newcomers are built."""
    from ..attention.engine import PQHSAEngine

    st = state_for(impl, layer)
    num_reqs = int(attn_metadata.seq_lens.shape[0])
    lens = list(host_seq_lens(attn_metadata))[:num_reqs]
    ids = list(host_first_blocks(attn_metadata))[:num_reqs]
    grp = st.get("group")
    table = _int32_table(attn_metadata, num_reqs)
    steady = (grp is not None and grp["ids"] == ids
              and all(now == before + 1 for now, before in zip(lens, grp["lens"])))
    if steady:
        eng = grp["engine"]
        eng.bind_paged(kv_cache, table)      # the block table may have grown
        eng.advance(1)
        grp["lens"], grp["appends"] = lens, grp["appends"] + 1
        STATS["pq_append_calls"] += 1
    else:
        t0 = time.perf_counter()
        where = {rid: j for j, rid in enumerate(grp["ids"])} if grp is not None else {}
        going_on = [where.get(ids[r]) if where.get(ids[r]) is not None and lens[r] == grp["lens"][where[ids[r]]] + 1
                    else None for r in range(num_reqs)]
        fresh = [r for r in range(num_reqs) if going_on[r] is None]
        newcomers = None
        if fresh:
            newcomers = PQHSAEngine(paper_index_config(), paper_attention_config(impl.scale), batch=len(fresh),
                                    kv_heads=impl.num_kv_heads, device=kv_cache.device)
            newcomers.bind_paged(kv_cache, table[fresh].contiguous())
            newcomers.build([lens[r] for r in fresh])
            STATS["pq_build_calls"] += 1
        if len(fresh) == num_reqs:
            eng = newcomers
            STATS["pq_batch_group_builds"] += 1
        else:
            sources = [(newcomers, fresh.index(r)) if going_on[r] is None else (grp["engine"], going_on[r])
                       for r in range(num_reqs)]
            eng = PQHSAEngine.regroup(sources)
            STATS["pq_batch_regroups"] += 1
        eng.bind_paged(kv_cache, table)
        staying = [r for r in range(num_reqs) if going_on[r] is not None]
        if staying:
            eng.advance(1, which=staying)     # their new token is indexed by the step below
            STATS["pq_append_calls"] += 1
        grp = st["group"] = {"engine": eng, "lens": lens, "ids": ids,
                             "appends": (grp["appends"] + 1) if (grp is not None and staying) else 0}
        STATS["pq_build_s_total"] += time.perf_counter() - t0
        STATS["sidecar"] = "PQHSAEngine"
    q, dst = query[:num_reqs], output[:num_reqs]
    groups = impl.num_heads // impl.num_kv_heads
    if dst.shape == q.shape and dst.dtype == q.dtype == kv_cache.dtype and dst.is_contiguous():
        eng.forward(q, groups, out=dst)                      # straight into vLLM's output buffer
    else:
        copy_ctx(output, eng.forward(q, groups), num_reqs)
    if grp["appends"] > 0 and flush_interval() > 0 and grp["appends"] % flush_interval() == 0:
        t1 = time.perf_counter()
        eng.apply_pending_index_update()
        STATS["pq_flush_s_total"] += time.perf_counter() - t1
        STATS["pq_flush_calls"] += 1
    STATS["pq_batch_steps"] += 1
    STATS["pq_batch_fused_steps"] += 1
    STATS["pq_batch_reqs_total"] += num_reqs
    STATS["pq_decode_calls"] += 1
    return output


def run_pq_decode_batch(impl, layer, query, key, value, kv_cache, attn_metadata, output) -> torch.Tensor:
    """``PQ_HSA_BATCH=1``: one sidecar per request of the decode batch
    (benchmarks/vllm_backend/pq_hsa_batch_decode.py:383-432 of the reference), or, by default,
    one engine for the whole batch (``batch_fused``)."""
    if batch_fused():
        return run_pq_decode_group(impl, layer, query, key, value, kv_cache, attn_metadata, output)
    st = state_for(impl, layer)
    per_req = st.setdefault("batch", {})
    num_reqs = int(attn_metadata.seq_lens.shape[0])
    lens = list(host_seq_lens(attn_metadata))
    for r in range(num_reqs):
        rs = per_req.get(r)
        sequential = rs is not None and lens[r] == rs["seq_len"] + 1
        if not sequential:
            adapter, _ = _build_sidecar(impl, kv_cache, attn_metadata, r)
            rs = per_req[r] = {"sidecar": adapter, "seq_len": lens[r], "appends": 0}
        else:
            adapter = rs["sidecar"]
            adapter.set_paged_kv_context(kv_cache, attn_metadata, r)
            adapter.append(key[r : r + 1], value[r : r + 1])
            rs["seq_len"], rs["appends"] = lens[r], rs["appends"] + 1
            if flush_interval() > 0 and rs["appends"] % flush_interval() == 0:
                flush_sidecar(adapter)
        ctx = adapter.forward(query[r : r + 1])
        copy_ctx(output[r : r + 1], ctx, 1)
    for stale in [r for r in per_req if r >= num_reqs]:
        del per_req[stale]
    STATS["pq_batch_steps"] += 1
    STATS["pq_batch_reqs_total"] += num_reqs
    STATS["pq_decode_calls"] += 1
    return output


def write_kv_to_cache(key, value, kv_cache, attn_metadata, impl=None, layer=None) -> None:
    """This step's K/V rows -> their paged slots (5-D layout; vLLM >= 0.10 writes the 4-D layout
    itself before calling forward).  Uses vLLM's cache op when it is loaded."""
    if kv_cache.dim() != 5:
        return
    key_cache, value_cache = kv_cache.unbind(0)
    op = getattr(getattr(torch.ops, "_C_cache_ops", None), "reshape_and_cache_flash", None)
    if op is not None and impl is not None and layer is not None:
        op(key, value, key_cache, value_cache, attn_metadata.slot_mapping, impl.kv_cache_dtype, layer._k_scale,
           layer._v_scale)
        return
    slots = attn_metadata.slot_mapping[: key.shape[0]].long()
    block_size = key_cache.shape[1]
    key_cache[slots // block_size, slots % block_size] = key.to(key_cache.dtype)
    value_cache[slots // block_size, slots % block_size] = value.to(value_cache.dtype)


def run_pq_decode_into_output(impl, layer, query, key, value, kv_cache, attn_metadata, output) -> torch.Tensor:
    t_cache = time.perf_counter()
    write_kv_to_cache(key, value, kv_cache, attn_metadata, impl, layer)
    STATS["pq_cache_write_s_total"] += time.perf_counter() - t_cache
    if batch_enabled():
        return run_pq_decode_batch(impl, layer, query, key, value, kv_cache, attn_metadata, output)
    ctx = run_pq_decode(impl, layer, query, key, value, kv_cache, attn_metadata)
    t_copy = time.perf_counter()
    copy_ctx(output, ctx, 1)
    STATS["pq_copy_ctx_s_total"] += time.perf_counter() - t_copy
    return output


def pq_or_dense_forward(impl, layer, query, key, value, kv_cache, attn_metadata, output: Optional[torch.Tensor],
                        dense_forward: Callable[[], torch.Tensor]) -> torch.Tensor:
    if (not pq_enabled()) or not should_pq_decode(attn_metadata):
        t_dense = time.perf_counter()
        out = dense_forward()
        STATS["dense_fa_s_total"] += time.perf_counter() - t_dense
        STATS["dense_fa_calls"] = int(STATS["dense_fa_calls"]) + 1
        return out
    allow_fallback = os.environ.get("PQ_HSA_FALLBACK", "0") == "1"
    try:
        assert output is not None
        return run_pq_decode_into_output(impl, layer, query, key, value, kv_cache, attn_metadata, output)
    except Exception as exc:
        STATS["last_error"] = f"{type(exc).__name__}: {exc}"
        STATS["dense_fallback_calls"] += 1
        if not allow_fallback:
            raise
        return dense_forward()
