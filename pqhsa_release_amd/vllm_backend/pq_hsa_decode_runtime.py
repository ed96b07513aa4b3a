"""Single-token-decode replacement hook for vLLM's FlashAttention backend.

The public surface is that of the reference's benchmarks/vllm_backend/pq_hsa_decode_runtime.py:
the same function names, ``PQ_HSA_*`` environment switches, ``STATS`` keys, reject / miss reason
strings and error convention, so a deployment script written against the reference reads the same
counters here.  The control flow is this module's own:

* ``should_pq_decode`` walks a table of (reason, test) pairs and counts the first that fails.
* Each layer's sidecar is driven by an explicit transition: ``plan_step`` looks at the layer's
  state and the step's metadata and names one ``Move`` (APPEND, RESTORE, EXTEND or BUILD) with
  the reasons that go into the counters; ``run_pq_decode`` executes the move.  A move that the
  sidecar declines (EXTEND) falls through to BUILD.
* ``PQ_HSA_BATCH=1`` serves a decode batch: by default all requests through one batched engine
  whose step appends and attends in the same launches (``run_pq_decode_group``), or with
  ``PQ_HSA_BATCH_FUSED=0`` one sidecar per batch row as the reference does.

Reference entry points mirrored: pq_or_dense_forward (:790-822), should_pq_decode (:302-341),
run_pq_decode (:492-716), prefix_cache_key / prefix_extend_match (:395-488), the per-request batch
loop (benchmarks/vllm_backend/pq_hsa_batch_decode.py:383-432).
"""

from __future__ import annotations

import contextlib
import dataclasses
import enum
import hashlib
import os
import time
from array import array
from typing import Any, Callable, Optional

import torch

from ..config import IVFPQConfig, SparseAttentionConfig
from .paged_kv_fa import flashattn_seq_len, gather_flashattn_kv, kv_cache_dims

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

# what describes the installation rather than the traffic: kept by reset_pq_hsa_runtime_stats
_STICKY = frozenset({"installed", "backend", "sidecar", "batched_heads_active", "cuda_graph_active", "batch_mode"})
_BLANK = {dict: dict, float: float, bool: int, int: int}


# ---------------------------------------------------------------------------- small helpers
def _env_int(name: str, default: int) -> int:
    return int(os.environ.get(name, str(default)))


def _env_on(name: str, default: str = "0") -> bool:
    return os.environ.get(name, default) == "1"


@contextlib.contextmanager
def _charge(*keys: str):
    """Add the wall time of the block to every STATS total named."""
    started = time.perf_counter()
    yield
    spent = time.perf_counter() - started
    for k in keys:
        STATS[k] += spent


def _tally(table: str, reason: str) -> None:
    STATS[table][reason] = STATS[table].get(reason, 0) + 1


def _memo(obj, attr: str, make: Callable[[], Any]):
    """``make()`` once per metadata object: every layer of a step is handed the same object, so
    host copies and digests are made by the first layer only.  Objects that refuse attributes
    simply recompute."""
    got = getattr(obj, attr, None)
    if got is None:
        got = make()
        with contextlib.suppress(Exception):
            setattr(obj, attr, got)
    return got


# ---------------------------------------------------------------------------- counters and state
def pq_hsa_runtime_stats() -> dict[str, Any]:
    return dict(STATS)


def reset_pq_hsa_runtime_stats() -> None:
    for key in STATS.keys() - _STICKY:
        blank = _BLANK.get(type(STATS[key]))
        STATS[key] = blank() if blank else None


# layer name (or impl id) -> state of that layer's sidecar; survives reset_pq_hsa_runtime_stats
_LAYER_STATE: dict[Any, dict[str, Any]] = {}


def reset_pq_hsa_layer_state() -> None:
    _LAYER_STATE.clear()


def layer_state_key(impl, layer) -> Any:
    name = getattr(layer, "layer_name", None) if layer is not None else None
    return id(impl) if name is None else name


def state_for(impl, layer) -> dict[str, Any]:
    return _LAYER_STATE.setdefault(layer_state_key(impl, layer),
                                   {"sidecar": None, "seq_len": None, "prefix_key": None, "appends": 0})


# ---------------------------------------------------------------------------- configuration
def sidecar_cls():
    # PQ_HSA_SIDECAR=loop|fast select two classes in the reference; both are the batched engine here
    from .gqa_sidecar import GQASidecar

    return GQASidecar


def paper_index_config() -> IVFPQConfig:
    return IVFPQConfig(
        num_lists=_env_int("PQ_HSA_NUM_LISTS", 512),
        nprobe=_env_int("PQ_HSA_NPROBE", 64),
        num_subspaces=_env_int("PQ_HSA_SUBSPACES", 8),
        num_bits=_env_int("PQ_HSA_BITS", 4),
        residual=True,
        coarse_max_iter=_env_int("PQ_HSA_COARSE_ITER", 1),
        pq_max_iter=_env_int("PQ_HSA_PQ_ITER", 2),
        pack_codes=True,
        topk_block_size=_env_int("PQ_HSA_TOPK_BLOCK", 1024),
        kernel_backend=os.environ.get("PQ_HSA_KERNEL", "mi355x"),
        rotation="none",
        direction_normalize=_env_on("PQ_HSA_DIR_NORM", "1"),
        seed=0,
    )


def paper_attention_config(scale: float) -> SparseAttentionConfig:
    return SparseAttentionConfig(
        sink_tokens=_env_int("PQ_HSA_SINK", 4),
        local_window=_env_int("PQ_HSA_LOCAL", 128),
        retrieval_topk=100,
        retrieval_top_fraction=float(os.environ.get("PQ_HSA_TOP_FRAC", "0.01")),
        nprobe=_env_int("PQ_HSA_NPROBE", 64),
        candidate_budget=_env_int("PQ_HSA_CAND_BUDGET", 4096),
        exact_rerank=True,
        scale=float(scale),
        mode="hybrid",
        hybrid_value_mode="centroid",
        hybrid_topk_source="all_pq",
        hybrid_denominator_source="all_pq",
        index_update_interval=_env_int("PQ_HSA_UPD_INTERVAL", 256),
        index_update_strategy="deferred",
        kv_storage="device",
        collect_attention_details=False,
        profile_attention_components=False,
    )


def pq_enabled() -> bool:
    return _env_on("PQ_HSA_ENABLE")


def batch_enabled() -> bool:
    STATS["batch_mode"] = _env_on("PQ_HSA_BATCH")
    return STATS["batch_mode"]


def batch_fused() -> bool:
    """``PQ_HSA_BATCH_FUSED`` (default on): the requests of a decode batch share one engine and one
    kernel sequence per layer; ``0`` keeps one sidecar per request, as the reference does."""
    return _env_on("PQ_HSA_BATCH_FUSED", "1")


def flush_interval() -> int:
    return _env_int("PQ_HSA_FLUSH_INTERVAL", 256)


def min_pq_seq() -> int:
    """Shortest sequence worth a sidecar: sink + local window and a few keys to index."""
    return _env_int("PQ_HSA_SINK", 4) + _env_int("PQ_HSA_LOCAL", 128) + 16


def _prefix_extend_enabled() -> bool:
    """``PQ_HSA_PREFIX_EXTEND=1``: when a request's prompt continues the checkpointed one, restore the
    index and take in only the added tokens instead of rebuilding.  Off by default."""
    return _env_on("PQ_HSA_PREFIX_EXTEND")


def _prefix_extend_max_frac() -> float:
    raw = os.environ.get("PQ_HSA_PREFIX_EXTEND_MAX_FRAC")
    try:
        return 0.5 if raw is None else float(raw)
    except ValueError:      # unparsable: the default
        return 0.5


# ---------------------------------------------------------------------------- the gate
def reject(reason: str) -> bool:
    _tally("reject", reason)
    return False


def host_seq_lens(attn_metadata) -> list[int]:
    """The batch's sequence lengths as host integers.  Reading them from the device waits for the
    GPU, so a host copy carried by the metadata is preferred and the list is made once per step."""
    def read():
        src = getattr(attn_metadata, "seq_lens_cpu", None)
        return [int(x) for x in (attn_metadata.seq_lens if src is None else src).tolist()]

    return _memo(attn_metadata, "_pq_host_seq_lens", read)


def _num_reqs(md) -> int:
    lens = getattr(md, "seq_lens", None)
    return -1 if lens is None else int(lens.shape[0])


def _gate_checks(md, batched: bool):
    """(reason, passes) in the order the reasons are reported; tests are lazy because the later
    ones read what the earlier ones establish."""
    yield "cascade", lambda: not getattr(md, "use_cascade", False)
    yield "max_query_len!=1", lambda: int(getattr(md, "max_query_len", 0)) == 1
    tokens = lambda: int(getattr(md, "num_actual_tokens", 0))
    if batched:
        yield "num_reqs<1", lambda: _num_reqs(md) >= 1
        yield "num_actual_tokens!=num_reqs", lambda: tokens() == _num_reqs(md)
        yield "seq_too_short", lambda: min(host_seq_lens(md)) >= min_pq_seq()
    else:
        yield "num_actual_tokens!=1", lambda: tokens() == 1
        yield "num_reqs!=1", lambda: _num_reqs(md) == 1
        yield "seq_too_short", lambda: flashattn_seq_len(md, 0) >= min_pq_seq()


def should_pq_decode(attn_metadata) -> bool:
    """Is this call a single-token decode step the sidecar can serve?  The first failing test is
    counted in ``STATS["reject"]`` under the reference's reason string."""
    if attn_metadata is None:
        return reject("no_metadata")
    for reason, passes in _gate_checks(attn_metadata, batch_enabled()):
        if not passes():
            return reject(reason)
    return True


# ---------------------------------------------------------------------------- tensors in and out
def as_decode_qkv(t: torch.Tensor) -> torch.Tensor:
    """The step's first token as ``[1, heads, dim]``."""
    if t.ndim not in (2, 3):
        raise ValueError(f"expected [T,H,D] or [T,D], got {tuple(t.shape)}")
    row = t[:1]
    return row if t.ndim == 3 else row.unsqueeze(0)


def copy_ctx(output: torch.Tensor, ctx: torch.Tensor, num_actual: int) -> None:
    dst = output[:num_actual]
    dst.copy_(ctx.reshape(dst.shape).to(dst.dtype))


def write_kv_to_cache(key, value, kv_cache, attn_metadata, impl=None, layer=None) -> None:
    """This step's K/V rows -> their paged slots (5-D layout; vLLM >= 0.10 writes the 4-D layout
    itself before calling forward).  Uses vLLM's cache op when it is loaded."""
    if kv_cache.dim() == 5:
        k_pages, v_pages = kv_cache[0], kv_cache[1]
        vllm_op = getattr(getattr(torch.ops, "_C_cache_ops", None), "reshape_and_cache_flash", None)
        if vllm_op is not None and impl is not None and layer is not None:
            vllm_op(key, value, k_pages, v_pages, attn_metadata.slot_mapping, impl.kv_cache_dtype, layer._k_scale,
                    layer._v_scale)
        else:
            slots = attn_metadata.slot_mapping[: key.shape[0]].long()
            block, within = slots // k_pages.shape[1], slots % k_pages.shape[1]
            k_pages[block, within] = key.to(k_pages.dtype)
            v_pages[block, within] = value.to(v_pages.dtype)


def flush_sidecar(adapter) -> None:
    apply = getattr(adapter, "apply_pending_index_update", None)
    if apply is not None:
        apply()


def _flush_if_due(appends: int, flush: Callable[[], Any]) -> None:
    every = flush_interval()
    if every > 0 and appends > 0 and appends % every == 0:
        with _charge("pq_flush_s_total"):
            flush()
        STATS["pq_flush_calls"] += 1


# ---------------------------------------------------------------------------- prompt identity
def _digest(token_ids) -> bytes:
    return hashlib.blake2b(array("I", token_ids).tobytes(), digest_size=16).digest()


def _first_request_prompt(attn_metadata):
    """Prompt token ids of the batch's first request, through the model runner the wrap layer hangs
    on the metadata: ``(ids, None)`` or ``(None, why)``."""
    model_runner = getattr(attn_metadata, "_pq_runner", None)
    if model_runner is None:
        return None, "no_runner"
    in_batch = model_runner.input_batch.req_ids
    if len(in_batch or ()) == 0:
        return None, "no_request"
    ids = getattr(model_runner.requests.get(in_batch[0]), "prompt_token_ids", None)
    return (ids, None) if ids is not None else (None, "no_prompt")


def prefix_cache_key(attn_metadata, seq_len: int):
    """``(context_len, digest of the prompt ids)`` of the request, or None when the runner or the
    prompt is not reachable from the metadata."""
    def make():
        ids, _ = _first_request_prompt(attn_metadata)
        if ids is None:
            return None
        return int(seq_len) - int(attn_metadata.max_query_len), _digest(ids)

    return _memo(attn_metadata, "_pq_prefix_cache_key", make)


def prefix_extend_match(attn_metadata, old_key, checkpoint_len, seq_len: int):
    """Does the current request's prompt strictly extend the checkpointed prompt?  ``old_key`` is the
    ``(context_len, digest)`` stored with the checkpoint, ``checkpoint_len`` the sidecar's length at
    that time (prompt + the first decode token).  Returns ``(ok, reason, new_key, delta_tokens)``
    with the reference's reason strings.  The digest of the new prompt's first ``context_len`` ids
    is kept on the metadata object, so the layers of one step hash it once."""
    no = lambda why, delta=0: (False, why, None, delta)
    if None in (old_key, checkpoint_len):
        return no("no_checkpoint")
    old_ctx, old_digest = old_key
    old_ctx = int(old_ctx)
    if int(checkpoint_len) != old_ctx + 1:
        return no("checkpoint_inconsistent")
    seq_len = int(seq_len)
    context_len = seq_len - int(attn_metadata.max_query_len)
    delta = seq_len - int(checkpoint_len)
    if delta <= 0 or context_len <= old_ctx:
        return no("not_longer")
    if delta > _prefix_extend_max_frac() * seq_len:
        return no("delta_too_large", delta)
    heads = _memo(attn_metadata, "_pq_prefix_ext_digests", dict)
    if old_ctx not in heads:
        ids, why = _first_request_prompt(attn_metadata)
        if ids is None and why != "no_prompt":
            return no(why, delta)
        if ids is None or len(ids) != context_len:
            return no("prompt_len_mismatch", delta)
        heads[old_ctx] = _digest(ids[:old_ctx])
    if heads[old_ctx] != old_digest:
        return no("prefix_digest_mismatch", delta)
    longer_key = prefix_cache_key(attn_metadata, seq_len)
    return no("no_prefix_key", delta) if longer_key is None else (True, "ok", longer_key, delta)


# ---------------------------------------------------------------------------- one request per step
class Move(enum.Enum):
    """What a layer's sidecar does with a decode step."""

    APPEND = "append"      # the sequence grew by the one token of this step
    RESTORE = "restore"    # the checkpointed prompt is back: roll the sidecar back to it
    EXTEND = "extend"      # the prompt continues the checkpointed one: take in the added tokens
    BUILD = "build"        # anything else: index the sequence from the paged cache


@dataclasses.dataclass
class Plan:
    move: Move
    prefix_key: Any = None            # of this step's request (None: not known)
    miss_reason: Optional[str] = None  # why the checkpoint could not be restored
    extend_reject: Optional[str] = None
    delta_tokens: int = 0


def _miss_reason(st, adapter, pkey) -> str:
    for reason, holds in (("no_adapter", adapter is None), ("no_prefix_key", pkey is None)):
        if holds:
            return reason
    return "prefix_key_mismatch" if pkey != st["prefix_key"] else "checkpoint_length_mismatch"


def plan_step(st: dict[str, Any], seq_len: int, attn_metadata) -> Plan:
    """The transition function of a layer's sidecar: from its state (``sidecar``, ``seq_len``,
    ``prefix_key``) and the step's metadata to the move to make.  Nothing is changed here."""
    adapter, prev = st["sidecar"], st["seq_len"]
    if adapter is not None and prev is not None and seq_len == int(prev) + 1:
        return Plan(Move.APPEND)
    pkey = prefix_cache_key(attn_metadata, int(seq_len))
    saved = getattr(adapter, "prefix_checkpoint_length", None)
    if adapter is not None and pkey is not None and pkey == st["prefix_key"] and saved is not None \
            and int(saved) == seq_len:
        return Plan(Move.RESTORE, prefix_key=pkey)
    plan = Plan(Move.BUILD, prefix_key=pkey, miss_reason=_miss_reason(st, adapter, pkey))
    if adapter is not None and _prefix_extend_enabled() and callable(getattr(adapter, "extend_prefix", None)):
        ok, why, new_key, delta = prefix_extend_match(attn_metadata, st["prefix_key"], saved, seq_len)
        if ok:
            return dataclasses.replace(plan, move=Move.EXTEND, prefix_key=new_key, delta_tokens=delta)
        plan.extend_reject = why
    return plan


def _build_sidecar(impl, kv_cache, attn_metadata, seq_idx: int):
    with _charge("pq_gather_s_total"):
        keys, values, gathered = gather_flashattn_kv(kv_cache, attn_metadata, seq_idx)
    with _charge("pq_build_s_total"):
        adapter = sidecar_cls()(paper_index_config(), paper_attention_config(impl.scale),
                                num_query_heads=impl.num_heads, num_kv_heads=impl.num_kv_heads)
        adapter = adapter.build_cache(keys, values)
        adapter.set_paged_kv_context(kv_cache, attn_metadata, seq_idx)
    STATS["pq_build_calls"] += 1
    STATS["layers_built"] += 1
    STATS["batched_heads_active"] = getattr(adapter, "batched_heads_active", None)
    STATS["sidecar"] = type(adapter).__name__
    return adapter, gathered


def _attend(adapter, q, *also: str) -> torch.Tensor:
    with _charge("pq_forward_only_s_total", *also):
        return adapter.forward(q)


def _move_append(st, plan, io) -> torch.Tensor:
    adapter = st.get("sidecar")
    adapter.set_paged_kv_context(io.kv_cache, io.attn_metadata, 0)
    with _charge("pq_append_s_total", "pq_forward_s_total"):
        adapter.append(as_decode_qkv(io.key), as_decode_qkv(io.value))
    ctx = _attend(adapter, io.q, "pq_forward_s_total")
    STATS["pq_append_calls"] += 1
    st["seq_len"], st["appends"] = io.seq_len, int(st["appends"]) + 1
    _flush_if_due(st["appends"], lambda: flush_sidecar(adapter))
    return ctx


def _move_restore(st, plan, io) -> torch.Tensor:
    adapter = st.get("sidecar")
    with _charge("pq_restore_s_total"):
        if not adapter.restore_prefix(as_decode_qkv(io.key), as_decode_qkv(io.value), kv_cache=io.kv_cache,
                                      attn_metadata=io.attn_metadata, seq_idx=0):
            raise RuntimeError("prefix sidecar checkpoint disappeared during restore")
    STATS["prefix_persist_hits"] += 1
    st["seq_len"], st["appends"] = io.seq_len, 0
    return _attend(adapter, io.q)


def _move_extend(st, plan, io) -> Optional[torch.Tensor]:
    """None when the sidecar declines: the caller builds instead."""
    adapter = st.get("sidecar")
    began = time.perf_counter()
    info = adapter.extend_prefix(as_decode_qkv(io.key), as_decode_qkv(io.value), kv_cache=io.kv_cache,
                                 attn_metadata=io.attn_metadata, seq_idx=0, new_length=io.seq_len)
    spent = time.perf_counter() - began
    if info is None:
        return None
    STATS["pq_extend_s_total"] += spent
    STATS["pq_forward_s_total"] += spent
    STATS["prefix_extend_hits"] += 1
    STATS["pq_extend_delta_tokens_total"] = int(STATS["pq_extend_delta_tokens_total"]) + int(plan.delta_tokens)
    STATS["pq_extend_last"] = dict(info, wall_s=spent)
    st.update(prefix_key=plan.prefix_key, seq_len=io.seq_len, appends=0)
    ctx = _attend(adapter, io.q, "pq_forward_s_total")
    adapter.checkpoint_prefix()          # the turn after this one may extend it again
    return ctx


def _move_build(st, plan, io) -> torch.Tensor:
    if plan.extend_reject is not None:
        _tally("prefix_extend_rejects", plan.extend_reject)
    STATS["prefix_persist_misses"] += 1
    _tally("prefix_miss_reasons", plan.miss_reason)
    adapter, gathered = _build_sidecar(io.impl, io.kv_cache, io.attn_metadata, 0)
    if gathered != io.seq_len:
        raise RuntimeError(f"gather seq {gathered} != metadata seq {io.seq_len}")
    st.update(sidecar=adapter, prefix_key=plan.prefix_key, seq_len=io.seq_len, appends=0)
    ctx = _attend(adapter, io.q, "pq_forward_s_total")
    adapter.checkpoint_prefix()
    STATS["cuda_graph_active"] = getattr(adapter, "cuda_graph_active", None)
    return ctx


@dataclasses.dataclass
class _StepIO:
    impl: Any
    q: torch.Tensor
    key: torch.Tensor
    value: torch.Tensor
    kv_cache: torch.Tensor
    attn_metadata: Any
    seq_len: int


def run_pq_decode(impl, layer, query, key, value, kv_cache, attn_metadata) -> torch.Tensor:
    """One request, one token: make the layer's move and return the context ``[1, Hq, D]``."""
    st = state_for(impl, layer)
    io = _StepIO(impl, as_decode_qkv(query), key, value, kv_cache, attn_metadata,
                 flashattn_seq_len(attn_metadata, 0))
    plan = plan_step(st, io.seq_len, attn_metadata)
    ctx = None
    if plan.move is Move.EXTEND:
        ctx = _move_extend(st, plan, io)
        if ctx is None:
            plan = dataclasses.replace(plan, move=Move.BUILD, extend_reject="adapter_declined",
                                       prefix_key=prefix_cache_key(attn_metadata, io.seq_len))
    if ctx is None:
        ctx = {Move.APPEND: _move_append, Move.RESTORE: _move_restore, Move.BUILD: _move_build}[plan.move](st, plan, io)
    STATS["pq_decode_calls"] += 1
    return ctx


# ---------------------------------------------------------------------------- a batch per step
def _int32_table(attn_metadata, num_reqs: int) -> torch.Tensor:
    table = attn_metadata.block_table[:num_reqs]
    if table.dtype != torch.int32 or not table.is_contiguous():
        table = table.to(torch.int32).contiguous()
    return table


def request_tags(attn_metadata, lens: list[int], table: torch.Tensor, block_size: int):
    """Who is in each batch row, as ``(now, before)`` lists of hashable tags, one per row: a
    request that was in the previous step's batch shows, as ``before``, the tag that step stored
    for it as ``now``.

    With the model runner reachable the tags are vLLM's request ids (``now == before``).  Without
    it a request is known by the physical blocks it alone owns: the first block together with the
    block of its newest token.  The first block by itself is not enough: with prefix caching two
    live requests that share a prompt prefix share it.  The block of the newest token is written
    by this request in this step, so no other live request holds it; ``before`` names the block
    of the token one earlier, which is the block the previous step stored.  Read from the device
    once per step (one small copy) and kept on the metadata object."""
    def make():
        runner = getattr(attn_metadata, "_pq_runner", None)
        ids = list(getattr(getattr(runner, "input_batch", None), "req_ids", None) or [])[: len(lens)]
        if len(ids) == len(lens) and all(i is not None for i in ids) and len(set(ids)) == len(ids):
            tags = [("req", i) for i in ids]
            return tags, tags
        rows = torch.arange(len(lens), device=table.device)
        last = torch.tensor(lens, device=table.device) - 1
        cols = torch.stack([torch.zeros_like(last), last // block_size, (last - 1).clamp_min(0) // block_size])
        first, newest, earlier = table[rows, cols].tolist()
        return ([("blk", f, b) for f, b in zip(first, newest)], [("blk", f, b) for f, b in zip(first, earlier)])

    return _memo(attn_metadata, "_pq_request_tags", make)


def _continuing_rows(grp, before: list, lens: list[int]) -> list[Optional[int]]:
    """For every row of this step's batch, the row of the previous group it continues (same
    request, one token longer) or None.  A tag that occurs twice, here or there, identifies
    nobody: those requests are built afresh rather than guessed at."""
    if grp is None:
        return [None] * len(lens)
    there: dict[Any, Optional[int]] = {}
    for j, tag in enumerate(grp["tags"]):
        there[tag] = None if tag in there else j
    seen_twice = {t for t in before if before.count(t) > 1}
    rows = []
    for tag, ln in zip(before, lens):
        j = None if tag in seen_twice else there.get(tag)
        rows.append(j if j is not None and ln == grp["lens"][j] + 1 else None)
    return rows


def run_pq_decode_group(impl, layer, query, key, value, kv_cache, attn_metadata, output) -> torch.Tensor:
    """All requests of the decode batch through one engine: the step's appends ride on the decode
    launches and every sequence, KV head and query row is served by the same kernels.  When the
    batch is the previous one advanced by one token each, the step is one call; when requests
    left, joined or changed rows, the index rows of those that continue are copied into a new
    group (nothing is re-encoded) and only the newcomers are built."""
    from ..attention.engine import PQHSAEngine

    st = state_for(impl, layer)
    num_reqs = _num_reqs(attn_metadata)
    lens = list(host_seq_lens(attn_metadata))[:num_reqs]
    table = _int32_table(attn_metadata, num_reqs)
    now, before = request_tags(attn_metadata, lens, table, kv_cache_dims(kv_cache)[0])
    grp = st.get("group")
    came_from = _continuing_rows(grp, before, lens)
    if grp is not None and len(grp["tags"]) == num_reqs and came_from == list(range(num_reqs)):
        eng = grp["engine"]
        eng.bind_paged(kv_cache, table)      # the block table may have grown
        eng.advance(1)
        grp.update(lens=lens, tags=now, appends=grp["appends"] + 1)
        STATS["pq_append_calls"] += 1
    else:
        with _charge("pq_build_s_total"):
            fresh = [r for r in range(num_reqs) if came_from[r] is None]
            staying = [r for r in range(num_reqs) if came_from[r] is not None]
            newcomers = None
            if fresh:
                newcomers = PQHSAEngine(paper_index_config(), paper_attention_config(impl.scale), batch=len(fresh),
                                        kv_heads=impl.num_kv_heads, device=kv_cache.device)
                newcomers.bind_paged(kv_cache, table[fresh].contiguous())
                newcomers.build([lens[r] for r in fresh])
                STATS["pq_build_calls"] += 1
            if not staying:
                eng = newcomers
                STATS["pq_batch_group_builds"] += 1
            else:
                eng = PQHSAEngine.regroup([(newcomers, fresh.index(r)) if came_from[r] is None
                                           else (grp["engine"], came_from[r]) for r in range(num_reqs)])
                STATS["pq_batch_regroups"] += 1
            eng.bind_paged(kv_cache, table)
            if staying:
                eng.advance(1, which=staying)     # their new token is indexed by the step below
                STATS["pq_append_calls"] += 1
            grp = st["group"] = {"engine": eng, "lens": lens, "tags": now,
                                 "appends": grp["appends"] + 1 if staying else 0}
        STATS["sidecar"] = "PQHSAEngine"
    q, dst = query[:num_reqs], output[:num_reqs]
    groups = impl.num_heads // impl.num_kv_heads
    if dst.shape == q.shape and dst.dtype == q.dtype == kv_cache.dtype and dst.is_contiguous():
        eng.forward(q, groups, out=dst)                      # straight into vLLM's output buffer
    else:
        copy_ctx(output, eng.forward(q, groups), num_reqs)
    _flush_if_due(grp["appends"], eng.apply_pending_index_update)
    STATS["pq_batch_fused_steps"] += 1
    return output


def _run_pq_decode_rows(impl, layer, query, key, value, kv_cache, attn_metadata, output) -> torch.Tensor:
    """One sidecar per batch row (the reference's form): built when the row is first seen or its
    length does not follow the previous step's, appended to otherwise."""
    per_row = state_for(impl, layer).setdefault("batch", {})
    lens = list(host_seq_lens(attn_metadata))
    num_reqs = _num_reqs(attn_metadata)
    for r in range(num_reqs):
        one = slice(r, r + 1)
        rs = per_row.get(r)
        if rs is None or lens[r] != rs["seq_len"] + 1:
            adapter, _ = _build_sidecar(impl, kv_cache, attn_metadata, r)
            per_row[r] = {"sidecar": adapter, "seq_len": lens[r], "appends": 0}
        else:
            adapter = rs["sidecar"]
            adapter.set_paged_kv_context(kv_cache, attn_metadata, r)
            adapter.append(key[one], value[one])
            rs.update(seq_len=lens[r], appends=rs["appends"] + 1)
            every = flush_interval()
            if every > 0 and rs["appends"] % every == 0:
                flush_sidecar(adapter)
        copy_ctx(output[one], adapter.forward(query[one]), 1)
    for gone in [r for r in per_row if r >= num_reqs]:
        del per_row[gone]
    return output


def run_pq_decode_batch(impl, layer, query, key, value, kv_cache, attn_metadata, output) -> torch.Tensor:
    """``PQ_HSA_BATCH=1``: the decode batch through one engine (``batch_fused``, the default) or
    through one sidecar per request."""
    serve = run_pq_decode_group if batch_fused() else _run_pq_decode_rows
    serve(impl, layer, query, key, value, kv_cache, attn_metadata, output)
    STATS["pq_batch_steps"] += 1
    STATS["pq_batch_reqs_total"] += _num_reqs(attn_metadata)
    STATS["pq_decode_calls"] += 1
    return output


# ---------------------------------------------------------------------------- entry points
def run_pq_decode_into_output(impl, layer, query, key, value, kv_cache, attn_metadata, output) -> torch.Tensor:
    with _charge("pq_cache_write_s_total"):
        write_kv_to_cache(key, value, kv_cache, attn_metadata, impl, layer)
    if batch_enabled():
        return run_pq_decode_batch(impl, layer, query, key, value, kv_cache, attn_metadata, output)
    ctx = run_pq_decode(impl, layer, query, key, value, kv_cache, attn_metadata)
    with _charge("pq_copy_ctx_s_total"):
        copy_ctx(output, ctx, 1)
    return output


def pq_or_dense_forward(impl, layer, query, key, value, kv_cache, attn_metadata, output: Optional[torch.Tensor],
                        dense_forward: Callable[[], torch.Tensor]) -> torch.Tensor:
    """The wrapped ``forward``: decode steps that pass the gate go to the sidecar, everything else
    to vLLM's own attention.  A failure in the sidecar is recorded and re-raised, or, with
    ``PQ_HSA_FALLBACK=1``, answered by the dense path."""
    if not (pq_enabled() and should_pq_decode(attn_metadata)):
        with _charge("dense_fa_s_total"):
            result = dense_forward()
        STATS["dense_fa_calls"] += 1
        return result
    try:
        if output is None:
            raise AssertionError("the decode hook needs vLLM's output buffer")
        return run_pq_decode_into_output(impl, layer, query, key, value, kv_cache, attn_metadata, output)
    except Exception as err:
        STATS.update(last_error=f"{type(err).__name__}: {err}", dense_fallback_calls=STATS["dense_fallback_calls"] + 1)
        if _env_on("PQ_HSA_FALLBACK"):
            return dense_forward()
        raise
