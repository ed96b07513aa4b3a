"""Model-facing decode adapters with the reference's call signatures.

``IVFPQDecodeAttentionAdapter`` mirrors pq_hsa/attention/decode_adapter.py:18-109 (one
independent index per (batch, head) stream, pq_hsa/attention/multihead.py:30-43);
``GQAIVFPQDecodeAttentionAdapter`` mirrors the GQA-sharing adapter of
benchmarks/e2e_pq_param_sweep.py:2834-2861, 3899-3921, 4805-4812 (query head ``h*G + g``
attends through KV head ``h``).  Both hand every call to one batched ``PQHSAEngine``: where
the reference loops over streams in Python, one kernel sequence covers all of them.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ..config import IVFPQConfig, SparseAttentionConfig
from .engine import PQHSAEngine


@dataclass(slots=True)
class StreamOutput:
    """Per-stream record of one query; the fields the reference's no-details ``AttentionOutput``
    carries (pq_hsa/attention/sparse_attention.py:1040-1058)."""

    output: torch.Tensor
    selected_count: int
    denominator_count: int
    approx_retrieval_count: int
    exact_retrieval_count: int
    candidate_count: int
    probed_list_count: int = 0


@dataclass(slots=True)
class MultiHeadAttentionOutput:
    output: torch.Tensor
    per_stream: tuple[StreamOutput, ...]
    leading_shape: tuple[int, ...]


class DecodeAttentionOutput:
    """``context`` plus the reference's per-query / per-stream records.  The records are host
    bookkeeping (one small object per query row and stream); they are built when ``per_query`` is
    first read, so a serving loop that only takes ``context`` does not pay for them."""

    __slots__ = ("context", "_per_query")

    def __init__(self, context: torch.Tensor, per_query) -> None:
        self.context = context
        self._per_query = per_query   # the records, or a function that builds them

    @property
    def per_query(self) -> tuple[MultiHeadAttentionOutput, ...]:
        if callable(self._per_query):
            self._per_query = self._per_query()
        return self._per_query


def _normalize_queries(queries: torch.Tensor) -> tuple[torch.Tensor, bool]:
    if queries.ndim == 3:
        return queries.unsqueeze(-2), False
    if queries.ndim == 4:
        return queries, True
    raise ValueError("queries must be [batch, heads, dim] or [batch, heads, query_len, dim]")


def _squeeze_decode_token(tensor: torch.Tensor, name: str) -> torch.Tensor:
    if tensor.ndim == 3:
        return tensor
    if tensor.ndim == 4 and tensor.shape[-2] == 1:
        return tensor.squeeze(-2)
    raise ValueError(f"{name} must be [batch, heads, dim] or [batch, heads, 1, dim]")


class _AdapterBase:
    def __init__(self, index_config: IVFPQConfig, attention_config: SparseAttentionConfig):
        self.index_config = index_config
        self.attention_config = attention_config
        self.engine: PQHSAEngine | None = None
        self._leading_shape: tuple[int, int] | None = None

    # -- shared plumbing ---------------------------------------------------------------
    def _check_built(self) -> PQHSAEngine:
        if self.engine is None:
            raise RuntimeError("build_cache must be called before using the adapter")
        return self.engine

    @property
    def leading_shape(self) -> tuple[int, ...]:
        if self._leading_shape is None:
            raise RuntimeError("build_cache must be called before reading leading_shape")
        return self._leading_shape

    @property
    def streams(self) -> tuple[tuple[int, int], ...]:
        """One (batch, kv head) pair per independent index, in the reference's flattening order."""
        if self._leading_shape is None:
            return ()
        b, h = self._leading_shape
        return tuple((i, j) for i in range(b) for j in range(h))

    def _build(self, keys: torch.Tensor, values: torch.Tensor, kv_heads: int) -> None:
        if keys.ndim != 4 or values.ndim != 4:
            raise ValueError("keys and values must be [batch, heads, seq, dim]")
        if keys.shape[:-2] != values.shape[:-2] or keys.shape[-2] != values.shape[-2]:
            raise ValueError("keys and values must have matching batch/head/sequence dimensions")
        if keys.shape[1] != kv_heads:
            raise ValueError(f"expected {kv_heads} KV heads, got {keys.shape[1]}")
        if keys.shape[-1] != 128 or values.shape[-1] != 128:
            raise ValueError("the MI355X kernels implement head dim 128")
        if not keys.is_cuda:
            raise RuntimeError("PQ-HSA decode attention needs device tensors: the MI355X kernels have no CPU path")
        self._leading_shape = (keys.shape[0], keys.shape[1])
        self.engine = PQHSAEngine(self.index_config, self.attention_config, batch=keys.shape[0],
                                  kv_heads=keys.shape[1], device=keys.device)
        self.engine.adopt(keys, values)
        self.engine.build([keys.shape[2]] * keys.shape[0])

    def append(self, keys: torch.Tensor, values: torch.Tensor) -> None:
        eng = self._check_built()
        k = _squeeze_decode_token(keys, "keys")
        v = _squeeze_decode_token(values, "values")
        expected = (*self._leading_shape, 128)
        if tuple(k.shape) != expected:
            raise ValueError(f"keys must have shape {expected}, got {tuple(k.shape)}")
        if tuple(v.shape) != expected:
            raise ValueError(f"values must have shape {expected}, got {tuple(v.shape)}")
        eng.write_rows(k, v)
        eng.advance(1)

    def apply_pending_index_update(self) -> int:
        eng = self._check_built()
        return eng.B * eng.H if eng.apply_pending_index_update() else 0

    def _per_query_later(self, context: torch.Tensor, groups: int):
        """context [B, H, Q, D] -> a function that builds the reference's per-query / per-stream
        records (host numbers only; nothing is read back from the device).  The counts are taken
        now, so later appends do not change what the records say about this step."""
        eng = self.engine
        from .. import ops

        ac = self.attention_config
        counts = []
        for b in range(eng.B):
            n, full = eng.n(b), eng.full_count(b)
            counts.append((n, full, ops.resolve_topk(n, ac.retrieval_top_fraction, ac.retrieval_topk)))

        def build() -> tuple[MultiHeadAttentionOutput, ...]:
            records = []
            for qpos in range(context.shape[2]):
                per_stream = []
                for b, (n, full, k) in enumerate(counts):
                    for h in range(context.shape[1]):
                        per_stream.append(StreamOutput(context[b, h, qpos], full + k, full + n, n, k, n))
                records.append(MultiHeadAttentionOutput(context[:, :, qpos], tuple(per_stream),
                                                        (context.shape[0], context.shape[1])))
            return tuple(records)

        return build

    def state_dict(self) -> dict[str, object]:
        eng = self._check_built()
        return {"attention": {"engine": eng.state_dict(), "leading_shape": tuple(self._leading_shape),
                              "index_config": _asdict(self.index_config),
                              "attention_config": _asdict(self.attention_config)}}

    def load_state_dict(self, state: dict[str, object]):
        attention = state.get("attention")
        if not isinstance(attention, dict):
            raise ValueError("adapter state must contain an attention dict")
        eng_state = attention["engine"]
        device = eng_state["index"]["codes"].device if "index" in eng_state else eng_state["keys"].device
        if device.type != "cuda":
            device = torch.device("cuda")
        self._leading_shape = tuple(attention["leading_shape"])
        self.engine = PQHSAEngine(self.index_config, self.attention_config, batch=int(eng_state["batch"]),
                                  kv_heads=int(eng_state["kv_heads"]), device=device)
        self.engine.load_state_dict(eng_state)
        return self


def _asdict(cfg) -> dict[str, object]:
    return {name: getattr(cfg, name) for name in cfg.__slots__}


class IVFPQDecodeAttentionAdapter(_AdapterBase):
    """keys/values ``[batch, heads, seq, dim]``; queries ``[batch, heads, dim]`` or
    ``[batch, heads, query_len, dim]`` (all query positions of a head attend the same cache)."""

    def build_cache(self, keys: torch.Tensor, values: torch.Tensor) -> "IVFPQDecodeAttentionAdapter":
        if keys.ndim != 4 or values.ndim != 4:
            raise ValueError("keys and values must be [batch, heads, seq, dim]")
        self._build(keys, values, keys.shape[1])
        return self

    @classmethod
    def from_state_dict(cls, state, *, index_config=None, attention_config=None):
        attention = state.get("attention")
        if not isinstance(attention, dict):
            raise ValueError("adapter state must contain an attention dict")
        ic = index_config or IVFPQConfig(**attention["index_config"])
        ac = attention_config or SparseAttentionConfig(**attention["attention_config"])
        return cls(ic, ac).load_state_dict(state)

    def forward(self, queries: torch.Tensor) -> DecodeAttentionOutput:
        eng = self._check_built()
        q, had_len = _normalize_queries(queries)
        b, h = self._leading_shape
        if tuple(q.shape[:2]) != (b, h) or q.shape[-1] != 128:
            raise ValueError(f"queries must have shape ({b}, {h}, query_len, 128), got {tuple(q.shape)}")
        qlen = q.shape[2]
        ctx = eng.forward(q.reshape(b, h * qlen, 128), qlen).reshape(b, h, qlen, 128).to(queries.dtype)
        per_query = self._per_query_later(ctx, qlen)
        return DecodeAttentionOutput(context=ctx if had_len else ctx.squeeze(-2), per_query=per_query)

    def decode_step(self, queries, keys=None, values=None, *, append_kv: bool = True) -> DecodeAttentionOutput:
        if append_kv:
            if keys is None or values is None:
                raise ValueError("keys and values are required when append_kv=True")
            self.append(keys, values)
        return self.forward(queries)


class GQAIVFPQDecodeAttentionAdapter(_AdapterBase):
    """One shared K/V cache + index per KV head for its group of query heads."""

    def __init__(self, index_config, attention_config, *, num_query_heads: int, num_key_value_heads: int,
                 share_layer_pq_codebook: bool = False):
        if num_query_heads % num_key_value_heads != 0:
            raise ValueError("num_query_heads must be divisible by num_key_value_heads, got "
                             f"{num_query_heads} and {num_key_value_heads}")
        super().__init__(index_config, attention_config)
        self.num_query_heads = int(num_query_heads)
        self.num_key_value_heads = int(num_key_value_heads)
        self.num_key_value_groups = self.num_query_heads // self.num_key_value_heads
        if self.num_key_value_groups > 16:
            raise ValueError("the MI355X kernels take GQA groups of at most 16 query heads")
        if share_layer_pq_codebook:
            raise ValueError("share_layer_pq_codebook is not implemented by the MI355X path")

    def build_cache(self, keys: torch.Tensor, values: torch.Tensor) -> "GQAIVFPQDecodeAttentionAdapter":
        if keys.ndim != 4 or values.ndim != 4:
            raise ValueError("keys and values must be [batch, kv_heads, seq, dim]")
        self._build(keys, values, self.num_key_value_heads)
        return self

    def forward(self, queries: torch.Tensor) -> DecodeAttentionOutput:
        eng = self._check_built()
        q = queries
        had_len = q.ndim == 4
        if had_len:
            if q.shape[2] != 1:
                raise ValueError("the GQA decode adapter takes one query position per step")
            q = q.squeeze(2)
        b = self._leading_shape[0]
        if q.ndim != 3 or tuple(q.shape) != (b, self.num_query_heads, 128):
            raise ValueError(f"queries must be [{b}, {self.num_query_heads}, (1,) 128], got {tuple(queries.shape)}")
        ctx = eng.forward(q, self.num_key_value_groups).to(queries.dtype)
        g = self.num_key_value_groups
        per_query = self._per_query_later(ctx.reshape(b, self.num_key_value_heads, g, 128), g)
        return DecodeAttentionOutput(context=ctx.unsqueeze(2) if had_len else ctx, per_query=per_query)

    def forward_context_fast(self, queries: torch.Tensor) -> torch.Tensor:
        """queries ``[B, Hq, 128]`` -> context, without the per-query records."""
        eng = self._check_built()
        return eng.forward(queries, self.num_key_value_groups).to(queries.dtype)

    def decode_step(self, queries, keys=None, values=None, *, append_kv: bool = True) -> DecodeAttentionOutput:
        if append_kv:
            if keys is None or values is None:
                raise ValueError("keys and values are required when append_kv=True")
            self.append(keys, values)
        return self.forward(queries)
