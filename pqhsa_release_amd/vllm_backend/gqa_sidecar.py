"""GQA sidecar: the object the vLLM decode runtime builds per layer and calls per step.

Same surface as the reference's ``GQASidecar`` / ``GQASidecarFast``
(benchmarks/vllm_backend/gqa_sidecar.py:11-76, gqa_sidecar_fast.py:48-187): ``build_cache``,
``append``, ``lean_append``, ``append_many``, ``forward``, ``set_paged_kv_context``,
``checkpoint_prefix`` / ``restore_prefix`` / ``extend_prefix`` / ``prefix_checkpoint_length`` and the
``batched_heads_active`` / ``cuda_graph_active`` flags.  One batched engine serves all KV
heads; once a paged context is set the exact rows are read from vLLM's pages in place and the
sidecar drops its own K/V copy.
"""

from __future__ import annotations

import time

import torch

from ..attention.decode_adapter import GQAIVFPQDecodeAttentionAdapter
from ..config import IVFPQConfig, SparseAttentionConfig


class GQASidecar:
    def __init__(self, index_config: IVFPQConfig, attention_config: SparseAttentionConfig, *,
                 num_query_heads: int, num_kv_heads: int) -> None:
        if num_query_heads % num_kv_heads != 0:
            raise ValueError("GQA requires num_query_heads % num_kv_heads == 0")
        self.index_config = index_config
        self.attention_config = attention_config
        self.num_query_heads = int(num_query_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.num_groups = self.num_query_heads // self.num_kv_heads
        self.adapter = GQAIVFPQDecodeAttentionAdapter(index_config, attention_config,
                                                      num_query_heads=self.num_query_heads,
                                                      num_key_value_heads=self.num_kv_heads)
        self.length = 0
        self._checkpoint: dict[str, object] | None = None
        self._paged = False

    # flags the runtime reports in its stats
    @property
    def batched_heads_active(self) -> bool:
        return self.adapter.engine is not None

    @property
    def cuda_graph_active(self) -> bool:
        return False

    @property
    def streams(self):
        return self.adapter.streams

    @property
    def prefix_checkpoint_length(self) -> int | None:
        return None if self._checkpoint is None else int(self._checkpoint["length"])

    def build_cache(self, keys: torch.Tensor, values: torch.Tensor) -> "GQASidecar":
        if keys.ndim != 4 or values.ndim != 4:
            raise ValueError("keys/values must be [1, kv_heads, seq, dim]")
        if keys.shape[0] != 1 or keys.shape[1] != self.num_kv_heads:
            raise ValueError(f"expected keys [1, {self.num_kv_heads}, S, D], got {tuple(keys.shape)}")
        self.adapter.build_cache(keys, values)
        self.length = int(keys.shape[2])
        self._paged = False
        return self

    def set_paged_kv_context(self, kv_cache: torch.Tensor, attn_metadata, seq_idx: int = 0) -> None:
        """Point the exact-attention reads at vLLM's paged cache (refreshed every step because the
        block table may have grown)."""
        table = attn_metadata.block_table
        if table.dtype != torch.int32 or not table.is_contiguous():
            table = table.to(torch.int32).contiguous()
        self.adapter.engine.bind_paged(kv_cache, table[seq_idx : seq_idx + 1])
        self._paged = True

    def append(self, keys: torch.Tensor, values: torch.Tensor) -> None:
        if keys.ndim != 3 or values.ndim != 3:
            raise ValueError("append keys/values must be [1, kv_heads, dim]")
        self.adapter.append(keys, values)
        self.length += 1

    def lean_append(self, keys: torch.Tensor, values: torch.Tensor, q_src=None) -> bool:
        """``[T, kv_heads, dim]`` rows straight from the model (T == 1 in steady decode)."""
        if keys.ndim != 3 or keys.shape[0] != 1:
            return False
        self.append(keys[:1], values[:1])
        return True

    def append_many(self, keys: torch.Tensor, values: torch.Tensor, *, flush_every: int = 0) -> int:
        if keys.ndim == 4:
            keys, values = keys[0], values[0]
        flushes = 0
        for i in range(int(keys.shape[1])):
            self.append(keys[:, i].unsqueeze(0), values[:, i].unsqueeze(0))
            if flush_every > 0 and (i + 1) % flush_every == 0:
                flushes += int(self.adapter.apply_pending_index_update() > 0)
        return flushes

    def forward(self, queries: torch.Tensor) -> torch.Tensor:
        """queries ``[1, q_heads, dim]`` -> context ``[1, q_heads, dim]``."""
        if queries.ndim != 3 or queries.shape[0] != 1:
            raise ValueError(f"queries must be [1, q_heads, dim], got {tuple(queries.shape)}")
        return self.adapter.forward_context_fast(queries)

    def apply_pending_index_update(self) -> int:
        return self.adapter.apply_pending_index_update()

    # prefix checkpoint: reuse the index when the same prompt comes back
    def checkpoint_prefix(self) -> None:
        self._checkpoint = {"length": self.length, "state": self.adapter.engine.state_dict()}

    def restore_prefix(self, keys: torch.Tensor, values: torch.Tensor, *, kv_cache=None, attn_metadata=None,
                       seq_idx: int = 0) -> bool:
        if self._checkpoint is None:
            return False
        self.adapter.engine.load_state_dict(self._checkpoint["state"])
        self.length = int(self._checkpoint["length"])
        if kv_cache is not None and attn_metadata is not None:
            self.set_paged_kv_context(kv_cache, attn_metadata, seq_idx)
        return True

    def extend_prefix(self, keys: torch.Tensor | None = None, values: torch.Tensor | None = None, *, kv_cache,
                      attn_metadata, seq_idx: int = 0, new_length: int) -> dict | None:
        """Restore the checkpointed prefix and grow it in place to ``new_length`` tokens: the next
        request's prompt is the checkpointed prompt followed by more tokens, which vLLM's prefill
        has already written to the paged cache (GQAIVFPQDecodeAttentionAdapter.extend_prefix,
        benchmarks/e2e_pq_param_sweep.py:3600-3733).  The added rows are encoded with the
        checkpointed tables after the configured update step (one EMA move under the deferred
        strategy), not by retraining.  The checkpoint's last row, the old request's first decode
        token, is overwritten by the new prompt; it must still lie in the exact window.  Returns
        counters and timings, or ``None`` when the caller has to rebuild."""
        if self._checkpoint is None:
            return None
        base, new_length = int(self._checkpoint["length"]), int(new_length)
        if new_length <= base or kv_cache is None or attn_metadata is None:
            return None
        info: dict = {"base_length": base, "new_length": new_length, "delta_tokens": new_length - base, "ring": False}
        t0 = time.perf_counter()
        if not self.restore_prefix(None, None):
            return None
        info["restore_s"] = time.perf_counter() - t0
        eng = self.adapter.engine
        delta_start = base - 1
        if eng._retrieval_end(0) > delta_start:
            return None                       # the row that changes is an indexed one
        t1 = time.perf_counter()
        if eng.keys_buf is not None:          # the sidecar keeps its own K/V copy: the new rows must land there
            from .paged_kv_fa import gather_flashattn_kv_range

            dk, dv = gather_flashattn_kv_range(kv_cache, attn_metadata, seq_idx, delta_start, new_length)
            eng._grow_dense(new_length)
            eng.keys_buf[0, :, delta_start:new_length].copy_(dk)
            eng.values_buf[0, :, delta_start:new_length].copy_(dv)
        else:
            self.set_paged_kv_context(kv_cache, attn_metadata, seq_idx)
        info["gather_s"] = time.perf_counter() - t1
        t2 = time.perf_counter()
        info["flush_applied_streams"] = eng.extend([new_length]) * self.num_kv_heads
        info["flush_s"] = time.perf_counter() - t2
        self.length = new_length
        info["total_s"] = time.perf_counter() - t0
        info["indexed_length"] = int(eng.indexed_len[0])
        info["retrieval_len"] = int(eng.n(0))
        return info


# the runtime's PQ_HSA_SIDECAR switch selects between two classes in the reference; both names
# resolve to the batched engine here
GQASidecarFast = GQASidecar
