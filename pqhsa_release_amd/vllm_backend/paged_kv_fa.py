"""Readers of vLLM's FLASH_ATTN paged KV cache, same signatures as the reference's
benchmarks/vllm_backend/paged_kv_fa.py (both page layouts: 5-D ``[2, blocks, block_size,
kv_heads, dim]`` and 4-D ``[blocks, kv_heads, block_size, 2*dim]``).

``split_kv_cache`` / ``kv_cache_dims`` / ``flashattn_seq_len`` are views and host integers; the
three gathers move rows with the HIP paged-gather kernels.  The decode kernels themselves do
not use these copies: they read the pages in place through ``ops.kv_paged``.
"""

from __future__ import annotations

import torch

from .. import ops


def flashattn_seq_len(attn_metadata, seq_idx: int = 0) -> int:
    """Sequence length of one request without a device sync where the metadata allows it
    (paged_kv_fa.py:13-25 of the reference)."""
    seq_lens = attn_metadata.seq_lens
    if seq_idx == 0 and int(seq_lens.shape[0]) == 1:
        return int(attn_metadata.max_seq_len)
    return int(seq_lens[seq_idx].item())


def is_new_kv_layout(kv_cache: torch.Tensor) -> bool:
    return kv_cache.dim() == 4


def split_kv_cache(kv_cache: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """(key_cache, value_cache) views shaped ``[blocks, block_size, kv_heads, dim]``."""
    if kv_cache.dim() == 5:
        return kv_cache[0], kv_cache[1]
    if kv_cache.dim() == 4:
        head_size = int(kv_cache.shape[-1]) // 2
        k, v = kv_cache.transpose(1, 2).split(head_size, dim=-1)
        return k, v
    raise ValueError(f"unsupported FLASH_ATTN kv_cache shape {tuple(kv_cache.shape)}")


def kv_cache_dims(kv_cache: torch.Tensor) -> tuple[int, int, int]:
    k, _ = split_kv_cache(kv_cache)
    return int(k.shape[1]), int(k.shape[2]), int(k.shape[3])


def _block_table(attn_metadata) -> torch.Tensor:
    table = attn_metadata.block_table
    if table.dtype != torch.int32 or not table.is_contiguous():
        table = table.to(torch.int32).contiguous()
    return table


def gather_flashattn_kv(kv_cache: torch.Tensor, attn_metadata, seq_idx: int = 0):
    """Contiguous K/V of one request, ``[1, kv_heads, seq, dim]`` each, plus the length."""
    seq_len = flashattn_seq_len(attn_metadata, seq_idx)
    _, kv_heads, head_dim = kv_cache_dims(kv_cache)
    if seq_len <= 0:
        empty = kv_cache.new_empty(1, kv_heads, 0, head_dim)
        return empty, empty, 0
    src = ops.kv_paged(kv_cache, _block_table(attn_metadata))
    k, v = ops.paged_gather_range(src, seq_idx, 0, seq_len)
    return k.unsqueeze(0), v.unsqueeze(0), seq_len


def gather_flashattn_kv_range(kv_cache: torch.Tensor, attn_metadata, seq_idx: int, start: int, end: int):
    """Token range ``[start, end)`` -> keys/values ``[kv_heads, n, dim]``."""
    n = int(end) - int(start)
    _, kv_heads, head_dim = kv_cache_dims(kv_cache)
    if n <= 0:
        empty = kv_cache.new_empty(kv_heads, 0, head_dim)
        return empty, empty
    src = ops.kv_paged(kv_cache, _block_table(attn_metadata))
    return ops.paged_gather_range(src, seq_idx, int(start), int(end))


def gather_flashattn_kv_at_indices(kv_cache: torch.Tensor, attn_metadata, seq_idx: int, token_indices: torch.Tensor):
    """Per-head scattered token gather; ``token_indices`` has the KV head as leading dim
    (e.g. ``[H, G, topk]``); returns keys/values shaped like it plus ``[dim]``."""
    src = ops.kv_paged(kv_cache, _block_table(attn_metadata))
    return ops.paged_gather_at(src, seq_idx, token_indices)
