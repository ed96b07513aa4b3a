"""Seeded synthetic K/V/query generator shared by the tests, the fixtures and the bench.

Keys of one KV head are a mixture of Gaussian clusters (centres N(0,1), within-cluster
sigma 0.3), scaled per channel by log-normal(0, 0.5) factors with a few outlier channels
multiplied by 8.  Values are N(0,1).  Each query is one of the keys plus N(0, 0.2) noise,
so a needle exists.  Every (sequence, KV head) draws from an independent seed.
"""

from __future__ import annotations

import torch


def head_seed(seed0: int, seq: int, head: int) -> int:
    return int(seed0) + 1000 * int(seq) + int(head)


def make_head(
    ctx: int,
    *,
    dim: int = 128,
    groups: int = 1,
    seed: int = 0,
    num_clusters: int = 512,
    sigma: float = 0.3,
    outlier_channels: int = 4,
    outlier_gain: float = 8.0,
    query_noise: float = 0.2,
    device: torch.device | str = "cpu",
    dtype: torch.dtype = torch.float32,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Return ``(keys [ctx, dim], values [ctx, dim], queries [groups, dim])`` for one KV head.

    Random numbers are always drawn on the CPU generator so that the same seed gives the
    same data wherever the tensors end up; ``dtype`` rounds K/V (queries follow).
    """

    gen = torch.Generator(device="cpu")
    gen.manual_seed(int(seed))
    centres = torch.randn(num_clusters, dim, generator=gen)
    member = torch.randint(0, num_clusters, (ctx,), generator=gen)
    keys = centres[member] + sigma * torch.randn(ctx, dim, generator=gen)
    channel_scale = torch.exp(0.5 * torch.randn(dim, generator=gen))
    outliers = torch.randperm(dim, generator=gen)[:outlier_channels]
    channel_scale[outliers] *= outlier_gain
    keys = keys * channel_scale
    values = torch.randn(ctx, dim, generator=gen)
    # needles are drawn from the part of the context that is neither sink nor recent
    lo = min(ctx - 1, 8)
    hi = max(lo + 1, ctx - 128)
    needle = torch.randint(lo, hi, (groups,), generator=gen)
    queries = keys[needle] + query_noise * torch.randn(groups, dim, generator=gen)
    keys = keys.to(dtype)
    values = values.to(dtype)
    queries = queries.to(dtype)
    return keys.to(device), values.to(device), queries.to(device)


def make_layer(
    ctx: int,
    *,
    batch: int = 1,
    kv_heads: int = 1,
    groups: int = 1,
    dim: int = 128,
    seed0: int = 0,
    device: torch.device | str = "cpu",
    dtype: torch.dtype = torch.float32,
    **kwargs,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``keys/values [B, H, ctx, dim]`` and ``queries [B, H*G, dim]`` (query head h*G+g <-> KV head h)."""

    keys = torch.empty(batch, kv_heads, ctx, dim, dtype=dtype, device=device)
    values = torch.empty_like(keys)
    queries = torch.empty(batch, kv_heads * groups, dim, dtype=dtype, device=device)
    for b in range(batch):
        for h in range(kv_heads):
            k, v, q = make_head(
                ctx,
                dim=dim,
                groups=groups,
                seed=head_seed(seed0, b, h),
                device=device,
                dtype=dtype,
                **kwargs,
            )
            keys[b, h] = k
            values[b, h] = v
            queries[b, h * groups : (h + 1) * groups] = q
    return keys, values, queries
