"""Index training (coarse k-means + per-subspace PQ k-means) with torch ops on the keys' device.

Training happens once after prefill and is not part of the decode hot path; it produces the
``coarse [L, D]`` / ``codebooks [M, 16, D/M]`` tensors that the HIP encode and scan kernels
consume.  The procedure mirrors the reference's (pq_hsa/index/kmeans.py:134-227 seeded Lloyd
iterations with empty-cluster reseeding; pq_hsa/index/ivfpq.py:275-348 coarse k-means on key
directions, then PQ on the residuals with seed + 10000 + subspace; pq_hsa/index/pq.py:47-95).

The seeded draws (the starting subset, replacements for empty clusters) are made with a CPU
generator whatever device the keys are on, as the reference makes them for the CPU tensors it
trains on: the same seed then starts the same trajectory here and there, and the arithmetic
(torch products on the keys' device) is all that can differ.
"""

from __future__ import annotations

import functools

import torch


def _nearest(vectors: torch.Tensor, centroids: torch.Tensor, chunk: int = 32768) -> torch.Tensor:
    cf = centroids.float()
    half_sq = (cf * cf).sum(dim=1)
    out = torch.empty(vectors.shape[0], dtype=torch.long, device=vectors.device)
    for s in range(0, vectors.shape[0], chunk):
        v = vectors[s : s + chunk].float()
        out[s : s + chunk] = (half_sq.unsqueeze(0) - 2.0 * (v @ cf.t())).argmin(dim=1)
    return out


def kmeans_l2(vectors: torch.Tensor, num_clusters: int, *, max_iter: int, seed: int = 0, eps: float = 1e-12,
              initial_centroids: torch.Tensor | None = None):
    """Lloyd iterations from a seeded random subset; returns ``(centroids, assignments)``."""
    if vectors.ndim != 2:
        raise ValueError(f"vectors must be [N, D], got {tuple(vectors.shape)}")
    n, dim = vectors.shape
    if n == 0:
        raise ValueError("cannot train k-means with zero vectors")
    if num_clusters <= 0:
        raise ValueError("num_clusters must be positive")
    gen = torch.Generator(device="cpu")
    gen.manual_seed(int(seed))
    dev = vectors.device
    if initial_centroids is not None:
        if tuple(initial_centroids.shape) != (num_clusters, dim):
            raise ValueError(f"initial_centroids must have shape ({num_clusters}, {dim})")
        centroids = initial_centroids.to(device=vectors.device, dtype=vectors.dtype).clone()
    elif n >= num_clusters:
        centroids = vectors[torch.randperm(n, generator=gen)[:num_clusters].to(dev)].clone()
    else:
        extra = torch.randint(0, n, (num_clusters - n,), generator=gen).to(dev)
        centroids = torch.cat([vectors, vectors[extra]], dim=0).clone()
    assign = torch.zeros(n, dtype=torch.long, device=vectors.device)
    for _ in range(max_iter):
        nxt = _nearest(vectors, centroids)
        same = torch.equal(assign, nxt)
        assign = nxt
        if same:
            break
        sums = torch.zeros(num_clusters, dim, dtype=torch.float32, device=vectors.device)
        sums.index_add_(0, assign, vectors.float())
        counts = torch.bincount(assign, minlength=num_clusters).float()
        filled = counts > 0
        sums[filled] /= counts[filled].unsqueeze(1).clamp_min(eps)
        empty = ~filled
        if bool(empty.any()):
            pick = torch.randint(0, n, (int(empty.sum().item()),), generator=gen).to(dev)
            sums[empty] = vectors[pick].float()
        centroids = sums.to(vectors.dtype)
    return centroids, _nearest(vectors, centroids)


def train_ivfpq(keys: torch.Tensor, *, num_lists: int, num_subspaces: int = 8, num_codes: int = 16,
                coarse_iter: int = 1, pq_iter: int = 2, seed: int = 0, eps: float = 1e-12):
    """Train one stream's index on its retrieval-region keys ``[N, D]`` (direction-normalised,
    residual PQ).  Returns fp32 ``(coarse [L', D], codebooks [M, num_codes, D/M])`` with
    ``L' = min(num_lists, N)``."""
    if keys.ndim != 2 or keys.shape[0] == 0:
        raise ValueError("cannot build IVF-PQ index with zero keys")
    if keys.shape[1] % num_subspaces != 0:
        raise ValueError(f"dim={keys.shape[1]} must be divisible by num_subspaces={num_subspaces}")
    k32 = keys.float()
    norms = torch.linalg.vector_norm(k32, dim=-1).clamp_min(eps)
    dirs = k32 / norms.unsqueeze(-1)
    lists = min(int(num_lists), dirs.shape[0])
    coarse, assign = kmeans_l2(dirs, lists, max_iter=coarse_iter, seed=seed, eps=eps)
    resid = dirs - coarse[assign]
    sub = keys.shape[1] // num_subspaces
    chunks = resid.reshape(resid.shape[0], num_subspaces, sub)
    books = []
    for m in range(num_subspaces):
        c, _ = kmeans_l2(chunks[:, m].contiguous(), num_codes, max_iter=pq_iter, seed=seed + 10_000 + m, eps=eps)
        books.append(c)
    return coarse.float().contiguous(), torch.stack(books, dim=0).float().contiguous()


# ---- all streams of equal length at once --------------------------------------------------------
# The per-stream procedure above issues a few hundred small launches per stream.  Streams of the
# same length (all KV heads of a sequence, and every sequence of the same context) share the seeded
# draws, so they train together as batched matrix products: the reference's own answer to the
# build time (pq_hsa/index/batched_build.py:82-167).


class _LazyGenerators:
    """One generator per problem, seeded as that problem's own call would seed it, created only
    for a problem that needs a draw of its own (an empty cluster) and first advanced past the
    draw of the start."""

    def __init__(self, seeds: list[int], n: int, shared_perm: bool) -> None:
        self.gens = [None] * len(seeds)
        self.seeds, self.n, self.shared_perm = seeds, n, shared_perm

    def get(self, s: int) -> torch.Generator:
        if self.gens[s] is None:
            g = torch.Generator(device="cpu")
            g.manual_seed(self.seeds[s])
            if self.shared_perm:
                torch.randperm(self.n, generator=g)
            self.gens[s] = g
        return self.gens[s]


def _nearest_batched(vectors: torch.Tensor, centroids: torch.Tensor, budget: int = 1 << 27,
                     unit_vectors: bool = False) -> torch.Tensor:
    """``vectors [S, N, D]``, ``centroids [S, K, D]`` -> nearest centroid per vector ``[S, N]``.
    ``unit_vectors``: the rows are unit directions (the coarse k-means); on the device, with
    D = 128, their nearest centroids then come from ``pqhsa_nearest_rows`` (matrix-core candidates,
    fixed-order fp32 decision) instead of a matrix of all products.  The subspace problems of the
    codebooks (D = 16 against 16 codewords) likewise go through ``pqhsa_nearest_codewords`` on the
    device.  Elsewhere: the reference's product form, with the arg-min fused on the device."""
    s, n, _ = vectors.shape
    cf = centroids.float()
    if (unit_vectors and vectors.is_cuda and vectors.shape[2] == 128 and vectors.dtype == torch.float32
            and vectors.is_contiguous() and 1 <= cf.shape[1] <= 4096 and n >= 128):
        from .. import ops
        return ops.nearest_rows(vectors, cf.contiguous())
    if (vectors.is_cuda and vectors.shape[2] == 16 and cf.shape[1] == 16 and vectors.dtype == torch.float32
            and vectors.is_contiguous() and s <= 65535):
        from .. import ops   # the subspace problems of the codebooks: one pass over the rows, no products
        return ops.nearest_codewords(vectors, cf.contiguous())
    half_sq = (cf * cf).sum(dim=2).unsqueeze(1)
    chunk = max(1024, budget // max(1, s * cf.shape[1]))
    out = torch.empty(s, n, dtype=torch.long, device=vectors.device)
    for i in range(0, n, chunk):
        v = vectors[:, i : i + chunk].float()
        dots = torch.bmm(v, cf.transpose(1, 2))
        if dots.is_cuda:  # one pass over the products (same arithmetic, ties to the lowest index)
            from .. import ops
            ops.nearest_from_products(dots, half_sq.reshape(s, -1), out[:, i : i + chunk])
        else:
            out[:, i : i + chunk] = (half_sq - 2.0 * dots).argmin(dim=2)
    return out


@functools.lru_cache(maxsize=64)
def _seeded_start(n: int, num_clusters: int, seed: int) -> torch.Tensor:
    """The first ``num_clusters`` entries of the seeded permutation of ``n`` (CPU generator, as the
    reference draws it).  Kept per (n, clusters, seed): every stream, sequence and layer of one
    length starts from the same draw, and a permutation of 131 072 takes the CPU about a millisecond."""
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed)
    return torch.randperm(n, generator=gen)[:num_clusters].clone()


def kmeans_l2_batched(vectors: torch.Tensor, num_clusters: int, *, max_iter: int, seed=0, eps: float = 1e-12,
                      unit_vectors: bool = False):
    """``kmeans_l2`` for ``S`` independent problems of one size, ``vectors [S, N, D]``: the seeded
    start (``seed``: one number for all problems, as S separate calls with one seed would draw,
    or one per problem) and the Lloyd iterations run as batched products; a problem whose
    assignment stops changing keeps its centroids, as the early exit of the per-stream loop does."""
    if vectors.ndim != 3:
        raise ValueError(f"vectors must be [S, N, D], got {tuple(vectors.shape)}")
    s, n, dim = vectors.shape
    if n == 0:
        raise ValueError("cannot train k-means with zero vectors")
    dev = vectors.device
    seeds = [int(x) for x in seed] if isinstance(seed, (list, tuple)) else [int(seed)] * s
    if len(seeds) != s:
        raise ValueError(f"{len(seeds)} seeds for {s} problems")
    lazy = _LazyGenerators(seeds, n, shared_perm=n >= num_clusters)
    if n >= num_clusters:
        start = torch.stack([_seeded_start(n, num_clusters, x) for x in seeds]).to(dev)               # [S, K]
        centroids = torch.gather(vectors, 1, start.unsqueeze(-1).expand(-1, -1, dim)).clone()
    else:
        # (every problem's own generator makes this draw: a later reseeding continues from it)
        extra = torch.stack([torch.randint(0, n, (num_clusters - n,), generator=lazy.get(i)) for i in range(s)]).to(dev)
        centroids = torch.cat([vectors, torch.gather(vectors, 1, extra.unsqueeze(-1).expand(-1, -1, dim))], dim=1).clone()
    assign = torch.zeros(s, n, dtype=torch.long, device=dev)
    live = torch.ones(s, dtype=torch.bool, device=dev)
    offsets = (torch.arange(s, device=dev) * num_clusters).unsqueeze(1)
    flat = vectors.reshape(s * n, dim).float()
    for _ in range(max_iter):
        nxt = _nearest_batched(vectors, centroids, unit_vectors=unit_vectors)
        same = (assign == nxt).all(dim=1)
        assign = torch.where(live.unsqueeze(1), nxt, assign)
        live = live & ~same
        if not bool(live.any()):
            break
        if num_clusters <= 64:
            # Few clusters (the 16 codewords of a subspace): row adds from a million keys would
            # queue up on 16 rows per problem.  The product with the 0/1 membership matrix adds
            # the same terms without that, and its column sums are the counts.
            # (the membership matrix [S, rows, K] is formed a slab of rows at a time, under the memory
            # budget of the assignment step; partial sums of slabs add up in fp32, another order than
            # one row add per key)
            ids = torch.arange(num_clusters, device=dev)
            rows = max(4096, (1 << 27) // max(1, s * num_clusters))
            sums = torch.zeros(s, num_clusters, dim, dtype=torch.float32, device=dev)
            counts = torch.zeros(s, num_clusters, dtype=torch.float32, device=dev)
            vf = flat.view(s, n, dim)
            for i in range(0, n, rows):
                member = (assign[:, i : i + rows].unsqueeze(-1) == ids).float()                    # [S, rows, K]
                sums += torch.bmm(member.transpose(1, 2), vf[:, i : i + rows])
                counts += member.sum(dim=1)
            sums, counts = sums.reshape(s * num_clusters, dim), counts.reshape(-1)
        else:
            where = (assign + offsets).reshape(-1)
            sums = torch.zeros(s * num_clusters, dim, dtype=torch.float32, device=dev)
            sums.index_add_(0, where, flat)
            counts = torch.zeros(s * num_clusters, dtype=torch.float32, device=dev)
            counts.index_add_(0, where, torch.ones(1, dtype=torch.float32, device=dev).expand(where.numel()))
        filled = counts > 0   # (float counts are exact below 2^24 keys per problem)
        sums = torch.where(filled.unsqueeze(1), sums / counts.unsqueeze(1).clamp_min(eps), sums)
        sums = sums.reshape(s, num_clusters, dim)
        empty = (~filled).reshape(s, num_clusters)
        if bool(empty.any()):
            for i in torch.nonzero(empty.any(dim=1)).flatten().tolist():
                if not bool(live[i]):
                    continue
                pick = torch.randint(0, n, (int(empty[i].sum().item()),), generator=lazy.get(i)).to(dev)
                sums[i][empty[i]] = vectors[i][pick].float()
        centroids = torch.where(live.view(s, 1, 1), sums.to(vectors.dtype), centroids)
    return centroids, _nearest_batched(vectors, centroids, unit_vectors=unit_vectors)


def train_ivfpq_batched(keys: torch.Tensor, *, num_lists: int, num_subspaces: int = 8, num_codes: int = 16,
                        coarse_iter: int = 1, pq_iter: int = 2, seed: int = 0, eps: float = 1e-12):
    """``train_ivfpq`` for ``S`` streams of one length at once: ``keys [S, N, D]`` ->
    ``(coarse [S, L', D], codebooks [S, M, num_codes, D/M])``, fp32."""
    if keys.ndim != 3 or keys.shape[1] == 0:
        raise ValueError("cannot build IVF-PQ index with zero keys")
    if keys.shape[2] % num_subspaces != 0:
        raise ValueError(f"dim={keys.shape[2]} must be divisible by num_subspaces={num_subspaces}")
    k32 = keys.float()
    norms = torch.linalg.vector_norm(k32, dim=-1).clamp_min(eps)
    dirs = k32 / norms.unsqueeze(-1)
    lists = min(int(num_lists), dirs.shape[1])
    coarse, assign = kmeans_l2_batched(dirs, lists, max_iter=coarse_iter, seed=seed, eps=eps, unit_vectors=True)
    resid = dirs - torch.gather(coarse, 1, assign.unsqueeze(-1).expand(-1, -1, dirs.shape[2]))
    sub = keys.shape[2] // num_subspaces
    chunks = resid.reshape(resid.shape[0], resid.shape[1], num_subspaces, sub)
    # the subspaces of all streams are one batch of problems, each with its own seed
    streams = resid.shape[0]
    problems = chunks.permute(0, 2, 1, 3).reshape(streams * num_subspaces, resid.shape[1], sub)
    books, _ = kmeans_l2_batched(problems, num_codes, max_iter=pq_iter,
                                 seed=[seed + 10_000 + m for _ in range(streams) for m in range(num_subspaces)], eps=eps)
    return coarse.float().contiguous(), books.reshape(streams, num_subspaces, num_codes, sub).float().contiguous()
