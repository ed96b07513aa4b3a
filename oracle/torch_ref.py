"""Torch-CPU restatement of the reference's PQ-HSA decode path.  TEST INFRASTRUCTURE.

This follows the reference op for op (same torch calls where the reference's arithmetic is
torch's: ``bmm``, ``matmul``, ``cdist().argmin``, ``topk``, ``exp``, ``scatter_add_``), so it is
the stand-in for the reference wherever the reference itself cannot run (the GPU box), and it
is the ``cpu_baseline`` timed by ``bench.py``.  Only ``tests/``, ``__graft_entry__.smoke()`` and
that bench leg may import it.  It is pinned against the golden fixtures written by
``tests/golden/make_fixtures.py`` from the real reference and against closed forms
(tests/test_oracle_*.py).

Reference files followed (relative to the reference tree):
  pack_4bit_codes / unpack_4bit_codes   pq_hsa/index/packing.py:6-34, 37-60
  kmeans_l2                              pq_hsa/index/kmeans.py:108-131, 134-227
  train_index                            pq_hsa/index/ivfpq.py:275-348, pq_hsa/index/pq.py:47-95
  encode_with_codebooks                  pq_hsa/index/ivfpq.py:350-433, 1001-1016, 1052-1059;
                                         pq_hsa/index/pq.py:97-115
  value_centroids                        pq_hsa/attention/kv_cache.py:688-728, 766-776
  approximate_scores                     pq_hsa/index/ivfpq.py:709-727, 1061-1118, 1179-1190,
                                         1238-1254; pq_hsa/index/pq.py:190-217;
                                         pq_hsa/kernels/lut_scan.py:92-114
  hybrid_forward_many                    pq_hsa/attention/sparse_attention.py:245-335, 759-1013
  RefStream                              pq_hsa/attention/kv_cache.py:195-314, 1160-1201;
                                         pq_hsa/attention/sparse_attention.py:219-227
  gather_paged / gather_paged_range /
  gather_paged_at                        benchmarks/vllm_backend/paged_kv_fa.py:44-57, 95-156
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field

import torch


# --------------------------------------------------------------------------- packing
def pack_4bit_codes(codes: torch.Tensor) -> torch.Tensor:
    if codes.ndim != 2:
        raise ValueError(f"codes must be [N, M], got {tuple(codes.shape)}")
    if codes.numel() > 0 and (codes.min() < 0 or codes.max() > 15):
        raise ValueError("4-bit packing requires codes in [0, 15]")
    c = codes.to(torch.uint8)
    n, m = c.shape
    if m % 2 == 1:
        c = torch.cat([c, torch.zeros(n, 1, dtype=torch.uint8)], dim=1)
    return (c[:, 0::2] & 0x0F) | (c[:, 1::2] << 4)


def unpack_4bit_codes(packed: torch.Tensor, num_subspaces: int) -> torch.Tensor:
    if packed.ndim != 2 or packed.shape[1] != (num_subspaces + 1) // 2:
        raise ValueError("packed codes must be [N, ceil(M/2)]")
    out = torch.empty(packed.shape[0], num_subspaces, dtype=torch.long)
    out[:, 0::2] = (packed[:, : (num_subspaces + 1) // 2] & 0x0F).long()
    if num_subspaces > 1:
        out[:, 1::2] = (packed[:, : num_subspaces // 2] >> 4).long()
    return out


def packed_to_words(packed: torch.Tensor) -> torch.Tensor:
    """[N, 4] uint8 -> [N] int64 holding the little-endian 32-bit word (nibble m at bit 4m)."""
    p = packed.long()
    return p[:, 0] | (p[:, 1] << 8) | (p[:, 2] << 16) | (p[:, 3] << 24)


# --------------------------------------------------------------------------- k-means
def _nearest_centroids(vectors: torch.Tensor, centroids: torch.Tensor, chunk: int = 16384) -> torch.Tensor:
    cf = centroids.float()
    csq = (cf * cf).sum(dim=1)
    out = torch.empty(vectors.shape[0], dtype=torch.long)
    for s in range(0, vectors.shape[0], chunk):
        v = vectors[s : s + chunk].float()
        out[s : s + chunk] = (csq.unsqueeze(0) - 2.0 * v.matmul(cf.t())).argmin(dim=1)
    return out


def kmeans_l2(vectors: torch.Tensor, num_clusters: int, *, max_iter: int, seed: int, eps: float = 1e-12):
    n, dim = vectors.shape
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed)
    if n >= num_clusters:
        perm = torch.randperm(n, generator=gen)
        centroids = vectors[perm[:num_clusters]].clone()
    else:
        extra = torch.randint(0, n, (num_clusters - n,), generator=gen)
        centroids = torch.cat([vectors, vectors[extra]], dim=0).clone()
    assign = torch.zeros(n, dtype=torch.long)
    for _ in range(max_iter):
        nxt = _nearest_centroids(vectors, centroids)
        if torch.equal(assign, nxt):
            assign = nxt
            break
        assign = nxt
        new = torch.zeros(num_clusters, dim, dtype=torch.float32)
        counts = torch.bincount(assign, minlength=num_clusters).float()
        new.index_add_(0, assign, vectors.float())
        non_empty = counts > 0
        new[non_empty] /= counts[non_empty].unsqueeze(1).clamp_min(eps)
        if (~non_empty).any():
            repl = torch.randint(0, n, (int((~non_empty).sum().item()),), generator=gen)
            new[~non_empty] = vectors[repl].float()
        centroids = new.to(vectors.dtype)
    return centroids, _nearest_centroids(vectors, centroids)


# --------------------------------------------------------------------------- index
@dataclass
class RefIndex:
    coarse: torch.Tensor            # [L, D]
    codebooks: torch.Tensor         # [M, 16, sd]
    list_ids: torch.Tensor          # [N] int64
    packed: torch.Tensor            # [N, M/2] uint8
    norms: torch.Tensor             # [N]
    eps: float = 1e-12

    @property
    def num_subspaces(self) -> int:
        return int(self.codebooks.shape[0])


def project(x: torch.Tensor, eps: float = 1e-12):
    norms = torch.linalg.vector_norm(x.float(), dim=-1).to(x.dtype).clamp_min(eps)
    return x / norms.unsqueeze(-1), norms


def pq_encode(vectors: torch.Tensor, codebooks: torch.Tensor) -> torch.Tensor:
    m, _, sd = codebooks.shape
    chunks = vectors.reshape(vectors.shape[0], m, sd)
    cols = [torch.cdist(chunks[:, s].float(), codebooks[s].float(), p=2).argmin(dim=1) for s in range(m)]
    return torch.stack(cols, dim=1)


def train_index(keys: torch.Tensor, *, num_lists: int, num_subspaces: int = 8, coarse_iter: int = 1,
                pq_iter: int = 2, seed: int = 0, eps: float = 1e-12) -> RefIndex:
    dirs, norms = project(keys, eps)
    num_lists = min(num_lists, dirs.shape[0])
    coarse, list_ids = kmeans_l2(dirs, num_lists, max_iter=coarse_iter, seed=seed, eps=eps)
    resid = dirs - coarse[list_ids]
    sd = keys.shape[1] // num_subspaces
    chunks = resid.reshape(resid.shape[0], num_subspaces, sd)
    books = []
    for s in range(num_subspaces):
        c, _ = kmeans_l2(chunks[:, s].contiguous(), 16, max_iter=pq_iter, seed=seed + 10_000 + s, eps=eps)
        books.append(c)
    codebooks = torch.stack(books, dim=0)
    codes = pq_encode(resid, codebooks)
    return RefIndex(coarse, codebooks, list_ids, pack_4bit_codes(codes), norms, eps)


def encode_rows(keys: torch.Tensor, coarse: torch.Tensor, codebooks: torch.Tensor, eps: float = 1e-12):
    dirs, norms = project(keys, eps)
    list_ids = torch.cdist(dirs.float(), coarse.float(), p=2).argmin(dim=1)
    codes = pq_encode(dirs - coarse[list_ids], codebooks)
    return norms, list_ids, pack_4bit_codes(codes)


def encode_with_codebooks(keys, coarse, codebooks, eps: float = 1e-12) -> RefIndex:
    norms, list_ids, packed = encode_rows(keys, coarse, codebooks, eps)
    return RefIndex(coarse, codebooks, list_ids, packed, norms, eps)


def index_add(index: RefIndex, keys: torch.Tensor) -> torch.Tensor:
    norms, list_ids, packed = encode_rows(keys, index.coarse, index.codebooks, index.eps)
    index.list_ids = torch.cat([index.list_ids, list_ids])
    index.norms = torch.cat([index.norms, norms])
    index.packed = torch.cat([index.packed, packed])
    return list_ids


def _ema_towards_means(table: torch.Tensor, rows: torch.Tensor, ids: torch.Tensor, lr: float, eps: float) -> torch.Tensor:
    """Entries of ``table`` that own rows move to (1 - lr) * entry + lr * mean(rows they own); the
    others stay (pq_hsa/index/ivfpq.py:1159-1177 for coarse centroids, pq_hsa/index/pq.py:155-170
    for the codewords of one subspace)."""
    sums = torch.zeros_like(table)
    counts = torch.bincount(ids, minlength=table.shape[0]).to(rows.dtype)
    sums.index_add_(0, ids, rows)
    non_empty = counts > 0
    means = sums[non_empty] / counts[non_empty].unsqueeze(1).clamp_min(eps)
    out = table.clone()
    out[non_empty] = (1.0 - lr) * table[non_empty] + lr * means
    return out


def online_refresh(index: RefIndex, keys: torch.Tensor, update_keys: torch.Tensor, lr: float = 0.05) -> RefIndex:
    """IVFPQIndex.online_refresh (pq_hsa/index/ivfpq.py:647-707) with
    ProductQuantizer.update_codebooks_ema (pq_hsa/index/pq.py:117-173): the update keys move the
    coarse centroids they are assigned to, are assigned again, their residuals move the codewords
    they are nearest to (assignments under the codebooks as they were), and then every key is
    re-assigned and re-encoded under the moved tables."""
    eps = index.eps
    dirs, norms = project(keys, eps)
    upd, _ = project(update_keys, eps)
    coarse, books = index.coarse, index.codebooks
    if upd.shape[0] > 0:
        lids = torch.cdist(upd.float(), coarse.float(), p=2).argmin(dim=1)
        coarse = _ema_towards_means(coarse, upd, lids, lr, eps)
        lids = torch.cdist(upd.float(), coarse.float(), p=2).argmin(dim=1)
        resid = upd - coarse[lids]
        m, _, sd = books.shape
        chunks = resid.reshape(resid.shape[0], m, sd)
        moved = books.clone()
        for s in range(m):
            near = torch.cdist(chunks[:, s].float(), books[s].float(), p=2).argmin(dim=1)
            moved[s] = _ema_towards_means(books[s], chunks[:, s], near, lr, eps)
        books = moved
    list_ids = torch.cdist(dirs.float(), coarse.float(), p=2).argmin(dim=1)
    codes = pq_encode(dirs - coarse[list_ids], books)
    return RefIndex(coarse, books, list_ids, pack_4bit_codes(codes), norms, eps)


def value_sums(values: torch.Tensor, list_ids: torch.Tensor, num_lists: int):
    sums = torch.zeros(num_lists, values.shape[1], dtype=values.dtype)
    sums.index_add_(0, list_ids, values)
    counts = torch.bincount(list_ids, minlength=num_lists).to(values.dtype)
    return sums, counts


def centroids_from_sums(sums: torch.Tensor, counts: torch.Tensor) -> torch.Tensor:
    out = torch.zeros_like(sums)
    ne = counts > 0
    out[ne] = sums[ne] / counts[ne].unsqueeze(1)
    return out


def value_centroids(values, list_ids, num_lists):
    return centroids_from_sums(*value_sums(values, list_ids, num_lists))


# --------------------------------------------------------------------------- scoring
def compute_lut(qh: torch.Tensor, codebooks: torch.Tensor) -> torch.Tensor:
    m, _, sd = codebooks.shape
    if qh.ndim == 1:
        return torch.bmm(codebooks, qh.reshape(m, sd).unsqueeze(2)).squeeze(2)
    q = qh.reshape(qh.shape[0], m, sd)
    return torch.bmm(q.permute(1, 0, 2), codebooks.transpose(1, 2)).permute(1, 0, 2)


def score_packed(packed: torch.Tensor, lut: torch.Tensor, num_subspaces: int) -> torch.Tensor:
    if lut.ndim == 2:
        scores = torch.zeros(packed.shape[0], dtype=lut.dtype)
        for s in range(num_subspaces):
            byte = packed[:, s // 2]
            code = ((byte >> 4) if s % 2 == 1 else (byte & 0x0F)).long()
            scores += lut[s].gather(0, code)
        return scores
    scores = torch.zeros(lut.shape[0], packed.shape[0], dtype=lut.dtype)
    for s in range(num_subspaces):
        byte = packed[:, s // 2]
        code = ((byte >> 4) if s % 2 == 1 else (byte & 0x0F)).long()
        scores += lut[:, s, :].gather(1, code.unsqueeze(0).expand(lut.shape[0], -1))
    return scores


def approximate_scores(index: RefIndex, query: torch.Tensor) -> torch.Tensor:
    """query [D] -> [N]; query [G, D] -> [G, N] (raw scores, before the attention scale)."""
    qn = torch.linalg.vector_norm(query.float(), dim=-1).to(query.dtype).clamp_min(index.eps)
    qh = query / qn if query.ndim == 1 else query / qn.unsqueeze(-1)
    scores = score_packed(index.packed, compute_lut(qh, index.codebooks), index.num_subspaces)
    if query.ndim == 1:
        scores = scores + index.coarse.matmul(qh)[index.list_ids]
        return scores * qn * index.norms
    scores = scores + qh.matmul(index.coarse.T)[:, index.list_ids]
    return scores * qn.unsqueeze(-1) * index.norms.unsqueeze(0)


def resolve_topk(n: int, fraction: float) -> int:
    return min(max(int(math.ceil(n * fraction)), 0), n)


# --------------------------------------------------------------------------- attention
def hybrid_forward_many(queries, keys, values, *, sink_end: int, retrieval_end: int, index: RefIndex,
                        vbar: torch.Tensor, fraction: float, scale: float, return_details: bool = False):
    """queries [G, D]; keys/values [len, D] of one KV head."""
    length = keys.shape[0]
    full_idx = torch.cat([torch.arange(0, sink_end), torch.arange(retrieval_end, length)])
    a = approximate_scores(index, queries) * scale                                   # [G, N]
    n = a.shape[1]
    k = resolve_topk(n, fraction)
    top_a, top_local = torch.topk(a, k=k, dim=1, sorted=True)
    top_global = top_local + sink_end
    fl = queries.matmul(keys[full_idx].T) * scale
    g = queries.shape[0]
    xk = keys[top_global.reshape(-1)].reshape(g, k, -1)
    xv = values[top_global.reshape(-1)].reshape(g, k, -1)
    xl = torch.bmm(xk, queries.unsqueeze(-1)).squeeze(-1) * scale
    row_max = None
    if full_idx.numel() > 0:
        row_max = fl.max(dim=1).values
    if n > 0:
        amax = top_a[:, 0] if k > 0 else a.max(dim=1).values
        row_max = amax if row_max is None else torch.maximum(row_max, amax)
    if k > 0:
        xmax = xl.max(dim=1).values
        row_max = xmax if row_max is None else torch.maximum(row_max, xmax)
    fe = torch.exp(fl - row_max[:, None])
    re = torch.exp(a - row_max[:, None])
    oe = re.gather(1, top_local)
    xe = torch.exp(xl - row_max[:, None])
    den = fe.sum(dim=1) + re.sum(dim=1) - oe.sum(dim=1) + xe.sum(dim=1)
    den = den.clamp_min(torch.finfo(den.dtype).tiny)
    out = (fe / den[:, None]).matmul(values[full_idx])
    if k > 0:
        out = out + torch.bmm((xe / den[:, None]).unsqueeze(1), xv).squeeze(1)
    mass = torch.zeros(g, vbar.shape[0], dtype=a.dtype)
    mass.scatter_add_(1, index.list_ids.unsqueeze(0).expand(g, -1), re)
    if k > 0:
        mass.scatter_add_(1, index.list_ids[top_local], -oe)
    out = out + (mass / den[:, None]).matmul(vbar)
    if return_details:
        return out, {"logits": a, "topk_local": top_local, "topk_logit": top_a, "mass": mass, "den": den,
                     "row_max": row_max}
    return out


@dataclass
class RefStream:
    """One (sequence, KV head) stream: full K/V + index over the retrieval region, with the
    incremental (interval-1) and deferred append behaviours of the reference cache."""

    sink: int
    local: int
    fraction: float
    scale: float
    num_lists: int = 512
    coarse_iter: int = 1
    pq_iter: int = 2
    seed: int = 0
    update_interval: int = 1
    strategy: str = "incremental"
    keys: torch.Tensor | None = None
    values: torch.Tensor | None = None
    index: RefIndex | None = None
    vbar: torch.Tensor | None = None
    indexed_length: int = 0
    pending: int = 0
    _sums: torch.Tensor | None = field(default=None, repr=False)
    _counts: torch.Tensor | None = field(default=None, repr=False)

    def regions(self) -> tuple[int, int]:
        length = self.keys.shape[0]
        sink_end = min(self.sink, length)
        idx_len = min(self.indexed_length, length)
        retrieval_end = max(sink_end, idx_len - self.local) if self.local > 0 else max(sink_end, idx_len)
        return sink_end, retrieval_end

    def build(self, keys, values, *, coarse=None, codebooks=None) -> "RefStream":
        self.keys, self.values = keys.clone(), values.clone()
        self.indexed_length = keys.shape[0]
        s, e = self.regions()
        if coarse is not None:
            self.index = encode_with_codebooks(self.keys[s:e], coarse, codebooks)
        else:
            self.index = train_index(self.keys[s:e], num_lists=self.num_lists, coarse_iter=self.coarse_iter,
                                     pq_iter=self.pq_iter, seed=self.seed)
        self.vbar = value_centroids(self.values[s:e], self.index.list_ids, self.index.coarse.shape[0])
        self._sums = self._counts = None
        return self

    def append(self, key, value) -> None:
        self.keys = torch.cat([self.keys, key[None]])
        self.values = torch.cat([self.values, value[None]])
        self.pending += 1
        if self.pending < self.update_interval or self.strategy == "deferred":
            return
        _, old_end = self.regions()
        self.indexed_length = self.keys.shape[0]
        self.pending = 0
        s, new_end = self.regions()
        if new_end == old_end:
            return
        list_ids = index_add(self.index, self.keys[old_end:new_end])
        num_lists = self.index.coarse.shape[0]
        if self._sums is None:
            self._sums, self._counts = value_sums(self.values[s:new_end], self.index.list_ids, num_lists)
        else:
            self._sums.index_add_(0, list_ids, self.values[old_end:new_end])
            self._counts += torch.bincount(list_ids, minlength=num_lists).to(self.values.dtype)
        self.vbar = centroids_from_sums(self._sums, self._counts)

    def apply_pending_index_update(self, lr: float = 0.05) -> bool:
        """The deferred strategy's flush (SparseKVCache.apply_pending_index_update ->
        _refresh_index_now -> _online_refresh_index, pq_hsa/attention/kv_cache.py:266-314, 666-676):
        the tokens appended since the last index update join the indexed length, the keys that enter
        the retrieval region are the update batch of an online refresh over all retrieval keys, and
        the per-list value means are rebuilt."""
        if self.strategy != "deferred" or self.pending == 0:
            return False
        _, old_end = self.regions()
        self.indexed_length = self.keys.shape[0]
        self.pending = 0
        s, new_end = self.regions()
        if new_end == old_end:
            return True
        self.index = online_refresh(self.index, self.keys[s:new_end], self.keys[old_end:new_end], lr)
        self.vbar = value_centroids(self.values[s:new_end], self.index.list_ids, self.index.coarse.shape[0])
        self._sums = self._counts = None
        return True

    def forward_many(self, queries, **kw):
        s, e = self.regions()
        return hybrid_forward_many(queries, self.keys, self.values, sink_end=s, retrieval_end=e,
                                   index=self.index, vbar=self.vbar, fraction=self.fraction,
                                   scale=self.scale, **kw)


# --------------------------------------------------------------------------- paged readers
def split_kv_cache(kv_cache: torch.Tensor):
    if kv_cache.dim() == 5:
        return kv_cache[0], kv_cache[1]
    if kv_cache.dim() == 4:
        d = kv_cache.shape[-1] // 2
        k, v = kv_cache.transpose(1, 2).split(d, dim=-1)
        return k, v
    raise ValueError(f"unsupported kv_cache shape {tuple(kv_cache.shape)}")


def gather_paged(kv_cache, block_table, seq_len: int):
    kc, vc = split_kv_cache(kv_cache)
    bs, h, d = kc.shape[1], kc.shape[2], kc.shape[3]
    nb = (seq_len + bs - 1) // bs
    blocks = block_table[:nb].long()
    k = kc[blocks].reshape(-1, h, d)[:seq_len].permute(1, 0, 2).unsqueeze(0).contiguous()
    v = vc[blocks].reshape(-1, h, d)[:seq_len].permute(1, 0, 2).unsqueeze(0).contiguous()
    return k, v


def gather_paged_range(kv_cache, block_table, start: int, end: int):
    kc, vc = split_kv_cache(kv_cache)
    bs, h, d = kc.shape[1], kc.shape[2], kc.shape[3]
    first, last = start // bs, (end - 1) // bs
    blocks = block_table[first : last + 1].long()
    row0 = start - first * bs
    k = kc[blocks].reshape(-1, h, d)[row0 : row0 + end - start].permute(1, 0, 2).contiguous()
    v = vc[blocks].reshape(-1, h, d)[row0 : row0 + end - start].permute(1, 0, 2).contiguous()
    return k, v


def gather_paged_at(kv_cache, block_table, token_indices: torch.Tensor):
    kc, vc = split_kv_cache(kv_cache)
    bs = kc.shape[1]
    h = token_indices.shape[0]
    blk = torch.div(token_indices, bs, rounding_mode="floor")
    rows = token_indices - blk * bs
    ids = block_table[blk.reshape(-1)].reshape(blk.shape).long()
    heads = torch.arange(h).view(h, *([1] * (token_indices.ndim - 1))).expand_as(token_indices)
    return kc[ids, rows.long(), heads], vc[ids, rows.long(), heads]
