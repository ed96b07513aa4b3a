"""Torch-facing wrappers of the C ABI: tensors in, tensors out, kernels on the current stream.

PyTorch only provides device memory and the stream here; every computation below is one of
the HIP kernels behind ``libpqhsa.so``.
"""

from __future__ import annotations

import ctypes
import math
from dataclasses import dataclass

import torch

from . import _lib
from ._lib import Index, KvView, Select

HEAD_DIM = 128
SUBSPACES = 8
CODES = 16
SUBDIM = HEAD_DIM // SUBSPACES
EPS = 1e-12


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return _lib.F32
    if dtype == torch.bfloat16:
        return _lib.BF16
    if dtype == torch.float16:
        return _lib.F16
    raise ValueError(f"unsupported dtype {dtype}")


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def _need_cuda(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise ValueError("PQ-HSA kernels need device tensors; there is no CPU path")


def padded_groups(groups: int) -> int:
    p = 1
    while p < groups:
        p <<= 1
    return p


def resolve_topk(n: int, fraction: float | None, topk: int) -> int:
    """k = min(max(ceil(n * fraction), 0), n) or min(topk, n)."""
    if fraction is not None and fraction > 0:
        k = int(math.ceil(n * fraction))
    else:
        k = int(topk)
    return min(max(k, 0), n)


# --------------------------------------------------------------------------- K/V views
@dataclass
class KvSource:
    """A ``pqhsa_kv_view`` plus the tensors it points into (kept alive)."""

    view: KvView
    keep: tuple
    dtype: torch.dtype
    batch: int
    kv_heads: int

    def ref(self):
        return ctypes.byref(self.view)


def kv_contiguous(keys: torch.Tensor, values: torch.Tensor) -> KvSource:
    """keys/values ``[B, H, cap, 128]`` with unit stride in the last dim and equal strides."""
    _need_cuda(keys, values)
    if keys.ndim != 4 or values.ndim != 4 or keys.shape[-1] != HEAD_DIM or values.shape[-1] != HEAD_DIM:
        raise ValueError(f"keys/values must be [B, H, S, {HEAD_DIM}]")
    if keys.stride() != values.stride() or keys.stride(-1) != 1 or keys.dtype != values.dtype:
        raise ValueError("keys and values must share dtype and strides, last dim contiguous")
    v = KvView()
    v.k_base, v.v_base = keys.data_ptr(), values.data_ptr()
    v.dtype, v.paged = dtype_code(keys.dtype), 0
    v.stride_seq, v.stride_head, v.stride_tok, v.stride_block = keys.stride(0), keys.stride(1), keys.stride(2), 0
    v.block_size, v.max_blocks, v.block_table = 0, 0, None
    return KvSource(v, (keys, values), keys.dtype, keys.shape[0], keys.shape[1])


def kv_paged(kv_cache: torch.Tensor, block_table: torch.Tensor) -> KvSource:
    """Paged cache in either layout: 5-D ``[2, blocks, bs, H, D]`` or 4-D ``[blocks, H, bs, 2*D]``."""
    _need_cuda(kv_cache, block_table)
    if block_table.dtype != torch.int32 or block_table.ndim != 2 or not block_table.is_contiguous():
        raise ValueError("block_table must be a contiguous int32 [B, max_blocks] tensor")
    v = KvView()
    esz = kv_cache.element_size()
    if kv_cache.dim() == 5:
        if kv_cache.shape[0] != 2 or kv_cache.shape[-1] != HEAD_DIM or kv_cache.stride(-1) != 1:
            raise ValueError(f"unsupported 5-D kv_cache shape {tuple(kv_cache.shape)}")
        v.k_base = kv_cache.data_ptr()
        v.v_base = kv_cache.data_ptr() + kv_cache.stride(0) * esz
        v.stride_block, v.stride_tok, v.stride_head = kv_cache.stride(1), kv_cache.stride(2), kv_cache.stride(3)
        v.block_size, heads = kv_cache.shape[2], kv_cache.shape[3]
    elif kv_cache.dim() == 4:
        if kv_cache.shape[-1] != 2 * HEAD_DIM or kv_cache.stride(-1) != 1:
            raise ValueError(f"unsupported 4-D kv_cache shape {tuple(kv_cache.shape)}")
        v.k_base = kv_cache.data_ptr()
        v.v_base = kv_cache.data_ptr() + HEAD_DIM * esz
        v.stride_block, v.stride_head, v.stride_tok = kv_cache.stride(0), kv_cache.stride(1), kv_cache.stride(2)
        v.block_size, heads = kv_cache.shape[2], kv_cache.shape[1]
    else:
        raise ValueError(f"unsupported FLASH_ATTN kv_cache shape {tuple(kv_cache.shape)}")
    v.dtype, v.paged, v.stride_seq = dtype_code(kv_cache.dtype), 1, 0
    v.max_blocks, v.block_table = block_table.shape[1], block_table.data_ptr()
    return KvSource(v, (kv_cache, block_table), kv_cache.dtype, block_table.shape[0], heads)


# --------------------------------------------------------------------------- device index
class DeviceIndex:
    """Device-resident IVF-PQ index of B x H streams (structure of arrays, spare capacity).

    Stored keys sit in two regions: the first ``n_sorted`` positions are ordered by list id
    (``pos`` maps a position back to the key's retrieval-local index), keys appended later
    follow in insertion order until ``finalize_layout`` sorts everything again.  A fixed random
    subset of the stored keys is kept in the ``s_*`` arrays for the threshold estimate.
    """

    SAMPLE_RATE = 32
    SAMPLE_MIN = 4096
    SAMPLE_MAX = 32768   # the threshold kernel keeps the sampled keys of one row in LDS

    def __init__(self, batch: int, kv_heads: int, num_lists: int, n_cap: int, device) -> None:
        n_cap = max(8, (int(n_cap) + 7) // 8 * 8)
        bh = batch * kv_heads
        self.batch, self.kv_heads, self.num_lists, self.n_cap = batch, kv_heads, int(num_lists), n_cap
        self.device = torch.device(device)
        dev = self.device
        self.codes = torch.zeros(bh, n_cap, dtype=torch.int32, device=dev)       # bit pattern of u32
        self.list_ids = torch.zeros(bh, n_cap, dtype=torch.int16, device=dev)    # bit pattern of u16
        self.norms = torch.zeros(bh, n_cap, dtype=torch.float32, device=dev)
        self.pos = torch.arange(n_cap, dtype=torch.int32, device=dev).repeat(bh, 1)
        self.coarse = torch.zeros(bh, num_lists, HEAD_DIM, dtype=torch.float32, device=dev)
        self.codebooks = torch.zeros(bh, SUBSPACES, CODES, SUBDIM, dtype=torch.float32, device=dev)
        self.vbar = torch.zeros(bh, num_lists, HEAD_DIM, dtype=torch.float32, device=dev)
        self.vsum = torch.zeros(bh, num_lists, HEAD_DIM, dtype=torch.float32, device=dev)
        self.vcount = torch.zeros(bh, num_lists, dtype=torch.float32, device=dev)
        self.n_idx = torch.zeros(batch, dtype=torch.int32, device=dev)
        self.n_sorted = torch.zeros(batch, dtype=torch.int32, device=dev)
        self.s_n = torch.zeros(batch, dtype=torch.int32, device=dev)
        self.s_cap = max(8, (self.sample_size(n_cap) + 7) // 8 * 8)
        self.s_codes = torch.zeros(bh, self.s_cap, dtype=torch.int32, device=dev)
        self.s_list_ids = torch.zeros(bh, self.s_cap, dtype=torch.int16, device=dev)
        self.s_norms = torch.zeros(bh, self.s_cap, dtype=torch.float32, device=dev)
        self.n_host = [0] * batch          # host mirrors
        self.n_sorted_host = [0] * batch
        self._struct = None

    @classmethod
    def regroup(cls, sources, n_cap: int) -> "DeviceIndex":
        """A new index whose sequence b is sequence ``seq`` of ``index`` for ``(index, seq) =
        sources[b]``: the rows are copied on the device, nothing is re-encoded.  All sources share
        KV heads and device; the new tables are as wide as the widest source's and a sequence from
        a narrower one leaves the rest unused (``pad_lists``).  ``n_cap`` is raised to the longest
        sequence if smaller."""
        first = sources[0][0]
        h = first.kv_heads
        if any(ix.kv_heads != h or ix.device != first.device for ix, _ in sources):
            raise ValueError("regroup: the source indexes differ in KV heads or device")
        lists = max(ix.num_lists for ix, _ in sources)
        n_cap = max(int(n_cap), max(ix.n_host[seq] for ix, seq in sources))
        new = cls(len(sources), h, lists, n_cap, first.device)
        for b, (ix, seq) in enumerate(sources):
            src, dst = slice(seq * h, (seq + 1) * h), slice(b * h, (b + 1) * h)
            n = ix.n_host[seq]
            for name in ("codes", "list_ids", "norms", "pos"):
                getattr(new, name)[dst, :n].copy_(getattr(ix, name)[src, :n])
            skeep = min(ix.s_cap, new.s_cap)
            for name in ("s_codes", "s_list_ids", "s_norms"):
                getattr(new, name)[dst, :skeep].copy_(getattr(ix, name)[src, :skeep])
            for name in ("coarse", "vbar", "vsum", "vcount"):
                getattr(new, name)[dst, : ix.num_lists].copy_(getattr(ix, name)[src])
            new.pad_lists(dst, ix.num_lists)
            new.codebooks[dst].copy_(ix.codebooks[src])
            new.s_n[b : b + 1].copy_(ix.s_n[seq : seq + 1])
            new.n_sorted_host[b] = ix.n_sorted_host[seq]
        new.set_counts([ix.n_host[seq] for ix, seq in sources])
        return new

    # Every component of an unused coarse centroid.  Keys are indexed by their direction (unit
    # vectors) and real centroids are means of directions, so a real centroid is within distance 2
    # of any key and one of these is about 1e5 away: it is never the nearest, its list stays empty
    # and its per-list sums stay zero.  Products with it stay far inside the fp32 range.
    PAD_CENTROID = 1.0e4

    def pad_lists(self, rows: slice, used: int) -> None:
        """Streams ``rows`` use only the first ``used`` coarse lists."""
        if used < self.num_lists:
            self.coarse[rows, used:] = self.PAD_CENTROID

    @classmethod
    def sample_size(cls, n: int) -> int:
        # a whole number of 1024-key slots (the threshold kernel holds the sample in registers, one
        # slot per thread), as close to n / SAMPLE_RATE as that allows
        want = max((n // cls.SAMPLE_RATE + 512) // 1024 * 1024, cls.SAMPLE_MIN)
        return min(n, cls.SAMPLE_MAX, want)

    @property
    def n_max(self) -> int:
        return max(self.n_host) if self.n_host else 0

    @property
    def n_mean(self) -> int:
        """Mean indexed keys per sequence (host mirror): the hint that sizes the scan's tiles."""
        return (sum(self.n_host) + len(self.n_host) - 1) // len(self.n_host) if self.n_host else 0

    def set_counts(self, counts) -> None:
        """Keys stored per sequence (a fresh encode leaves them in insertion order: nothing is
        sorted, nothing sampled, until ``finalize_layout``)."""
        self.n_host = [int(c) for c in counts]
        if max(self.n_host, default=0) > self.n_cap:
            raise ValueError("index capacity exceeded")
        self.n_sorted_host = [min(s, n) for s, n in zip(self.n_sorted_host, self.n_host)]
        self.n_idx.copy_(torch.tensor(self.n_host, dtype=torch.int32))
        self.n_sorted.copy_(torch.tensor(self.n_sorted_host, dtype=torch.int32))

    def note_appended(self, counts) -> None:
        """Host-side bookkeeping after a fused append + decode step: the device already holds the
        new counts (the step stored them), only the host mirror moves."""
        self.n_host = [n + int(c) for n, c in zip(self.n_host, counts)]
        if max(self.n_host, default=0) > self.n_cap:
            raise ValueError("index capacity exceeded")

    def reset_layout(self) -> None:
        """Declare the stored keys to be in insertion order again (after a bulk re-encode)."""
        self.n_sorted_host = [0] * self.batch
        self.n_sorted.zero_()
        self.s_n.zero_()
        self.pos.copy_(torch.arange(self.n_cap, dtype=torch.int32, device=self.device).expand_as(self.pos))

    def finalize_layout(self, seed: int = 0) -> None:
        """Order every stream's stored keys by list id (stable, so keys of a list keep their
        insertion order) and draw the sampled subset: one key from each of ``sample_size(n)``
        equal strata of the list-ordered keys, the place inside a stratum from an integer hash of
        (seed, sequence, stratum).  Torch ops on the device, off the decode path; nothing waits
        for the host.  Sequences of one length that follow each other are ordered in one go."""
        h = self.kv_heads
        b = 0
        while b < self.batch:
            n = self.n_host[b]
            e = b + 1
            while e < self.batch and self.n_host[e] == n:
                e += 1
            if n > 0:
                rows = slice(b * h, e * h)
                lids = self.list_ids[rows, :n].to(torch.int32) & 0xFFFF
                order = torch.argsort(lids, dim=1, stable=True)
                for t in (self.codes, self.list_ids, self.norms, self.pos):
                    t[rows, :n] = torch.gather(t[rows, :n], 1, order)
                ns = self.sample_size(n)
                seqs = torch.arange(b, e, device=self.device, dtype=torch.int64).repeat_interleave(h).unsqueeze(1)
                pick = self._sample_positions(n, ns, int(seed), seqs)                 # [(e - b) * h, ns]
                self.s_codes[rows, :ns] = torch.gather(self.codes[rows, :n], 1, pick)
                self.s_list_ids[rows, :ns] = torch.gather(self.list_ids[rows, :n], 1, pick)
                self.s_norms[rows, :ns] = torch.gather(self.norms[rows, :n], 1, pick)
            for i in range(b, e):
                self.n_sorted_host[i] = n
            b = e
        self.n_sorted.copy_(torch.tensor(self.n_sorted_host, dtype=torch.int32))
        self.s_n.copy_(torch.tensor([self.sample_size(n) if n > 0 else 0 for n in self.n_host], dtype=torch.int32))

    def _sample_positions(self, n: int, ns: int, seed: int, seqs: torch.Tensor) -> torch.Tensor:
        """Ascending positions in ``[0, n)``, one per stratum ``[i n / ns, (i + 1) n / ns)``; the
        heads of a sequence share them (``seqs``: the sequence number of every row, ``[rows, 1]``)."""
        i = torch.arange(ns, device=self.device, dtype=torch.int64).unsqueeze(0)
        lo, hi = i * n // ns, (i + 1) * n // ns
        x = (i + 1) * 0x9E3779B1 + (seqs + 1) * 0x85EBCA77 + (seed + 1) * 0xC2B2AE3D
        x = (x ^ (x >> 15)) * 0x2C1B3C6D & 0xFFFFFFFF
        x = (x ^ (x >> 12)) * 0x297A2D39 & 0xFFFFFFFF
        x = x ^ (x >> 15)
        return lo + x % (hi - lo)

    def tail_max(self) -> int:
        return max((n - s for n, s in zip(self.n_host, self.n_sorted_host)), default=0)

    def struct(self) -> Index:
        if self._struct is None:
            s = Index()
            s.codes, s.list_ids, s.norms = self.codes.data_ptr(), self.list_ids.data_ptr(), self.norms.data_ptr()
            s.pos = self.pos.data_ptr()
            s.coarse, s.codebooks = self.coarse.data_ptr(), self.codebooks.data_ptr()
            s.vbar, s.vsum, s.vcount = self.vbar.data_ptr(), self.vsum.data_ptr(), self.vcount.data_ptr()
            s.n_idx, s.n_sorted = self.n_idx.data_ptr(), self.n_sorted.data_ptr()
            s.s_codes, s.s_list_ids, s.s_norms = (self.s_codes.data_ptr(), self.s_list_ids.data_ptr(),
                                                  self.s_norms.data_ptr())
            s.s_n, s.s_cap, s.n_cap = self.s_n.data_ptr(), self.s_cap, self.n_cap
            s.num_lists, s.batch, s.kv_heads = self.num_lists, self.batch, self.kv_heads
            self._struct = s
        return self._struct

    def ref(self):
        return ctypes.byref(self.struct())

    def list_ids_long(self) -> torch.Tensor:
        """List ids by stored position as int64 (the int16 tensor holds uint16 bit patterns)."""
        return self.list_ids.to(torch.int64) & 0xFFFF

    def by_key(self, bh: int, n: int):
        """(codes, list_ids, norms) of stream ``bh`` indexed by retrieval-local key index."""
        where = self.pos[bh, :n].to(torch.int64)
        out = []
        for t in (self.codes, self.list_ids, self.norms):
            u = torch.empty_like(t[bh, :n])
            u[where] = t[bh, :n]
            out.append(u)
        return tuple(out)

    def key_lists(self) -> torch.Tensor:
        """List id of every key by retrieval-local index, ``[BH, n_cap]`` int16 (u16 bits)."""
        out = torch.zeros_like(self.list_ids)
        out.scatter_(1, self.pos.to(torch.int64), self.list_ids)
        return out

    def packed_bytes(self, bh: int, n: int) -> torch.Tensor:
        """The reference's ``[N, 4]`` uint8 packing (by key index) is the little-endian view of
        the code words."""
        return self.by_key(bh, n)[0].contiguous().view(torch.uint8).reshape(n, 4)


def _i32(values, device) -> torch.Tensor:
    return torch.tensor([int(v) for v in values], dtype=torch.int32, device=device)


# --------------------------------------------------------------------------- index maintenance
BULK_ENCODE_MIN_ROWS = 128    # from here on the matrix-core candidate pass pays for its two extra launches
BULK_ENCODE_MAX_LISTS = 4096


def encode(kv: KvSource, index: DeviceIndex, sink: int, slot0, count, *, eps: float = EPS,
           bulk: bool | None = None) -> None:
    """Encode ``count[b]`` key rows per sequence starting at index slot ``slot0[b]``.

    Many rows at once go through ``pqhsa_encode_bulk`` (same results bit for bit; ``bulk`` forces
    or forbids that path), whose scratch memory is a temporary of this call."""
    lib = _lib.load()
    s0, c = _i32(slot0, index.device), _i32(count, index.device)
    cmax = int(max(count))
    if bulk is None:
        bulk = cmax >= BULK_ENCODE_MIN_ROWS
    if bulk and cmax > 0 and index.num_lists <= BULK_ENCODE_MAX_LISTS:
        need = lib.pqhsa_encode_bulk_workspace_bytes(index.batch, index.kv_heads, index.num_lists, cmax)
        ws = torch.empty(need, dtype=torch.uint8, device=index.device)
        rc = lib.pqhsa_encode_bulk(kv.ref(), index.ref(), int(sink), s0.data_ptr(), c.data_ptr(), cmax, eps,
                                   ws.data_ptr(), need, _stream())
        _lib.check(rc, "pqhsa_encode_bulk")
        return
    rc = lib.pqhsa_encode(kv.ref(), index.ref(), int(sink), s0.data_ptr(), c.data_ptr(), cmax, eps, _stream())
    _lib.check(rc, "pqhsa_encode")


def nearest_rows(vectors: torch.Tensor, centroids: torch.Tensor, *, eps: float = EPS) -> torch.Tensor:
    """Nearest centroid to the direction of every row: ``vectors [P, R, 128]``, ``centroids
    [P, K, 128]`` contiguous fp32 -> int64 ``[P, R]`` (``pqhsa_nearest_rows``; K <= 4096)."""
    _need_cuda(vectors, centroids)
    p, r, d = vectors.shape
    k = centroids.shape[1]
    if (d != HEAD_DIM or tuple(centroids.shape) != (p, k, HEAD_DIM) or vectors.dtype != torch.float32
            or centroids.dtype != torch.float32 or not vectors.is_contiguous() or not centroids.is_contiguous()):
        raise ValueError(f"nearest_rows: vectors [P, R, {HEAD_DIM}] and centroids [P, K, {HEAD_DIM}] contiguous fp32")
    lib = _lib.load()
    out = torch.empty(p, r, dtype=torch.int64, device=vectors.device)
    need = lib.pqhsa_nearest_rows_workspace_bytes(p, k, r)
    ws = torch.empty(need, dtype=torch.uint8, device=vectors.device)
    rc = lib.pqhsa_nearest_rows(vectors.data_ptr(), centroids.data_ptr(), p, r, k, eps, out.data_ptr(), r,
                                ws.data_ptr(), need, _stream())
    _lib.check(rc, "pqhsa_nearest_rows")
    return out


def nearest_codewords(rows: torch.Tensor, words: torch.Tensor) -> torch.Tensor:
    """``rows [P, R, 16]`` against ``words [P, 16, 16]`` (contiguous fp32): the nearest codeword of
    every row, int64 ``[P, R]`` (``pqhsa_nearest_codewords``)."""
    _need_cuda(rows, words)
    p, r, d = rows.shape
    if (d != SUBDIM or tuple(words.shape) != (p, CODES, SUBDIM) or rows.dtype != torch.float32
            or words.dtype != torch.float32 or not rows.is_contiguous() or not words.is_contiguous()):
        raise ValueError(f"nearest_codewords: rows [P, R, {SUBDIM}] and words [P, {CODES}, {SUBDIM}] contiguous fp32")
    out = torch.empty(p, r, dtype=torch.int64, device=rows.device)
    rc = _lib.load().pqhsa_nearest_codewords(rows.data_ptr(), words.data_ptr(), p, r, out.data_ptr(), r, _stream())
    _lib.check(rc, "pqhsa_nearest_codewords")
    return out


def nearest_from_products(dots: torch.Tensor, sq: torch.Tensor, out: torch.Tensor) -> None:
    """``out[p, j]`` = first argmin over k of ``sq[p, k] - 2 * dots[p, j, k]``; ``dots [P, R, K]``
    and ``sq [P, K]`` contiguous fp32, ``out`` int64 ``[P, R]`` with unit stride along R (a column
    slice of a wider tensor is fine)."""
    _need_cuda(dots, sq, out)
    p, r, k = dots.shape
    if (dots.dtype != torch.float32 or sq.dtype != torch.float32 or out.dtype != torch.int64 or not dots.is_contiguous()
            or not sq.is_contiguous() or tuple(sq.shape) != (p, k) or tuple(out.shape) != (p, r) or (r > 1 and out.stride(1) != 1)):
        raise ValueError("nearest_from_products: dots [P, R, K] / sq [P, K] contiguous fp32, out [P, R] int64")
    rc = _lib.load().pqhsa_nearest_from_products(dots.data_ptr(), sq.data_ptr(), p, r, k, out.data_ptr(),
                                                 out.stride(0) if p > 1 else r, _stream())
    _lib.check(rc, "pqhsa_nearest_from_products")


def value_summaries(kv: KvSource, index: DeviceIndex, sink: int) -> None:
    lib = _lib.load()
    rc = lib.pqhsa_value_summaries(kv.ref(), index.ref(), int(sink), int(index.n_max), _stream())
    _lib.check(rc, "pqhsa_value_summaries")


def encode_append(kv: KvSource, index: DeviceIndex, sink: int, slot0, count, *, eps: float = EPS,
                  slot0_dev: torch.Tensor | None = None, count_dev: torch.Tensor | None = None,
                  count_max: int | None = None) -> None:
    lib = _lib.load()
    s0 = slot0_dev if slot0_dev is not None else _i32(slot0, index.device)
    c = count_dev if count_dev is not None else _i32(count, index.device)
    cmax = int(count_max if count_max is not None else max(count))
    rc = lib.pqhsa_encode_append(kv.ref(), index.ref(), int(sink), s0.data_ptr(), c.data_ptr(), cmax, eps, _stream())
    _lib.check(rc, "pqhsa_encode_append")


# --------------------------------------------------------------------------- scoring
def lut_build(q: torch.Tensor, index: DeviceIndex, groups: int, *, eps: float = EPS):
    """q ``[B, H*G, 128]`` -> qnorm ``[BH, Gp]``, lut ``[BH, 8, 16, Gp]``, list_scores ``[BH, L, Gp]``."""
    _need_cuda(q)
    lib = _lib.load()
    bh, gp = index.batch * index.kv_heads, padded_groups(groups)
    if tuple(q.shape) != (index.batch, index.kv_heads * groups, HEAD_DIM) or not q.is_contiguous():
        raise ValueError(f"q must be contiguous [B, H*G, {HEAD_DIM}], got {tuple(q.shape)}")
    qnorm = torch.empty(bh, gp, dtype=torch.float32, device=q.device)
    lut = torch.empty(bh, SUBSPACES, CODES, gp, dtype=torch.float32, device=q.device)
    ls = torch.empty(bh, index.num_lists, gp, dtype=torch.float32, device=q.device)
    rc = lib.pqhsa_lut_build(q.data_ptr(), dtype_code(q.dtype), index.ref(), groups, eps, qnorm.data_ptr(),
                             lut.data_ptr(), ls.data_ptr(), _stream())
    _lib.check(rc, "pqhsa_lut_build")
    return qnorm, lut, ls


def lut_scan(index: DeviceIndex, groups: int, qnorm, lut, list_scores, scale: float) -> torch.Tensor:
    """Approximate logits ``[BH, G, n_cap]`` (columns >= n_idx are not written)."""
    lib = _lib.load()
    bh = index.batch * index.kv_heads
    logits = torch.zeros(bh, groups, index.n_cap, dtype=torch.float32, device=index.device)
    rc = lib.pqhsa_lut_scan(index.ref(), groups, int(index.n_max), qnorm.data_ptr(), lut.data_ptr(),
                            list_scores.data_ptr(), float(scale), logits.data_ptr(), index.n_cap, _stream())
    _lib.check(rc, "pqhsa_lut_scan")
    return logits


def lut_scan_mass(index: DeviceIndex, groups: int, qnorm, lut, list_scores, scale: float, ref: torch.Tensor) -> torch.Tensor:
    """Per-list background mass of every query row, ``[BH, L, padded G]``: the sum over each list's
    stored keys of ``exp(logit - ref[bh, g])`` (``ref`` float32 ``[BH, padded G]``), in one pass over
    the index without writing logits (``pqhsa_lut_scan_mass``)."""
    lib = _lib.load()
    _need_cuda(ref)
    bh = index.batch * index.kv_heads
    gp = int(lib.pqhsa_padded_groups(groups))
    if ref.dtype != torch.float32 or tuple(ref.shape) != (bh, gp) or not ref.is_contiguous():
        raise ValueError(f"ref must be a contiguous float32 [{bh}, {gp}] tensor")
    mass = torch.empty(bh, index.num_lists, gp, dtype=torch.float32, device=index.device)
    rc = lib.pqhsa_lut_scan_mass(index.ref(), groups, int(index.n_max), qnorm.data_ptr(), lut.data_ptr(),
                                 list_scores.data_ptr(), float(scale), ref.data_ptr(), mass.data_ptr(), _stream())
    _lib.check(rc, "pqhsa_lut_scan_mass")
    return mass


def lut_scan_stats(index: DeviceIndex, groups: int, qnorm, lut, list_scores, scale: float, block_keys: int = 4096):
    """Block statistics of the scan without writing logits (``pqhsa_lut_scan_stats``): ``(block_max,
    block_expsum)``, both float32 ``[BH, G, blocks]`` over blocks of ``block_keys`` consecutive stored
    keys; an empty block holds ``-inf`` and 0."""
    lib = _lib.load()
    if block_keys < 1:
        raise ValueError("block_keys must be positive")
    bh = index.batch * index.kv_heads
    n_max = int(index.n_max)
    blocks = max(1, -(-n_max // block_keys))
    bmax = torch.empty(bh, groups, blocks, dtype=torch.float32, device=index.device)
    bexp = torch.empty_like(bmax)
    rc = lib.pqhsa_lut_scan_stats(index.ref(), groups, n_max, qnorm.data_ptr(), lut.data_ptr(), list_scores.data_ptr(),
                                  float(scale), int(block_keys), blocks, bmax.data_ptr(), bexp.data_ptr(), _stream())
    _lib.check(rc, "pqhsa_lut_scan_stats")
    return bmax, bexp


def block_reduce(block_max: torch.Tensor, block_expsum: torch.Tensor):
    """Fold block statistics ``[..., blocks]`` into ``(row_max, exp_sum)`` of shape ``[...]``
    (``pqhsa_block_reduce``): ``row_max + log(exp_sum)`` is the row's log-sum-exp."""
    lib = _lib.load()
    _need_cuda(block_max)
    _need_cuda(block_expsum)
    if block_max.shape != block_expsum.shape or block_max.ndim < 1 or block_max.shape[-1] < 1:
        raise ValueError("block_max and block_expsum must have the same shape [..., blocks >= 1]")
    if block_max.dtype != torch.float32 or block_expsum.dtype != torch.float32:
        raise ValueError("block statistics must be float32")
    bm, be = block_max.contiguous(), block_expsum.contiguous()
    blocks = bm.shape[-1]
    rows = bm.numel() // blocks
    row_max = torch.empty(bm.shape[:-1], dtype=torch.float32, device=bm.device)
    exp_sum = torch.empty_like(row_max)
    rc = lib.pqhsa_block_reduce(bm.data_ptr(), be.data_ptr(), rows, blocks, row_max.data_ptr(), exp_sum.data_ptr(), _stream())
    _lib.check(rc, "pqhsa_block_reduce")
    return row_max, exp_sum


def topk_radix(logits: torch.Tensor, n, k):
    """Exact top-k of each row of ``logits [rows, stride]``; ``n``/``k`` per row.  Returns
    (indices int32 [rows, k_cap], values f32 [rows, k_cap]), the selected keys in no particular order."""
    _need_cuda(logits)
    lib = _lib.load()
    if logits.ndim != 2 or logits.dtype != torch.float32 or logits.stride(1) != 1:
        raise ValueError("logits must be a float32 [rows, stride] matrix")
    rows = logits.shape[0]
    n_t, k_t = _i32(n, logits.device), _i32(k, logits.device)
    n_max, k_cap = int(max(n, default=0)), max(int(max(k, default=0)), 1)
    ws_bytes = lib.pqhsa_topk_workspace_bytes(rows, n_max)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=logits.device)
    idx = torch.full((rows, k_cap), -1, dtype=torch.int32, device=logits.device)
    val = torch.zeros(rows, k_cap, dtype=torch.float32, device=logits.device)
    rc = lib.pqhsa_topk_radix(logits.data_ptr(), logits.stride(0), rows, n_t.data_ptr(), k_t.data_ptr(), n_max,
                              idx.data_ptr(), val.data_ptr(), k_cap, ws.data_ptr(), ws_bytes, _stream())
    _lib.check(rc, "pqhsa_topk_radix")
    return idx, val


# --------------------------------------------------------------------------- decode step
class DecodeWorkspace:
    """Scratch memory of ``pqhsa_decode_step`` for a fixed (B, H, G, n_cap, L, k_cap)."""

    def __init__(self, index: DeviceIndex, groups: int, k_cap: int) -> None:
        lib = _lib.load()
        self.k_cap = max(int(k_cap), 1)
        self.groups = groups
        self._shape = (index.batch, index.kv_heads, groups, index.n_cap, index.num_lists, self.k_cap)
        self.bytes = lib.pqhsa_decode_workspace_bytes(*self._shape)
        self.buf = torch.zeros(self.bytes, dtype=torch.uint8, device=index.device)
        rows = index.batch * index.kv_heads * groups
        self.topk_idx = torch.full((rows, self.k_cap), -1, dtype=torch.int32, device=index.device)
        self.topk_val = torch.zeros(rows, self.k_cap, dtype=torch.float32, device=index.device)
        self.topk_cnt = torch.zeros(rows, dtype=torch.int32, device=index.device)

    def _head_offset(self, getter) -> int:
        return getter(self.buf.data_ptr()) - self.buf.data_ptr()

    def rescans(self) -> int:
        """Rows re-scanned in full because the sampled threshold kept fewer than k candidates
        (synchronises: reads a device counter)."""
        off = self._head_offset(_lib.load().pqhsa_decode_rescan_counter)
        return int(self.buf[off : off + 4].view(torch.int32).item())

    def fused_aborts(self) -> int:
        """Waits between workgroups of the fused scan + selection + attention launch that ran out
        (each abandons its step); 0 in normal operation (synchronises: reads a device counter)."""
        off = self._head_offset(_lib.load().pqhsa_decode_fused_aborts)
        return int(self.buf[off : off + 4].view(torch.int32).item())

    def candidate_counts(self) -> torch.Tensor:
        """Candidates the last step's scan kept per query row, int32 [B*H, padded groups]
        (a view of device memory inside the workspace; rows of a padded group hold 0)."""
        off = self._head_offset(_lib.load().pqhsa_decode_candidate_counts)
        b, h, g = self._shape[:3]
        gp = _lib.load().pqhsa_padded_groups(g)
        return self.buf[off : off + 4 * b * h * gp].view(torch.int32).view(b * h, gp)


def decode_step(q: torch.Tensor, out: torch.Tensor, kv: KvSource, index: DeviceIndex, groups: int,
                seq_lens: torch.Tensor, *, sink: int, full_max: int, fraction: float | None, topk: int,
                scale: float, workspace: DecodeWorkspace, eps: float = EPS, n_max: int | None = None,
                append_count: torch.Tensor | None = None, general_path: bool = False,
                n_mean: int | None = None, one_launch: bool = False, share_rows: bool = False,
                separate_tables: bool = False) -> torch.Tensor:
    """One PQ-HSA decode-attention step for the whole batch; the result is written to ``out``.
    ``n_mean`` (default: the index's host-side mean key count) is the hint that sizes the scan's tiles
    for ragged batches; results do not depend on it.
    Short contexts are served by a single kernel (same results); ``general_path`` keeps such a step
    on the general path (``PQHSA_SELECT_GENERAL_PATH``); ``one_launch`` asks for the scan, selection
    and attention of the general path as a single launch (``PQHSA_SELECT_ONE_LAUNCH``: batches of
    about one length, GQA groups of 3 to 8; same results, measured slower than the three launches).
    ``share_rows`` asks for one fetch per KV head of a K/V row that several query rows of a GQA group
    selected (``PQHSA_SELECT_SHARE_ROWS``: groups of 2 to 8; same results, measured slower).
    ``separate_tables`` keeps the table building and the threshold estimate of a step as two launches
    where they would share one (``PQHSA_SELECT_SEPARATE_TABLES``; same results).
    With ``append_count`` (device int32 [B]) the step first appends one key to every sequence whose
    entry is positive (``pqhsa_append_decode_step``): ``n_max`` must count the appended key and the
    caller calls ``index.note_appended`` afterwards."""
    _need_cuda(q, out, seq_lens)
    lib = _lib.load()
    if tuple(q.shape) != (index.batch, index.kv_heads * groups, HEAD_DIM) or not q.is_contiguous():
        raise ValueError(f"q must be contiguous [B, H*G, {HEAD_DIM}], got {tuple(q.shape)}")
    if out.shape != q.shape or out.dtype != q.dtype or not out.is_contiguous():
        raise ValueError("out must match q in shape and dtype")
    if seq_lens.dtype != torch.int32 or seq_lens.numel() != index.batch:
        raise ValueError("seq_lens must be int32 [B]")
    sel = Select()
    sel.fraction = float(fraction) if fraction else 0.0
    sel.topk = int(topk)
    sel.k_cap = workspace.k_cap
    sel.flags = ((_lib.SELECT_GENERAL_PATH if general_path else 0) | (_lib.SELECT_ONE_LAUNCH if one_launch else 0)
                 | (_lib.SELECT_SHARE_ROWS if share_rows else 0)
                 | (_lib.SELECT_SEPARATE_TABLES if separate_tables else 0))
    sel.n_mean = index.n_mean if n_mean is None else max(0, min(int(n_mean), 2**31 - 1))
    n_max = index.n_max if n_max is None else int(n_max)
    args = (q.data_ptr(), dtype_code(q.dtype), out.data_ptr(), kv.ref(), index.ref(), groups, seq_lens.data_ptr(),
            int(sink), n_max, int(full_max), ctypes.byref(sel), float(scale), eps, workspace.topk_idx.data_ptr(),
            workspace.topk_val.data_ptr(), workspace.topk_cnt.data_ptr(), workspace.buf.data_ptr(), workspace.bytes)
    if append_count is None:
        rc = lib.pqhsa_decode_step(*args, _stream())
    else:
        if append_count.dtype != torch.int32 or append_count.numel() != index.batch or not append_count.is_cuda:
            raise ValueError("append_count must be a device int32 [B] tensor")
        rc = lib.pqhsa_append_decode_step(*args, append_count.data_ptr(), _stream())
    _lib.check(rc, "pqhsa_decode_step")
    return out


def decode_step_launches(index: DeviceIndex, groups: int, workspace: DecodeWorkspace, *, n_max: int | None = None,
                         appending: bool = False, general_path: bool = False, one_launch: bool = False,
                         separate_tables: bool = False) -> int:
    """Kernel launches ``decode_step`` makes for a step of this shape: 1 when the short-context
    kernel serves it, 3 when scan, selection and attention share a launch, 4 when the tables and the
    threshold estimate do, else 5 (``pqhsa_decode_step_launches``).  No GPU work."""
    sel = Select()
    sel.k_cap = workspace.k_cap
    sel.n_mean = index.n_mean
    sel.flags = ((_lib.SELECT_GENERAL_PATH if general_path else 0) | (_lib.SELECT_ONE_LAUNCH if one_launch else 0)
                 | (_lib.SELECT_SEPARATE_TABLES if separate_tables else 0))
    n_max = index.n_max if n_max is None else int(n_max)
    return int(_lib.load().pqhsa_decode_step_launches(index.ref(), groups, n_max, ctypes.byref(sel), int(appending)))


class DecodeCall:
    """A decode step with every argument resolved once: ``run()`` is one C call.

    For steady-state loops whose tensors do not move (the serving loop, the bench): the
    ctypes arguments are built at construction, so the per-step host cost is the foreign
    call itself.  ``n_max``/``full_max`` may be updated between steps.
    """

    def __init__(self, q, out, kv: KvSource, index: DeviceIndex, groups: int, seq_lens, *, sink: int,
                 full_max: int, fraction: float | None, topk: int, scale: float, workspace: DecodeWorkspace,
                 eps: float = EPS, n_max: int | None = None, append_count: torch.Tensor | None = None,
                 general_path: bool = False, one_launch: bool = False, share_rows: bool = False,
                 separate_tables: bool = False, flags: int = 0) -> None:
        _need_cuda(q, out, seq_lens)
        if append_count is not None and (append_count.dtype != torch.int32 or append_count.numel() != index.batch
                                         or not append_count.is_cuda):
            raise ValueError("append_count must be a device int32 [B] tensor")
        if tuple(q.shape) != (index.batch, index.kv_heads * groups, HEAD_DIM) or not q.is_contiguous():
            raise ValueError(f"q must be contiguous [B, H*G, {HEAD_DIM}], got {tuple(q.shape)}")
        if out.shape != q.shape or out.dtype != q.dtype or not out.is_contiguous():
            raise ValueError("out must match q in shape and dtype")
        lib = _lib.load()
        self._fn = lib.pqhsa_decode_step if append_count is None else lib.pqhsa_append_decode_step
        self._append = () if append_count is None else (append_count.data_ptr(),)
        self._index = index
        self._sel = Select()
        self._sel.fraction = float(fraction) if fraction else 0.0
        self._sel.topk = int(topk)
        self._sel.k_cap = workspace.k_cap
        self._sel.flags = (int(flags) | (_lib.SELECT_GENERAL_PATH if general_path else 0)
                           | (_lib.SELECT_ONE_LAUNCH if one_launch else 0) | (_lib.SELECT_SHARE_ROWS if share_rows else 0)
                           | (_lib.SELECT_SEPARATE_TABLES if separate_tables else 0))
        self._sel.n_mean = index.n_mean
        self._keep = (q, out, kv, index, seq_lens, workspace, append_count)
        self.n_max = index.n_max if n_max is None else int(n_max)
        self.full_max = int(full_max)
        self._workspace = workspace
        self._head = (q.data_ptr(), dtype_code(q.dtype), out.data_ptr(), kv.ref(), index.ref(), groups)
        self._seq_lens = seq_lens.data_ptr()
        self._sink = int(sink)
        self._tail = (ctypes.byref(self._sel), float(scale), eps, workspace.topk_idx.data_ptr(),
                      workspace.topk_val.data_ptr(), workspace.topk_cnt.data_ptr())
        self.out = out

    def run(self, stream: int | None = None, seq_lens_ptr: int | None = None) -> None:
        """One step.  With ``append_count`` set at construction this is the fused append + decode
        step: ``n_max`` must already count the appended key, and the caller records the append in
        the index's host-side mirror afterwards (``DeviceIndex.note_appended``).  ``seq_lens_ptr``
        overrides the sequence-length array for this step (an int32 [B] device pointer)."""
        ws = self._workspace
        rc = self._fn(*self._head, self._seq_lens if seq_lens_ptr is None else seq_lens_ptr, self._sink, self.n_max,
                      self.full_max, *self._tail, ws.buf.data_ptr(), ws.bytes, *self._append,
                      _stream() if stream is None else stream)
        if rc:
            _lib.check(rc, "pqhsa_decode_step")

    def capture(self, warm: bool = True) -> "torch.cuda.CUDAGraph":
        """Record the step's kernels into a HIP graph (the graphed steady state of the reference's
        sidecar, benchmarks e2e:6052-6235).  The step clears its scratch with kernels, so the
        graph holds no memset nodes.  A replay runs on the tensors' current contents (new queries
        are copied into ``q``, counts and sequence lengths live in device memory); ``n_max``,
        ``full_max`` and the launch shapes are those of the capture, so the index must not outgrow
        them: a step that appends is captured with ``n_max`` (and the workspace's ``k_cap``) at the
        length the sequences will grow to.  ``warm`` runs the step once before the capture, so that
        the kernels are loaded and their attributes set; a caller whose step appends has run one
        itself (the warm-up would append a key) and passes ``warm=False``."""
        if warm:
            self.run()                  # once outside: kernel attributes are set before capture
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            self.run()
        self.graph = graph
        return graph

    def replay(self) -> None:
        self.graph.replay()


def hybrid_attend_paged(q, out, kv: KvSource, index: DeviceIndex, groups: int, seq_lens, *, sink: int, full_max: int,
                        topk_idx, topk_val, topk_cnt, list_mass, row_max, scale: float) -> torch.Tensor:
    """Exact hybrid attention given a selection and per-list masses (``list_mass [BH, G, L]`` over
    all indexed keys of each list, relative to ``row_max [BH, G]``)."""
    _need_cuda(q, out, topk_idx, topk_val, topk_cnt, list_mass, row_max)
    lib = _lib.load()
    ws_bytes = lib.pqhsa_attend_workspace_bytes(index.batch, index.kv_heads, groups, index.num_lists)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
    key_lists = index.key_lists()
    rc = lib.pqhsa_hybrid_attend_paged(q.data_ptr(), dtype_code(q.dtype), out.data_ptr(), kv.ref(), index.ref(),
                                       groups, seq_lens.data_ptr(), int(sink), int(full_max), topk_idx.data_ptr(),
                                       topk_val.data_ptr(), topk_cnt.data_ptr(), topk_idx.shape[-1],
                                       key_lists.data_ptr(), index.n_cap, list_mass.data_ptr(), row_max.data_ptr(),
                                       float(scale), ws.data_ptr(), ws_bytes, _stream())
    _lib.check(rc, "pqhsa_hybrid_attend_paged")
    return out


# --------------------------------------------------------------------------- paged readers
def paged_gather_range(kv: KvSource, seq: int, start: int, end: int):
    """Token range [start, end) of sequence ``seq`` -> K, V ``[H, n, 128]``."""
    lib = _lib.load()
    n = max(int(end) - int(start), 0)
    dev = kv.keep[0].device
    out_k = torch.empty(kv.kv_heads, n, HEAD_DIM, dtype=kv.dtype, device=dev)
    out_v = torch.empty_like(out_k)
    if n:
        rc = lib.pqhsa_paged_gather_range(kv.ref(), kv.kv_heads, int(seq), int(start), n, out_k.data_ptr(),
                                          out_v.data_ptr(), _stream())
        _lib.check(rc, "pqhsa_paged_gather_range")
    return out_k, out_v


def paged_gather_at(kv: KvSource, seq: int, positions: torch.Tensor):
    """positions int64 ``[H, ...]`` -> K, V shaped like ``positions`` + ``[128]``."""
    lib = _lib.load()
    _need_cuda(positions)
    if positions.shape[0] != kv.kv_heads:
        raise ValueError("positions must have the KV head as leading dimension")
    flat = positions.reshape(kv.kv_heads, -1).to(torch.int64).contiguous()
    n = flat.shape[1]
    out_k = torch.empty(kv.kv_heads, n, HEAD_DIM, dtype=kv.dtype, device=positions.device)
    out_v = torch.empty_like(out_k)
    if n:
        rc = lib.pqhsa_paged_gather_at(kv.ref(), kv.kv_heads, int(seq), flat.data_ptr(), n, out_k.data_ptr(),
                                       out_v.data_ptr(), _stream())
        _lib.check(rc, "pqhsa_paged_gather_at")
    shape = (*positions.shape, HEAD_DIM)
    return out_k.reshape(shape), out_v.reshape(shape)


PROBE_SLOTS = 4096


def gather_probe(kv: KvSource, positions: torch.Tensor, checks: torch.Tensor | None = None) -> torch.Tensor:
    """Read the K and V rows at token ``positions`` (int32 ``[B*H, count]``, every entry a valid token
    of its sequence) and return the per-workgroup checksums (int32 ``[4096]``; their XOR is the XOR
    of all 32-bit words read).  A measurement aid: timed, it gives the rate at which the GPU
    delivers scattered rows of this cache (``pqhsa_gather_probe``)."""
    _need_cuda(positions)
    if positions.dtype != torch.int32 or positions.ndim != 2 or positions.shape[0] != kv.batch * kv.kv_heads \
            or not positions.is_contiguous():
        raise ValueError("positions must be a contiguous int32 [B*H, count] tensor")
    if checks is None:
        checks = torch.zeros(PROBE_SLOTS, dtype=torch.int32, device=positions.device)
    elif checks.dtype != torch.int32 or checks.numel() != PROBE_SLOTS or not checks.is_cuda:
        raise ValueError(f"checks must be a device int32 [{PROBE_SLOTS}] tensor")
    rc = _lib.load().pqhsa_gather_probe(kv.ref(), kv.batch, kv.kv_heads, positions.data_ptr(), positions.shape[1],
                                        checks.data_ptr(), _stream())
    _lib.check(rc, "pqhsa_gather_probe")
    return checks
