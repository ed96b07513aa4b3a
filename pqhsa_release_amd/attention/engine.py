"""Device-side state of PQ-HSA decode attention for a batch of sequences.

``PQHSAEngine`` owns what the reference spreads over ``SparseKVCache`` + ``IVFPQIndex`` +
``IVFPQSparseAttention`` for every (sequence, KV head) stream
(pq_hsa/attention/kv_cache.py:68-314, 1160-1201; pq_hsa/index/ivfpq.py:275-433, 598-707;
pq_hsa/attention/sparse_attention.py:219-335): the sink / retrieval / local region
bookkeeping, the trained index and its per-step updates, and the forward call.  All
arithmetic runs in the HIP kernels behind ``pqhsa_release_amd.ops``; torch supplies memory
and the few small tensor updates of the (off-hot-path) codebook refresh.
"""

from __future__ import annotations

import math

import torch

from .. import ops
from ..config import IVFPQConfig, SparseAttentionConfig, validate_for_kernels
from ..index.train import train_ivfpq_batched

D = ops.HEAD_DIM


class PQHSAEngine:
    def __init__(self, index_config: IVFPQConfig, attention_config: SparseAttentionConfig, *, batch: int,
                 kv_heads: int, device, growth_margin: int = 4096) -> None:
        validate_for_kernels(index_config, attention_config)
        self.index_config, self.attention_config = index_config, attention_config
        self.B, self.H = int(batch), int(kv_heads)
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise RuntimeError("PQ-HSA decode attention needs a GPU: the MI355X kernels have no CPU path")
        self.growth_margin = int(growth_margin)
        self.resort_tail = 4096     # appended keys tolerated in insertion order before a re-sort
        self.sink, self.local = attention_config.sink_tokens, attention_config.local_window
        self.kv: ops.KvSource | None = None
        self.keys_buf = self.values_buf = None      # dense storage owned by the engine (optional)
        self.index: ops.DeviceIndex | None = None
        self.lens = [0] * self.B                    # tokens in the cache
        self.indexed_len = [0] * self.B             # tokens visible to the index bookkeeping
        self.pending = [0] * self.B                 # appended since the last index update
        self.deferred_pending = False
        self._fused_append = False                  # one token was appended; the next forward() encodes it
        self._append_counts: dict[tuple, torch.Tensor] = {}
        self.seq_lens = torch.zeros(self.B, dtype=torch.int32, device=self.device)
        self._ws: dict[int, ops.DecodeWorkspace] = {}
        self.index_adds = self.index_rebuilds = self.online_codebook_updates = self.deferred_index_updates = 0

    # ------------------------------------------------------------------ regions
    def _sink_end(self, b: int) -> int:
        return min(self.sink, self.lens[b])

    def _retrieval_end(self, b: int) -> int:
        s = self._sink_end(b)
        idx_len = min(self.indexed_len[b], self.lens[b])
        return max(s, idx_len - self.local) if self.local > 0 else max(s, idx_len)

    def n(self, b: int) -> int:
        """Indexed (retrieval-region) keys of sequence b."""
        return self._retrieval_end(b) - self._sink_end(b)

    def full_count(self, b: int) -> int:
        return self._sink_end(b) + self.lens[b] - self._retrieval_end(b)

    # ------------------------------------------------------------------ storage
    def bind_dense(self, keys: torch.Tensor, values: torch.Tensor) -> None:
        """Use caller-provided ``[B, H, cap, 128]`` tensors as the K/V store."""
        self.kv = ops.kv_contiguous(keys, values)
        self.keys_buf, self.values_buf = keys, values

    def bind_paged(self, kv_cache: torch.Tensor, block_table: torch.Tensor) -> None:
        """Read K/V rows in place from a paged cache; the engine keeps no copy of its own."""
        self.kv = ops.kv_paged(kv_cache, block_table)
        self.keys_buf = self.values_buf = None

    def adopt(self, keys: torch.Tensor, values: torch.Tensor) -> None:
        """Copy ``[B, H, S, 128]`` K/V into an engine-owned buffer with spare capacity."""
        b, h, s, _ = keys.shape
        cap = s + self.growth_margin
        kb = torch.empty(b, h, cap, D, dtype=keys.dtype, device=self.device)
        vb = torch.empty_like(kb)
        kb[:, :, :s].copy_(keys)
        vb[:, :, :s].copy_(values)
        self.bind_dense(kb, vb)

    def _grow_dense(self, need: int) -> None:
        cap = self.keys_buf.shape[2]
        if need <= cap:
            return
        new_cap = need + self.growth_margin
        kb = torch.empty(self.B, self.H, new_cap, D, dtype=self.keys_buf.dtype, device=self.device)
        vb = torch.empty_like(kb)
        kb[:, :, :cap].copy_(self.keys_buf)
        vb[:, :, :cap].copy_(self.values_buf)
        self.bind_dense(kb, vb)

    def write_rows(self, keys: torch.Tensor, values: torch.Tensor) -> None:
        """Store one new ``[B, H, 128]`` K/V row per sequence at its current length (dense store)."""
        if self.keys_buf is None:
            return  # paged: the owner of the cache has already written the row
        self._grow_dense(max(self.lens) + 1)
        if len(set(self.lens)) == 1:
            self.keys_buf[:, :, self.lens[0]].copy_(keys)
            self.values_buf[:, :, self.lens[0]].copy_(values)
        else:
            for b, ln in enumerate(self.lens):
                self.keys_buf[b, :, ln].copy_(keys[b])
                self.values_buf[b, :, ln].copy_(values[b])

    # ------------------------------------------------------------------ index
    def _lists_of(self, count: int) -> int:
        """Coarse lists a stream of ``count`` keys trains: the configured number, or one per key
        when there are fewer keys than that (IVFPQIndex.build, pq_hsa/index/ivfpq.py:300)."""
        return max(1, min(self.index_config.num_lists, int(count)))

    def _alloc_index(self, n_need: int, num_lists: int) -> None:
        old = self.index
        self.index = ops.DeviceIndex(self.B, self.H, num_lists, n_need + self.growth_margin, self.device)
        self._ws.clear()
        if old is not None and old.num_lists == num_lists:
            keep = min(old.n_cap, self.index.n_cap)
            for name in ("codes", "list_ids", "norms", "pos"):
                getattr(self.index, name)[:, :keep].copy_(getattr(old, name)[:, :keep])
            skeep = min(old.s_cap, self.index.s_cap)
            for name in ("s_codes", "s_list_ids", "s_norms"):
                getattr(self.index, name)[:, :skeep].copy_(getattr(old, name)[:, :skeep])
            for name in ("coarse", "codebooks", "vbar", "vsum", "vcount", "s_n"):
                getattr(self.index, name).copy_(getattr(old, name))
            self.index.n_sorted_host = list(old.n_sorted_host)

    def _retrieval_block(self, b: int, count: int, start: int = 0) -> torch.Tensor:
        """``count`` retrieval-region keys of every KV head of sequence b from retrieval-local index
        ``start`` on, ``[H, count, 128]``."""
        s = self._sink_end(b) + start
        if self.keys_buf is not None:
            return self.keys_buf[b, :, s : s + count]
        return ops.paged_gather_range(self.kv, b, s, s + count)[0]

    def build(self, lens, *, coarse: torch.Tensor | None = None, codebooks: torch.Tensor | None = None) -> None:
        """(Re)build the index over the retrieval region of every sequence.  Without
        ``coarse``/``codebooks`` (``[BH, L, 128]`` / ``[BH, 8, 16, 16]`` or one set shared by all
        streams) each stream trains its own (IVFPQIndex.build); with them this is
        ``build_with_codebooks``."""
        if self.kv is None:
            raise RuntimeError("bind K/V storage before building the index")
        self.lens = [int(x) for x in lens]
        self.indexed_len = list(self.lens)
        self.pending = [0] * self.B
        self.deferred_pending = False
        self._fused_append = False
        counts = [self.n(b) for b in range(self.B)]
        # the tables are as wide as the longest sequence needs; a shorter sequence trains its own,
        # smaller number of lists and the columns it leaves unused are filled with centroids that no
        # key can be nearest to (DeviceIndex.pad_lists), so every stream keeps the reference's lists
        lists = self._lists_of(max(counts)) if coarse is None else int(coarse.shape[-2])
        self.index = None
        self._alloc_index(max(counts), lists)
        ic = self.index_config
        if coarse is None:
            # sequences of one length train together, all their KV heads at once
            by_count: dict[int, list[int]] = {}
            for b in range(self.B):
                if counts[b] > 0:
                    by_count.setdefault(counts[b], []).append(b)
            for n, seqs in by_count.items():
                step = max(1, ((1 << 31) // (n * ops.HEAD_DIM * 4)) // self.H)  # about 2 GB of fp32 keys per batch
                for i in range(0, len(seqs), step):
                    part = seqs[i : i + step]
                    rows = torch.stack([self._retrieval_block(b, n) for b in part]).reshape(-1, n, ops.HEAD_DIM)
                    c, cb = train_ivfpq_batched(rows, num_lists=self._lists_of(n), coarse_iter=ic.coarse_max_iter,
                                                pq_iter=ic.pq_max_iter, seed=ic.seed, eps=ic.eps)
                    del rows
                    for j, b in enumerate(part):
                        sl = slice(b * self.H, (b + 1) * self.H)
                        self.index.coarse[sl, : c.shape[1]].copy_(c[j * self.H : (j + 1) * self.H])
                        self.index.pad_lists(sl, c.shape[1])
                        self.index.codebooks[sl].copy_(cb[j * self.H : (j + 1) * self.H])
        else:
            self.index.coarse.copy_(coarse.to(self.device, torch.float32).expand_as(self.index.coarse))
            self.index.codebooks.copy_(codebooks.to(self.device, torch.float32).expand_as(self.index.codebooks))
        self.index.set_counts(counts)
        if max(counts) > 0:
            ops.encode(self.kv, self.index, self.sink, [0] * self.B, counts, eps=ic.eps)
            self.index.finalize_layout(seed=ic.seed)
            ops.value_summaries(self.kv, self.index, self.sink)   # after the sort: one atomic per run of a list
        self.seq_lens.copy_(torch.tensor(self.lens, dtype=torch.int32))
        self.index_rebuilds += 1

    def _ensure_capacity(self, n_need: int) -> None:
        if n_need > self.index.n_cap:
            counts = list(self.index.n_host)
            self._alloc_index(n_need, self.index.num_lists)
            self.index.set_counts(counts)

    @classmethod
    def regroup(cls, sources) -> "PQHSAEngine":
        """A new engine whose sequence b is sequence ``seq`` of ``engine`` for ``(engine, seq) =
        sources[b]``: index rows and bookkeeping are copied, nothing is rebuilt.  For serving
        batches whose membership changes (a request leaves, another joins); the caller binds the
        K/V storage of the new batch afterwards."""
        first = sources[0][0]
        for eng, _ in sources:
            eng._settle()
            if eng.index is None:
                raise RuntimeError("regroup: every source engine must have a built index")
        new = cls(first.index_config, first.attention_config, batch=len(sources), kv_heads=first.H,
                  device=first.device, growth_margin=first.growth_margin)
        need = max(eng.index.n_host[seq] for eng, seq in sources)
        new.index = ops.DeviceIndex.regroup([(eng.index, seq) for eng, seq in sources], need + new.growth_margin)
        new.lens = [eng.lens[seq] for eng, seq in sources]
        new.indexed_len = [eng.indexed_len[seq] for eng, seq in sources]
        new.pending = [eng.pending[seq] for eng, seq in sources]
        new.deferred_pending = any(eng.deferred_pending and eng.pending[seq] > 0 for eng, seq in sources)
        new.seq_lens.copy_(torch.tensor(new.lens, dtype=torch.int32))
        return new

    def advance(self, count: int = 1, which=None) -> None:
        """Bookkeeping after ``count`` tokens were appended to every sequence, or to the sequences
        listed in ``which`` (SparseKVCache.append, pq_hsa/attention/kv_cache.py:195-226)."""
        ac = self.attention_config
        some = range(self.B) if which is None else [int(b) for b in which]
        for b in some:
            self.lens[b] += count
            self.pending[b] += count
        if which is None:
            self.seq_lens += count
        else:
            self.seq_lens.copy_(torch.tensor(self.lens, dtype=torch.int32))
        if self._fused_append:
            # a second append before the step that would have carried the first: settle the first now
            self._fused_append = False
            self._refresh_index_now()
            return
        if (count == 1 and ac.index_update_strategy == "incremental" and ac.index_update_interval == 1
                and self.index is not None and self.index.n_max > 0):
            # the usual serving step (one token, then attend): the next forward() appends and attends
            # in the same launches
            self._fused_append = True
            return
        if max(self.pending) >= ac.index_update_interval:
            if ac.index_update_strategy == "deferred":
                if not self.deferred_pending:
                    self.deferred_index_updates += 1
                self.deferred_pending = True
            else:
                self._refresh_index_now()

    def extend(self, new_lens) -> int:
        """The K/V store now holds ``new_lens[b]`` tokens of sequence b (at least as many as before;
        only rows outside the indexed region may have changed).  The added rows are taken into the
        index the way a run of appended tokens is at an index update, whatever the update interval
        (extend_prefix, benchmarks/e2e_pq_param_sweep.py:3600-3733, steps 3 and 4).  Returns the
        number of sequences whose index grew."""
        self._settle()
        new_lens = [int(x) for x in new_lens]
        if len(new_lens) != self.B or any(n1 < n0 for n0, n1 in zip(self.lens, new_lens)):
            raise ValueError("extend: one length per sequence, none shorter than before")
        before = [self.n(b) for b in range(self.B)]
        for b in range(self.B):
            self.pending[b] += new_lens[b] - self.lens[b]
        self.lens = new_lens
        self.seq_lens.copy_(torch.tensor(self.lens, dtype=torch.int32))
        self._refresh_index_now()
        self.deferred_pending = False
        return sum(1 for b in range(self.B) if self.n(b) > before[b])

    def _settle(self) -> None:
        """Bring the index up to date if an append is still waiting for the next forward()."""
        if self._fused_append:
            self._fused_append = False
            self._refresh_index_now()

    def apply_pending_index_update(self) -> bool:
        self._settle()
        if not self.deferred_pending:
            return False
        self._refresh_index_now()
        self.deferred_pending = False
        return True

    def _refresh_index_now(self) -> None:
        """SparseKVCache._refresh_index_now (pq_hsa/attention/kv_cache.py:276-314)."""
        strategy = self.attention_config.index_update_strategy
        if strategy == "rebuild" or self.index is None or self.index.n_max == 0:
            self.build(self.lens)
            return
        old = [self.n(b) for b in range(self.B)]
        self.indexed_len = list(self.lens)
        self.pending = [0] * self.B
        new = [self.n(b) for b in range(self.B)]
        added = [n1 - n0 for n0, n1 in zip(old, new)]
        if max(added) <= 0:
            return
        self._ensure_capacity(max(new))
        if strategy in {"online", "deferred"}:
            self._online_refresh(old, added)
            self.online_codebook_updates += 1
        else:
            ops.encode_append(self.kv, self.index, self.sink, old, added, eps=self.index_config.eps)
            self.index_adds += 1
        self.index.set_counts(new)
        if self.index.tail_max() >= self.resort_tail:
            self.index.finalize_layout(seed=self.index_config.seed)

    def _online_refresh(self, old, added) -> None:
        """EMA move of the coarse centroids and PQ codewords towards the newly indexed keys, then
        re-encode every indexed key (IVFPQIndex.online_refresh, pq_hsa/index/ivfpq.py:647-707;
        ProductQuantizer.update_codebooks_ema, pq_hsa/index/pq.py:117-173).  The assignments come
        from the HIP encode kernel; the small per-list means are torch ops on the device."""
        ic, idx = self.index_config, self.index
        lr = ic.online_codebook_lr
        H, L, M = self.H, idx.num_lists, ops.SUBSPACES
        dev = self.device
        # sequences that gained the same number of keys move their tables in one go (all KV heads
        # and subspaces at once); nothing below waits for the host
        groups: dict[int, list[int]] = {}
        for b in range(self.B):
            if added[b] > 0:
                groups.setdefault(added[b], []).append(b)
        batches = []
        for cnt, seqs in groups.items():
            rows = torch.cat([self._retrieval_block(b, cnt, start=old[b]).float() for b in seqs])      # [S, cnt, 128]
            dirs = rows / torch.linalg.vector_norm(rows, dim=-1, keepdim=True).clamp_min(ic.eps)
            streams = (torch.tensor(seqs, device=dev).unsqueeze(1) * H + torch.arange(H, device=dev)).reshape(-1, 1)
            first = torch.tensor([old[b] for b in seqs], device=dev).repeat_interleave(H).unsqueeze(1)
            where = streams * idx.n_cap + first + torch.arange(cnt, device=dev)                           # [S, cnt] flat slots
            batches.append((dirs, streams, where))

        ops.encode(self.kv, idx, self.sink, old, added, eps=ic.eps)          # lists of the new rows
        for dirs, streams, where in batches:
            lids = idx.list_ids.view(-1)[where].to(torch.int64) & 0xFFFF
            _ema_rows(idx.coarse.view(-1, D), dirs.reshape(-1, D), (lids + streams * L).reshape(-1), lr, ic.eps)
        ops.encode(self.kv, idx, self.sink, old, added, eps=ic.eps)          # re-assign with moved lists
        shifts = 4 * torch.arange(M, device=dev)
        for dirs, streams, where in batches:
            lids = idx.list_ids.view(-1)[where].to(torch.int64) & 0xFFFF
            centre = idx.coarse.view(-1, D)[(lids + streams * L).reshape(-1)].view_as(dirs)
            resid = dirs - centre
            words = idx.codes.view(-1)[where].to(torch.int64) & 0xFFFFFFFF
            code = (words.unsqueeze(-1) >> shifts) & 15                                                   # [S, cnt, 8]
            book = (streams.unsqueeze(-1) * M + torch.arange(M, device=dev)) * 16                         # [S, 1, 8]
            _ema_rows(idx.codebooks.view(-1, ops.SUBDIM), resid.reshape(-1, ops.SUBDIM), (code + book).reshape(-1),
                      lr, ic.eps)
        new = [o + a for o, a in zip(old, added)]
        idx.reset_layout()
        idx.set_counts(new)
        ops.encode(self.kv, idx, self.sink, [0] * self.B, new, eps=ic.eps)
        idx.finalize_layout(seed=ic.seed)
        ops.value_summaries(self.kv, idx, self.sink)

    # ------------------------------------------------------------------ forward
    def forward(self, q: torch.Tensor, groups: int, out: torch.Tensor | None = None) -> torch.Tensor:
        """q ``[B, H*groups, 128]`` -> context of the same shape and dtype."""
        if self.index is None:
            raise RuntimeError("build_cache must be called before forward")
        ac = self.attention_config
        if q.dtype != self.kv.dtype and q.dtype != torch.float32:
            q = q.float()
        q = q.contiguous()
        if out is None:
            out = torch.empty_like(q)
        scale = (1.0 / math.sqrt(D)) if ac.scale is None else float(ac.scale)
        append_count, added = None, None
        if self._fused_append:
            self._fused_append = False
            old = [self.n(b) for b in range(self.B)]
            was = (list(self.indexed_len), list(self.pending))
            self.indexed_len = list(self.lens)
            self.pending = [0] * self.B
            added = [self.n(b) - n0 for b, n0 in enumerate(old)]
            if max(added) > 1 or max(self.n(b) for b in range(self.B)) > self.index.n_cap:
                # not the one-key case after all (or the index must grow first): the separate path,
                # from the bookkeeping as it stood (only some sequences may have advanced)
                self.indexed_len, self.pending = was
                self._refresh_index_now()
                added = None
            elif max(added) == 1:
                key = tuple(added)
                if key not in self._append_counts:
                    self._append_counts[key] = torch.tensor(added, dtype=torch.int32, device=self.device)
                append_count = self._append_counts[key]
            else:
                added = None
        ws = self._ws.get(groups)       # looked up only now: an index that had to grow above has dropped the old ones
        k_cap = ops.resolve_topk(self.index.n_cap, ac.retrieval_top_fraction, ac.retrieval_topk)
        if ws is None or ws.k_cap < k_cap:
            ws = self._ws[groups] = ops.DecodeWorkspace(self.index, groups, k_cap)
        full_max = max(self.full_count(b) for b in range(self.B))
        n_max = self.index.n_max + (1 if append_count is not None else 0)
        ops.decode_step(q, out, self.kv, self.index, groups, self.seq_lens, sink=self.sink, full_max=full_max,
                        fraction=ac.retrieval_top_fraction, topk=ac.retrieval_topk, scale=scale, workspace=ws,
                        eps=self.index_config.eps, n_max=n_max, append_count=append_count)
        if append_count is not None:
            self.index.note_appended(added)
            self.index_adds += 1
            if self.index.tail_max() >= self.resort_tail:
                self.index.finalize_layout(seed=self.index_config.seed)
        return out

    def last_topk(self, groups: int):
        """(indices, logits, counts) of the most recent forward for ``groups`` rows per KV head."""
        ws = self._ws[groups]
        return ws.topk_idx, ws.topk_val, ws.topk_cnt

    # ------------------------------------------------------------------ checkpoint
    def state_dict(self) -> dict[str, object]:
        self._settle()
        idx = self.index
        state: dict[str, object] = {
            "lens": list(self.lens), "indexed_len": list(self.indexed_len), "pending": list(self.pending),
            "deferred_pending": self.deferred_pending, "batch": self.B, "kv_heads": self.H,
        }
        if idx is not None:
            state["index"] = {name: getattr(idx, name).detach().clone() for name in
                              ("codes", "list_ids", "norms", "pos", "coarse", "codebooks", "vbar", "vsum", "vcount",
                               "s_codes", "s_list_ids", "s_norms", "s_n")}
            state["index_counts"] = list(idx.n_host)
            state["index_sorted"] = list(idx.n_sorted_host)
            state["num_lists"] = idx.num_lists
        if self.keys_buf is not None:
            top = max(self.lens)
            state["keys"] = self.keys_buf[:, :, :top].detach().clone()
            state["values"] = self.values_buf[:, :, :top].detach().clone()
        return state

    def load_state_dict(self, state: dict[str, object]) -> None:
        if int(state["batch"]) != self.B or int(state["kv_heads"]) != self.H:
            raise ValueError("state does not match the engine's batch / KV heads")
        self.lens = [int(x) for x in state["lens"]]
        self.indexed_len = [int(x) for x in state["indexed_len"]]
        self.pending = [int(x) for x in state["pending"]]
        self.deferred_pending = bool(state["deferred_pending"])
        if "keys" in state:
            self.adopt(state["keys"].to(self.device), state["values"].to(self.device))
        if "index" in state:
            tensors = state["index"]
            self.index = None
            self._alloc_index(max(int(c) for c in state["index_counts"]), int(state["num_lists"]))
            keep = min(self.index.n_cap, tensors["codes"].shape[1])
            for name in ("codes", "list_ids", "norms", "pos"):
                getattr(self.index, name)[:, :keep].copy_(tensors[name][:, :keep])
            skeep = min(self.index.s_cap, tensors["s_codes"].shape[1])
            for name in ("s_codes", "s_list_ids", "s_norms"):
                getattr(self.index, name)[:, :skeep].copy_(tensors[name][:, :skeep])
            for name in ("coarse", "codebooks", "vbar", "vsum", "vcount", "s_n"):
                getattr(self.index, name).copy_(tensors[name])
            self.index.n_sorted_host = [int(x) for x in state["index_sorted"]]
            self.index.set_counts(state["index_counts"])
        self.seq_lens.copy_(torch.tensor(self.lens, dtype=torch.int32))


def _ema_rows(table: torch.Tensor, vectors: torch.Tensor, assign: torch.Tensor, lr: float, eps: float) -> None:
    """table[j] <- (1 - lr) * table[j] + lr * mean(vectors assigned to j), for non-empty j."""
    sums = torch.zeros_like(table)
    sums.index_add_(0, assign, vectors.to(table.dtype))
    counts = torch.bincount(assign, minlength=table.shape[0]).to(table.dtype).unsqueeze(1)
    means = sums / counts.clamp_min(eps)
    # (rows nothing was assigned to keep their bits; no mask is read back by the host)
    table.copy_(torch.where(counts > 0, (1.0 - lr) * table + lr * means, table))
