"""Helpers shared by the GPU parity tests: seeded problems, oracle indices, device upload."""

from __future__ import annotations

import math

import numpy as np
import torch

from oracle import fixed
from oracle import torch_ref as tr
from pqhsa_release_amd import ops
from pqhsa_release_amd.synth import make_head

DIM = 128
SCALE = 1.0 / math.sqrt(DIM)


def words_of(packed: torch.Tensor) -> np.ndarray:
    return tr.packed_to_words(packed).numpy().astype(np.uint32)


class Problem:
    """Seeded K/V/queries for B sequences x H KV heads, a trained index per stream (CPU, via the
    torch oracle's k-means) and the fixed-order oracle's encoding of every stream."""

    def __init__(self, *, lens, heads=1, groups=1, lists=64, sink=4, local=64, seed=0, dtype=torch.float32,
                 clusters=None):
        self.lens = list(lens)
        self.B, self.H, self.G, self.L = len(self.lens), heads, groups, lists
        self.sink, self.local, self.dtype = sink, local, dtype
        self.keys, self.values, self.queries, self.index = {}, {}, {}, {}
        for b, ln in enumerate(self.lens):
            for h in range(heads):
                k, v, q = make_head(ln, groups=groups, seed=seed + 1000 * b + h, num_clusters=clusters or lists)
                # the oracles see the fp32 up-cast of the rounded tensors
                k, v, q = k.to(dtype).float(), v.to(dtype).float(), q.to(dtype).float()
                self.keys[b, h], self.values[b, h], self.queries[b, h] = k, v, q
                n = self.n(b)
                if n == 0:
                    self.index[b, h] = None
                    continue
                ref = tr.train_index(k[sink : sink + n], num_lists=lists, seed=seed)
                norms, lids, codes = fixed.encode(k[sink : sink + n].numpy(), ref.coarse.numpy(),
                                                  ref.codebooks.numpy())
                _, _, vbar = fixed.value_summaries(v[sink : sink + n].numpy(), lids, lists)
                self.index[b, h] = {"coarse": ref.coarse.numpy(), "codebooks": ref.codebooks.numpy(),
                                    "codes": codes, "list_ids": lids, "norms": norms, "vbar": vbar}

    def n(self, b: int) -> int:
        ln = self.lens[b]
        s = min(self.sink, ln)
        return max(s, ln - self.local) - s

    @property
    def n_max(self) -> int:
        return max(self.n(b) for b in range(self.B))

    def q_tensor(self, device="cuda") -> torch.Tensor:
        q = torch.stack([torch.cat([self.queries[b, h] for h in range(self.H)]) for b in range(self.B)])
        return q.to(self.dtype).to(device).contiguous()

    def dense_kv(self, device="cuda", extra=0):
        cap = max(self.lens) + extra
        k = torch.zeros(self.B, self.H, cap, DIM, dtype=self.dtype)
        v = torch.zeros_like(k)
        for (b, h), t in self.keys.items():
            k[b, h, : t.shape[0]] = t.to(self.dtype)
            v[b, h, : t.shape[0]] = self.values[b, h].to(self.dtype)
        return k.to(device), v.to(device)

    def paged_kv(self, layout="5d", block_size=16, shuffle=True, device="cuda", seed=0):
        blocks_per = [(ln + block_size - 1) // block_size for ln in self.lens]
        total = sum(blocks_per) + 3
        gen = torch.Generator().manual_seed(seed)
        order = torch.randperm(total, generator=gen) if shuffle else torch.arange(total)
        table = torch.zeros(self.B, max(blocks_per), dtype=torch.int32)
        at = 0
        for b, nb in enumerate(blocks_per):
            table[b, :nb] = order[at : at + nb].to(torch.int32)
            at += nb
        if layout == "5d":
            cache = torch.zeros(2, total, block_size, self.H, DIM, dtype=self.dtype)
            kc, vc = cache[0], cache[1]
        else:
            cache = torch.zeros(total, self.H, block_size, 2 * DIM, dtype=self.dtype)
            kc, vc = tr.split_kv_cache(cache)
        for (b, h), t in self.keys.items():
            ln = t.shape[0]
            pos = torch.arange(ln)
            blk = table[b, pos // block_size].long()
            kc[blk, pos % block_size, h] = t.to(self.dtype)
            vc[blk, pos % block_size, h] = self.values[b, h].to(self.dtype)
        return cache.to(device), table.to(device)

    def device_index(self, device="cuda", spare=64, upload_codes=True, finalize=True) -> ops.DeviceIndex:
        idx = ops.DeviceIndex(self.B, self.H, self.L, self.n_max + spare, device)
        for (b, h), ix in self.index.items():
            bh = b * self.H + h
            n = self.n(b)
            if ix is None:
                continue
            idx.coarse[bh] = torch.from_numpy(ix["coarse"]).to(device)
            idx.codebooks[bh] = torch.from_numpy(ix["codebooks"]).to(device)
            if upload_codes:
                idx.codes[bh, :n] = torch.from_numpy(ix["codes"].view(np.int32)).to(device)
                idx.list_ids[bh, :n] = torch.from_numpy(ix["list_ids"].view(np.int16)).to(device)
                idx.norms[bh, :n] = torch.from_numpy(ix["norms"]).to(device)
                idx.vbar[bh] = torch.from_numpy(ix["vbar"]).to(device)
        idx.set_counts([self.n(b) for b in range(self.B)])
        if upload_codes and finalize:
            idx.finalize_layout()      # list-sorted storage + sampled subset, as after a build
        return idx

    def seq_lens(self, device="cuda") -> torch.Tensor:
        return torch.tensor(self.lens, dtype=torch.int32, device=device)

    def oracle_step(self, b, h, fraction):
        return fixed.decode_step(self.queries[b, h].numpy(), self.keys[b, h].numpy(), self.values[b, h].numpy(),
                                 self.index[b, h], sink=self.sink, local=self.local, fraction=fraction, scale=SCALE)


def u16(t: torch.Tensor) -> np.ndarray:
    return t.cpu().numpy().view(np.uint16)


def u32(t: torch.Tensor) -> np.ndarray:
    return t.cpu().numpy().view(np.uint32)
