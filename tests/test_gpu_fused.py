"""The decode step with scan, selection and exact attention in ONE launch (workgroups hand work to
each other through counters in the workspace), against the fixed-order oracle and against the
same step with the three launched apart.  Everything goes through the C ABI."""

import numpy as np
import pytest
import torch

from pqhsa_release_amd import ops
from tests.gpu_util import DIM, SCALE, Problem

pytestmark = pytest.mark.gpu


def _cuda():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    return "cuda"


def _kv(p, layout):
    return ops.kv_contiguous(*p.dense_kv()) if layout == "dense" else ops.kv_paged(*p.paged_kv(layout))


CASES = [
    dict(lens=[3000, 3000], heads=2, groups=4, lists=64, dtype=torch.bfloat16, fraction=0.02, kv="5d"),
    dict(lens=[20000], heads=2, groups=4, lists=64, dtype=torch.float32, fraction=0.02, kv="dense"),
    dict(lens=[5000, 4900, 5100, 5000], heads=3, groups=3, lists=32, dtype=torch.bfloat16, fraction=0.05, kv="4d"),
    dict(lens=[9000], heads=2, groups=7, lists=48, dtype=torch.float16, fraction=0.03, kv="4d"),
    dict(lens=[2500, 2500, 2500, 2500], heads=8, groups=4, lists=16, dtype=torch.bfloat16, fraction=0.02, kv="5d"),
    dict(lens=[40000], heads=1, groups=5, lists=128, dtype=torch.bfloat16, fraction=0.01, kv="5d"),
]


@pytest.mark.parametrize("case", CASES, ids=[str(i) for i in range(len(CASES))])
def test_fused_step_matches_oracle_and_separate_launches(case):
    dev = _cuda()
    p = Problem(lens=case["lens"], heads=case["heads"], groups=case["groups"], lists=case["lists"],
                dtype=case["dtype"], seed=77)
    idx = p.device_index(dev)
    kv = _kv(p, case["kv"])
    k_cap = ops.resolve_topk(p.n_max, case["fraction"], 0)
    ws = ops.DecodeWorkspace(idx, p.G, k_cap)
    assert ops.decode_step_launches(idx, p.G, ws, general_path=True, one_launch=True) == 3
    assert ops.decode_step_launches(idx, p.G, ws, general_path=True, separate_tables=True) == 5
    q = p.q_tensor().float()
    tol = 1e-4 if case["dtype"] == torch.float32 else 2e-3
    results = {}
    for separate in (True, False, False):   # the fused form twice: the workspace's counters start over each step
        out = torch.full_like(q, float("nan"))
        ws.topk_idx.fill_(-1)
        ws.topk_cnt.fill_(-1)
        ops.decode_step(q, out, kv, idx, p.G, p.seq_lens(), sink=p.sink, full_max=p.sink + p.local,
                        fraction=case["fraction"], topk=0, scale=SCALE, workspace=ws, general_path=True,
                        one_launch=not separate)
        torch.cuda.synchronize()
        assert ws.fused_aborts() == 0
        tidx = ws.topk_idx.cpu().numpy().reshape(p.B, p.H, p.G, -1)
        cnt = ws.topk_cnt.cpu().numpy().reshape(p.B, p.H, p.G)
        o = out.cpu().numpy().reshape(p.B, p.H, p.G, DIM)
        results[separate] = o
        for (b, h) in p.index:
            want_out, want_idx, _ = p.oracle_step(b, h, case["fraction"])
            k = want_idx.shape[1]
            assert (cnt[b, h] == k).all(), (separate, b, h)
            for g in range(p.G):
                assert np.array_equal(np.sort(tidx[b, h, g, :k]), np.sort(want_idx[g])), (separate, b, h, g)
            assert float(np.abs(o[b, h] - want_out).max()) <= tol, (separate, b, h)
    assert float(np.abs(results[True] - results[False]).max()) <= 1e-5


def test_fused_step_rescans_and_ties():
    """Rows the fused selection cannot settle from its histogram take the general streaming
    selection inside the same launch: a sample that puts the threshold too high (every row keeps
    fewer than k candidates and is re-scored in full), and keys with many equal logits."""
    dev = _cuda()
    p = Problem(lens=[20000], heads=1, groups=3, lists=32, seed=29)
    idx = p.device_index(dev)
    _, _, logits = p.oracle_step(0, 0, 0.02)
    ns = int(idx.s_n[0])
    best = np.argsort(-logits.max(axis=0), kind="stable")[:ns].copy()
    codes, lists, norms = idx.by_key(0, p.n(0))
    pick = torch.from_numpy(best).to(dev)
    idx.s_codes[0, :ns], idx.s_list_ids[0, :ns], idx.s_norms[0, :ns] = codes[pick], lists[pick], norms[pick]
    kv = ops.kv_contiguous(*p.dense_kv())
    ws = ops.DecodeWorkspace(idx, p.G, ops.resolve_topk(p.n_max, 0.02, 0))
    assert ops.decode_step_launches(idx, p.G, ws, general_path=True, one_launch=True) == 3
    q = p.q_tensor()
    out = torch.full_like(q, float("nan"))
    before = ws.rescans()
    ops.decode_step(q, out, kv, idx, p.G, p.seq_lens(), sink=p.sink, full_max=p.sink + p.local, fraction=0.02,
                    topk=0, scale=SCALE, workspace=ws, general_path=True, one_launch=True)
    torch.cuda.synchronize()
    assert ws.fused_aborts() == 0 and ws.rescans() - before == p.G
    want_out, want_idx, _ = p.oracle_step(0, 0, 0.02)
    tidx = ws.topk_idx.cpu().numpy().reshape(p.G, -1)
    for g in range(p.G):
        assert np.array_equal(np.sort(tidx[g, : want_idx.shape[1]]), np.sort(want_idx[g])), g
    assert float(np.abs(out.cpu().numpy().reshape(p.G, DIM) - want_out).max()) <= 1e-4

    # equal logits: every key of the stream gets the same code, list and norm, so all logits of a
    # row are equal and the lowest retrieval-local indices must win
    p2 = Problem(lens=[18000], heads=1, groups=4, lists=16, seed=31)
    idx2 = p2.device_index(dev, finalize=False)
    n = p2.n(0)
    idx2.codes[0, :n] = int(idx2.codes[0, 0])
    idx2.list_ids[0, :n] = int(idx2.list_ids[0, 0])
    idx2.norms[0, :n] = float(idx2.norms[0, 0])
    idx2.finalize_layout()
    kv2 = ops.kv_contiguous(*p2.dense_kv())
    k = ops.resolve_topk(n, 0.02, 0)
    ws2 = ops.DecodeWorkspace(idx2, p2.G, k)
    q2 = p2.q_tensor()
    out2 = torch.full_like(q2, float("nan"))
    assert ops.decode_step_launches(idx2, p2.G, ws2, general_path=True, one_launch=True) == 3
    ops.decode_step(q2, out2, kv2, idx2, p2.G, p2.seq_lens(), sink=p2.sink, full_max=p2.sink + p2.local, fraction=0.02,
                    topk=0, scale=SCALE, workspace=ws2, general_path=True, one_launch=True)
    torch.cuda.synchronize()
    assert ws2.fused_aborts() == 0
    got = ws2.topk_idx.cpu().numpy().reshape(p2.G, -1)
    for g in range(p2.G):
        assert np.array_equal(np.sort(got[g, :k]), np.arange(k)), g
    assert bool(torch.isfinite(out2).all())


def test_fused_step_with_the_append_riding_on_it():
    """The fused launch after an append that rides on the step's first two launches: the new key
    counts reach the index, and the top-k equals a top-k of the scanned logits."""
    dev = _cuda()
    p = Problem(lens=[6000, 6000], heads=2, groups=4, lists=32, dtype=torch.bfloat16, seed=91)
    room = 4
    lens0 = [ln - room for ln in p.lens]
    n0 = [ln - p.local - p.sink for ln in lens0]
    # an index over the first len - room tokens, encoded on the device from the paged cache
    idx = ops.DeviceIndex(p.B, p.H, p.L, max(n0) + room + 64, dev)
    for (b, h), ix in p.index.items():
        idx.coarse[b * p.H + h] = torch.from_numpy(ix["coarse"]).to(dev)
        idx.codebooks[b * p.H + h] = torch.from_numpy(ix["codebooks"]).to(dev)
    kv = ops.kv_paged(*p.paged_kv("5d"))
    idx.set_counts(n0)
    ops.encode(kv, idx, p.sink, [0] * p.B, n0)
    idx.finalize_layout()
    ops.value_summaries(kv, idx, p.sink)
    k_cap = ops.resolve_topk(max(n0) + room, 0.03, 0)
    ws = ops.DecodeWorkspace(idx, p.G, k_cap)
    q = p.q_tensor().float()
    ones = torch.ones(p.B, dtype=torch.int32, device=dev)
    for t in range(1, room + 1):
        out = torch.full_like(q, float("nan"))
        seq = torch.tensor([ln + t for ln in lens0], dtype=torch.int32, device=dev)
        n_now = max(n0) + t
        assert ops.decode_step_launches(idx, p.G, ws, n_max=n_now, appending=True, general_path=True, one_launch=True) == 3
        ops.decode_step(q, out, kv, idx, p.G, seq, sink=p.sink, full_max=p.sink + p.local, fraction=0.03, topk=0,
                        scale=SCALE, workspace=ws, n_max=n_now, append_count=ones, general_path=True, one_launch=True)
        idx.note_appended([1] * p.B)
        torch.cuda.synchronize()
        assert ws.fused_aborts() == 0
        assert idx.n_idx.cpu().tolist() == [n + t for n in n0]
        qnorm, lut, ls = ops.lut_build(q, idx, p.G)
        logits = ops.lut_scan(idx, p.G, qnorm, lut, ls, SCALE)
        for b in range(p.B):
            n = n0[b] + t
            k = ops.resolve_topk(n, 0.03, 0)
            rows = slice(b * p.H, (b + 1) * p.H)
            tidx = ws.topk_idx.view(p.B * p.H, p.G, -1)[rows, :, :k].to(torch.int64)
            tval = ws.topk_val.view(p.B * p.H, p.G, -1)[rows, :, :k]
            lg = logits.view(p.B * p.H, p.G, -1)[rows, :, :n]
            assert torch.equal(torch.gather(lg, 2, tidx), tval), (t, b)
            assert torch.equal(tval.sort(dim=2, descending=True).values, torch.topk(lg, k, dim=2).values), (t, b)
        assert bool(torch.isfinite(out).all())


# ---- K/V rows fetched once per KV head ------------------------------------------------------------
def _steps(p, idx, kv, ws, q, fraction, **kw):
    out = torch.full_like(q, float("nan"))
    ws.topk_idx.fill_(-1)
    ops.decode_step(q, out, kv, idx, p.G, p.seq_lens(), sink=p.sink, full_max=p.sink + p.local, fraction=fraction,
                    topk=0, scale=SCALE, workspace=ws, general_path=True, **kw)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("overlap", ["identical", "disjoint", "half"])
@pytest.mark.parametrize("groups, dtype", [(4, torch.bfloat16), (2, torch.float32), (7, torch.float16)])
def test_rows_of_a_group_that_select_identical_disjoint_and_half_overlapping_keys(overlap, groups, dtype):
    """The attention that fetches a selected K/V row once per KV head, on groups whose query rows
    select the same keys (every row is fetched for all rows by one owner), different keys (every
    row fetches its own) or half of each other's: top-k sets are the oracle's, outputs within the
    bound, and equal to the form in which every query row fetches its own rows."""
    dev = _cuda()
    p = Problem(lens=[9000, 9000], heads=2, groups=groups, lists=32, dtype=dtype, seed=501)
    gen = torch.Generator().manual_seed(9)
    for (b, h), q in p.queries.items():
        keys = p.keys[b, h]
        if overlap == "identical":      # the same query in every row of the group
            q[:] = q[0]
        elif overlap == "disjoint":     # needles far apart: unrelated keys
            picks = torch.randperm(p.lens[b] - 200, generator=gen)[: p.G] + 100
            q[:] = (keys[picks] + 0.05 * torch.randn(p.G, DIM, generator=gen)).to(dtype).float()
        else:                           # pairs of rows around one needle each: about half of a pair's keys in common
            picks = torch.randperm(p.lens[b] - 200, generator=gen)[: (p.G + 1) // 2] + 100
            q[:] = (keys[picks].repeat_interleave(2, 0)[: p.G] + 0.25 * torch.randn(p.G, DIM, generator=gen)).to(dtype).float()
    idx = p.device_index(dev)
    kv = _kv(p, "5d" if dtype != torch.float32 else "dense")
    ws = ops.DecodeWorkspace(idx, p.G, ops.resolve_topk(p.n_max, 0.04, 0))
    q = p.q_tensor().float()
    shared = _steps(p, idx, kv, ws, q, 0.04, share_rows=True)
    tidx = ws.topk_idx.cpu().numpy().reshape(p.B, p.H, p.G, -1)
    own = _steps(p, idx, kv, ws, q, 0.04)
    tol = 1e-4 if dtype == torch.float32 else 2e-3
    o = shared.cpu().numpy().reshape(p.B, p.H, p.G, DIM)
    common = []
    for (b, h) in p.index:
        want_out, want_idx, _ = p.oracle_step(b, h, 0.04)
        k = want_idx.shape[1]
        for g in range(p.G):
            assert np.array_equal(np.sort(tidx[b, h, g, :k]), np.sort(want_idx[g])), (b, h, g)
        assert float(np.abs(o[b, h] - want_out).max()) <= tol, (b, h)
        union = len(set(np.concatenate([want_idx[g] for g in range(p.G)]).tolist()))
        common.append(1.0 - union / (p.G * k))
    assert float((shared - own).abs().max()) <= 2e-5
    if overlap == "identical":
        assert min(common) > 0.4 if p.G == 2 else min(common) > 0.7      # every key shared by all rows
    elif overlap == "disjoint":
        assert max(common) < 0.3


def test_shared_fetch_over_many_rows_and_chunks():
    """Many streams, the largest number of chunks per row the launch uses, rows that share most of their
    keys: every output row must be folded exactly once (rows start as NaN), over repeated steps."""
    dev = _cuda()
    p = Problem(lens=[30000] * 3, heads=4, groups=4, lists=32, dtype=torch.bfloat16, seed=77)
    for (b, h), q in p.queries.items():
        q[2:] = q[:2]                    # two pairs of equal rows
    idx = p.device_index(dev)
    kv = _kv(p, "4d")
    ws = ops.DecodeWorkspace(idx, p.G, ops.resolve_topk(p.n_max, 0.1, 0))   # about 3 000 rows per query: several chunks
    q = p.q_tensor()
    ref = _steps(p, idx, kv, ws, q, 0.1).float()
    assert bool(torch.isfinite(ref).all())
    for rep in range(40):
        got = _steps(p, idx, kv, ws, q, 0.1, share_rows=True).float()
        assert bool(torch.isfinite(got).all()), rep
        assert float((got - ref).abs().max()) <= 2e-2, rep      # (bf16 outputs: one step of rounding)
    o = got.cpu().numpy().reshape(p.B, p.H, p.G, DIM)
    for (b, h) in list(p.index)[:3]:
        want_out, _, _ = p.oracle_step(b, h, 0.1)
        assert float(np.abs(o[b, h] - want_out).max()) <= 2e-3 + 2.0 ** -8 * float(np.abs(want_out).max()), (b, h)
