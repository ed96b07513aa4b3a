"""Pin the oracles with what the mathematics fixes, mirroring the reference's own CPU tests
(tests/test_packing.py, test_lut_scan.py, test_pq_scores.py, test_sparse_attention.py)."""

import numpy as np
import pytest
import torch

from oracle import fixed
from oracle import torch_ref as tr


def test_packing_literal_vectors():
    # tests/test_packing.py:7-36 of the reference
    codes = torch.tensor([[0, 1, 2, 3], [15, 14, 13, 12]])
    packed = tr.pack_4bit_codes(codes)
    assert packed.dtype == torch.uint8 and packed.shape == (2, 2)
    assert packed.tolist() == [[0x10, 0x32], [0xEF, 0xCD]]
    assert torch.equal(tr.unpack_4bit_codes(packed, 4), codes)
    odd = torch.tensor([[1, 2, 3], [4, 5, 6]])
    p = tr.pack_4bit_codes(odd)
    assert p.shape == (2, 2) and torch.all((p[:, -1] >> 4) == 0)
    assert torch.equal(tr.unpack_4bit_codes(p, 3), odd)
    with pytest.raises(ValueError, match=r"\[0, 15\]"):
        tr.pack_4bit_codes(torch.tensor([[0, 16]]))


def test_packed_word_has_nibble_m_at_bit_4m():
    codes = torch.randint(0, 16, (50, 8), generator=torch.Generator().manual_seed(1))
    words = tr.packed_to_words(tr.pack_4bit_codes(codes)).numpy()
    for m in range(8):
        assert np.array_equal((words >> (4 * m)) & 15, codes[:, m].numpy())


def _random_index(n, lists, seed, dim=128):
    g = torch.Generator().manual_seed(seed)
    coarse = torch.nn.functional.normalize(torch.randn(lists, dim, generator=g), dim=1)
    books = 0.1 * torch.randn(8, 16, dim // 8, generator=g)
    keys = torch.randn(n, dim, generator=g) * 3.0
    return keys, coarse, books


def test_scan_equals_dense_lut_gather_sum():
    # tests/test_lut_scan.py:20-41, 60-70 of the reference: packed scan == lut.gather(codes).sum
    g = torch.Generator().manual_seed(17)
    codes = torch.randint(0, 16, (231, 8), generator=g)
    lut = torch.randn(3, 8, 16, generator=g)
    words = tr.packed_to_words(tr.pack_4bit_codes(codes)).numpy().astype(np.uint32)
    zeros_l = np.zeros(231, np.uint16)
    got = fixed.scan(words, zeros_l, np.ones(231, np.float32), lut.numpy(), np.zeros((3, 1), np.float32),
                     np.ones(3, np.float32), 1.0)
    expected = lut.gather(2, codes.T.unsqueeze(0).expand(3, -1, -1)).sum(dim=1)
    np.testing.assert_allclose(got, expected.numpy(), rtol=1e-5, atol=1e-6)
    got_t = tr.score_packed(tr.pack_4bit_codes(codes), lut, 8)
    np.testing.assert_allclose(got_t.numpy(), expected.numpy(), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("which", ["fixed", "torch"])
def test_scores_equal_query_dot_reconstruction(which):
    # tests/test_pq_scores.py:153-175, 298-332: approximate score == q . reconstruct(), atol 1e-5
    keys, coarse, books = _random_index(400, 24, 5)
    q = torch.randn(3, 128, generator=torch.Generator().manual_seed(6))
    idx = tr.encode_with_codebooks(keys, coarse, books)
    codes = tr.unpack_4bit_codes(idx.packed, 8)
    recon = torch.cat([books[m, codes[:, m]] for m in range(8)], dim=1) + coarse[idx.list_ids]
    recon = recon * idx.norms[:, None]
    expected = q.double() @ recon.double().T
    if which == "torch":
        got = tr.approximate_scores(idx, q).double().numpy()
    else:
        qn, lut, ls = fixed.lut_build(q.numpy(), coarse.numpy(), books.numpy())
        words = tr.packed_to_words(idx.packed).numpy().astype(np.uint32)
        got = fixed.scan(words, idx.list_ids.numpy().astype(np.uint16), idx.norms.numpy(), lut, ls, qn, 1.0)
    np.testing.assert_allclose(got, expected.numpy(), rtol=1e-5, atol=1e-5 * float(expected.abs().max()))


def test_fixed_encode_is_brute_force_nearest():
    keys, coarse, books = _random_index(120, 16, 9)
    norms, lists, codes = fixed.encode(keys.numpy(), coarse.numpy(), books.numpy())
    k64 = keys.double()
    nrm = k64.norm(dim=1)
    np.testing.assert_allclose(norms, nrm.numpy(), rtol=1e-6)
    dirs = k64 / nrm[:, None]
    d = ((dirs[:, None, :] - coarse.double()[None]) ** 2).sum(-1)
    srt = d.sort(dim=1).values
    clear = (srt[:, 1] - srt[:, 0]) > 1e-6
    assert np.array_equal(lists[clear.numpy()], d.argmin(1).numpy()[clear.numpy()])
    res = dirs - coarse.double()[torch.from_numpy(lists.astype(np.int64))]
    for m in range(8):
        dd = ((res[:, None, m * 16 : (m + 1) * 16] - books.double()[m][None]) ** 2).sum(-1)
        s2 = dd.sort(dim=1).values
        ok = ((s2[:, 1] - s2[:, 0]) > 1e-7).numpy()
        assert np.array_equal(((codes >> (4 * m)) & 15)[ok], dd.argmin(1).numpy()[ok])


def test_topk_is_sort_with_lowest_index_ties():
    rng = np.random.default_rng(3)
    logits = rng.standard_normal(500).astype(np.float32)
    logits[[7, 100, 300, 301]] = logits.max() + 1.0          # 4-way tie at the top
    logits[[50, 60, 70]] = np.sort(logits)[::-1][12]          # ties at the k boundary
    for k in (0, 1, 3, 13, 14, 15, 500):
        idx, val = fixed.topk(logits, k)
        order = np.lexsort((np.arange(500), -logits.astype(np.float64)))[:k]
        assert np.array_equal(idx, order.astype(np.int32))
        assert np.array_equal(val, logits[order])
    # -0.0 and +0.0 are one value: the tie goes to the lowest index
    z = np.array([-1.0, 0.0, -0.0, 0.0, -0.0], np.float32)
    idx, _ = fixed.topk(z, 2)
    assert idx.tolist() == [1, 2]
    # k = ceil(N * fraction) (tests/test_sparse_attention.py:185-216)
    assert fixed.resolve_topk(8124, 0.02) == 163 and fixed.resolve_topk(131004, 0.02) == 2621
    assert fixed.resolve_topk(10, 1.0) == 10 and tr.resolve_topk(262076, 0.02) == 5242


@pytest.mark.parametrize("which", ["fixed", "torch"])
def test_all_selected_reduces_to_dense_softmax(which):
    # tests/test_sparse_attention.py:40-103, tests/test_decode_adapter.py:11-47: with every
    # indexed key attended exactly the hybrid output is textbook softmax attention
    keys, coarse, books = _random_index(200, 8, 21)
    keys = keys * 0.3
    g = torch.Generator().manual_seed(22)
    values = torch.randn(200, 128, generator=g)
    q = torch.randn(2, 128, generator=g)
    sink, local, scale = 3, 10, 1.0 / np.sqrt(128)
    idx = tr.encode_with_codebooks(keys[sink : 200 - local], coarse, books)
    vbar = tr.value_centroids(values[sink : 200 - local], idx.list_ids, 8)
    dense = torch.softmax((q.double() @ keys.double().T) * scale, dim=-1) @ values.double()
    if which == "torch":
        out = tr.hybrid_forward_many(q, keys, values, sink_end=sink, retrieval_end=200 - local, index=idx,
                                     vbar=vbar, fraction=1.0, scale=scale).numpy()
    else:
        index = {"coarse": coarse.numpy(), "codebooks": books.numpy(),
                 "codes": tr.packed_to_words(idx.packed).numpy().astype(np.uint32),
                 "list_ids": idx.list_ids.numpy().astype(np.uint16), "norms": idx.norms.numpy(),
                 "vbar": vbar.numpy()}
        out, _, _ = fixed.decode_step(q.numpy(), keys.numpy(), values.numpy(), index, sink=sink, local=local,
                                      fraction=1.0, scale=scale)
    np.testing.assert_allclose(out, dense.numpy(), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("which", ["fixed", "torch"])
def test_centroid_background_closed_form(which):
    # tests/test_sparse_attention.py:775-832 and tests/test_acceptance_contracts.py:6-75:
    # weights = softmax over [exact full | approx with top-k overwritten by exact]; output =
    # full + selected + (unselected weight per list) @ value centroids
    keys, coarse, books = _random_index(300, 12, 31)
    keys = keys * 0.3
    g = torch.Generator().manual_seed(32)
    values = torch.randn(300, 128, generator=g)
    q = torch.randn(3, 128, generator=g)
    sink, local, scale, frac = 4, 20, 1.0 / np.sqrt(128), 0.1
    n = 300 - local - sink
    idx = tr.encode_with_codebooks(keys[sink : sink + n], coarse, books)
    vbar = tr.value_centroids(values[sink : sink + n], idx.list_ids, 12)
    a = (tr.approximate_scores(idx, q) * scale).double()
    k = tr.resolve_topk(n, frac)
    expected = []
    for r in range(3):
        top = torch.topk(a[r], k).indices
        hybrid = a[r].clone()
        hybrid[top] = (keys[sink + top].double() @ q[r].double()) * scale
        full_idx = torch.cat([torch.arange(sink), torch.arange(sink + n, 300)])
        fl = (keys[full_idx].double() @ q[r].double()) * scale
        w = torch.softmax(torch.cat([fl, hybrid]), dim=0)
        assert abs(float(w.sum()) - 1.0) < 1e-9
        wf, wr = w[: full_idx.numel()], w[full_idx.numel() :].clone()
        sel = wr[top].clone()
        wr[top] = 0
        mass = torch.zeros(12, dtype=torch.float64).index_add_(0, idx.list_ids, wr)
        expected.append(wf @ values[full_idx].double() + sel @ values[sink + top].double() + mass @ vbar.double())
    expected = torch.stack(expected).numpy()
    if which == "torch":
        out = tr.hybrid_forward_many(q, keys, values, sink_end=sink, retrieval_end=sink + n, index=idx,
                                     vbar=vbar, fraction=frac, scale=scale).numpy()
    else:
        index = {"coarse": coarse.numpy(), "codebooks": books.numpy(),
                 "codes": tr.packed_to_words(idx.packed).numpy().astype(np.uint32),
                 "list_ids": idx.list_ids.numpy().astype(np.uint16), "norms": idx.norms.numpy(),
                 "vbar": vbar.numpy()}
        out, _, _ = fixed.decode_step(q.numpy(), keys.numpy(), values.numpy(), index, sink=sink, local=local,
                                      fraction=frac, scale=scale)
    np.testing.assert_allclose(out, expected, rtol=2e-4, atol=2e-5)


def test_attend_keeps_its_digits_when_a_selected_key_is_overrated():
    """The C oracle's attention where the approximate logit of a selected key lies tens of nats
    above every exact logit (key norms of several hundred make such rows): its weight relative to
    the largest term present is 1 against exact terms of 1e-15, so a form that adds every
    approximate weight and takes the selected ones back loses the digits.  The oracle leaves the
    selected keys out instead; checked against a float64 softmax over exactly the terms present."""
    rng = np.random.default_rng(5)
    n, sink, local, dim, lists = 200, 4, 8, 128, 6
    length = sink + n + local
    keys = rng.standard_normal((length, dim)).astype(np.float32)
    values = rng.standard_normal((length, dim)).astype(np.float32)
    q = rng.standard_normal((2, dim)).astype(np.float32)
    scale = 1.0
    list_ids = rng.integers(0, lists, n).astype(np.uint16)
    vbar = rng.standard_normal((lists, dim)).astype(np.float32)
    exact = (keys[sink : sink + n].astype(np.float64) @ q.astype(np.float64).T).T * scale
    logits = (exact + rng.standard_normal((2, n))).astype(np.float32)      # approximate logits: exact + noise ...
    k = 20
    topk = np.stack([np.argsort(-logits[g], kind="stable")[:k] for g in range(2)]).astype(np.int32)
    logits[0, topk[0, 0]] += 40.0                                           # ... and one selected key overrated by 40 nats
    logits[1, topk[1, :3]] += np.float32(60.0)
    out = fixed.attend(q, keys, values, sink, logits, topk, list_ids, vbar, scale)
    for g in range(2):
        full = list(range(sink)) + list(range(sink + n, length))
        pos = full + [sink + int(i) for i in topk[g]]
        le = (keys[pos].astype(np.float64) @ q[g].astype(np.float64)) * scale
        rest = np.ones(n, bool)
        rest[topk[g]] = False
        lb = logits[g].astype(np.float64)[rest]
        m = max(le.max(), lb.max())
        we, wb = np.exp(le - m), np.exp(lb - m)
        mass = np.bincount(list_ids[rest].astype(np.int64), weights=wb, minlength=lists)
        want = (we @ values[pos].astype(np.float64) + mass @ vbar.astype(np.float64)) / (we.sum() + mass.sum())
        np.testing.assert_allclose(out[g], want, rtol=1e-5, atol=1e-6)


def test_value_centroids_are_segment_means():
    g = torch.Generator().manual_seed(40)
    values = torch.randn(90, 16, generator=g)
    lists = torch.randint(0, 7, (90,), generator=g)
    lists[lists == 3] = 2                                     # list 3 stays empty
    vbar_t = tr.value_centroids(values, lists, 7)
    _, counts, vbar_c = fixed.value_summaries(values.numpy(), lists.numpy().astype(np.uint16), 7)
    for l in range(7):
        sel = values[lists == l]
        want = sel.double().mean(0).numpy() if sel.shape[0] else np.zeros(16)
        np.testing.assert_allclose(vbar_t[l].numpy(), want, atol=1e-6)
        np.testing.assert_allclose(vbar_c[l], want, atol=1e-6)
        assert counts[l] == sel.shape[0]


@pytest.mark.parametrize("layout", ["5d", "4d"])
def test_paged_readers_are_identity_through_a_shuffled_block_table(layout):
    g = torch.Generator().manual_seed(50)
    bs, heads, dim, seq = 16, 3, 128, 203
    nb = (seq + bs - 1) // bs
    k = torch.randn(seq, heads, dim, generator=g).to(torch.bfloat16)
    v = torch.randn(seq, heads, dim, generator=g).to(torch.bfloat16)
    table = torch.randperm(nb + 5, generator=g)[:nb].to(torch.int32)
    if layout == "5d":
        cache = torch.zeros(2, nb + 5, bs, heads, dim, dtype=torch.bfloat16)
        kc, vc = cache[0], cache[1]
    else:
        cache = torch.zeros(nb + 5, heads, bs, 2 * dim, dtype=torch.bfloat16)
        kc, vc = tr.split_kv_cache(cache)
    for p in range(seq):
        kc[table[p // bs], p % bs] = k[p]
        vc[table[p // bs], p % bs] = v[p]
    gk, gv = tr.gather_paged(cache, table, seq)
    assert torch.equal(gk[0], k.permute(1, 0, 2)) and torch.equal(gv[0], v.permute(1, 0, 2))
    rk, rv = tr.gather_paged_range(cache, table, 37, 150)
    assert torch.equal(rk, k[37:150].permute(1, 0, 2)) and torch.equal(rv, v[37:150].permute(1, 0, 2))
    tok = torch.randint(0, seq, (heads, 2, 9), generator=g)
    ak, av = tr.gather_paged_at(cache, table, tok)
    for h in range(heads):
        assert torch.equal(ak[h], k[tok[h], h]) and torch.equal(av[h], v[tok[h], h])
    # the C oracle's addressing
    kc_c = kc if kc.is_contiguous() else kc
    strides = (kc_c.stride(0), kc_c.stride(1), kc_c.stride(2))
    base = cache.view(torch.int16).reshape(-1).numpy().view(np.uint16)
    off = kc_c.storage_offset()
    pos = np.array([0, 15, 16, 17, 202, 101], np.int64)
    got = fixed.paged_gather(base[off:], strides, dim, bs, table.numpy(), 1, pos)
    want = k[torch.from_numpy(pos), 1].view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, want)
