"""GPU parity tests: every HIP kernel, through the C ABI, against the fixed-order CPU oracle.

Integer results (packed codes, list ids, top-k index sets) and fp32 table/score values are
compared bit-exactly; attention outputs within 1e-4 (fp32 K/V) or 2e-3 max-abs (bf16 K/V).
"""

import numpy as np
import pytest
import torch

from oracle import fixed
from tests.gpu_util import DIM, SCALE, Problem, u16, u32

pytestmark = pytest.mark.gpu

ops = pytest.importorskip("pqhsa_release_amd.ops")


def _cuda():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    return "cuda"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("paged", [None, "5d", "4d"])
def test_encode_bulk_and_row_kernels_match_oracle_bitwise(dtype, paged):
    dev = _cuda()
    p = Problem(lens=[900, 517], heads=2, lists=48, dtype=dtype, seed=3)
    idx = p.device_index(dev, upload_codes=False)
    if paged:
        cache, table = p.paged_kv(paged)
        kv = ops.kv_paged(cache, table)
    else:
        kv = ops.kv_contiguous(*p.dense_kv())
    counts = [p.n(b) for b in range(p.B)]
    # bulk kernel for all but the last 5 rows, one-row kernel for the rest
    ops.encode(kv, idx, p.sink, [0, 0], [c - 5 for c in counts])
    ops.encode(kv, idx, p.sink, [c - 5 for c in counts], [5, 5])
    torch.cuda.synchronize()
    for (b, h), ix in p.index.items():
        bh, n = b * p.H + h, p.n(b)
        assert np.array_equal(u32(idx.codes[bh, :n]), ix["codes"]), (b, h)
        assert np.array_equal(u16(idx.list_ids[bh, :n]), ix["list_ids"]), (b, h)
        assert np.array_equal(idx.norms[bh, :n].cpu().numpy(), ix["norms"]), (b, h)
    # the reference's [N, 4] uint8 packing is the byte view of the words
    packed = idx.packed_bytes(0, p.n(0)).cpu().numpy()
    w = p.index[0, 0]["codes"]
    assert np.array_equal(packed[:, 1] >> 4, (w >> 12) & 15) and np.array_equal(packed[:, 0] & 15, w & 15)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("paged", [None, "5d"])
def test_encode_with_matrix_core_candidates_matches_oracle_bitwise(dtype, paged):
    """pqhsa_encode_bulk: the nearest list comes from two candidates of a half-precision matrix
    product, measured in the oracle's order; 48 lists leave half of the second tile as padding."""
    dev = _cuda()
    p = Problem(lens=[900, 517], heads=2, lists=48, dtype=dtype, seed=3)
    idx = p.device_index(dev, upload_codes=False)
    kv = ops.kv_paged(*p.paged_kv(paged)) if paged else ops.kv_contiguous(*p.dense_kv())
    counts = [p.n(b) for b in range(p.B)]
    ops.encode(kv, idx, p.sink, [0, 0], [c - 300 for c in counts], bulk=True)
    ops.encode(kv, idx, p.sink, [c - 300 for c in counts], [300, 300], bulk=True)     # a second call, from an offset
    torch.cuda.synchronize()
    for (b, h), ix in p.index.items():
        bh, n = b * p.H + h, p.n(b)
        assert np.array_equal(u32(idx.codes[bh, :n]), ix["codes"]), (b, h)
        assert np.array_equal(u16(idx.list_ids[bh, :n]), ix["list_ids"]), (b, h)
        assert np.array_equal(idx.norms[bh, :n].cpu().numpy(), ix["norms"]), (b, h)
        assert np.array_equal(idx.pos[bh, :n].cpu().numpy(), np.arange(n)), (b, h)


@pytest.mark.parametrize("case", ["clustered", "twin_lists", "wide_tables", "beyond_half_precision", "one_list",
                                  "odd_keys", "between_two_lists", "between_three_lists", "many_lists",
                                  "padded_lists"])
def test_encode_with_matrix_core_candidates_equals_the_full_measurement(case):
    """The candidate pass never changes a bit of the encode, also where its estimate cannot tell
    lists apart: centroid rows that are equal or 1e-5 apart (every key near them measures all
    lists), keys half way between two or three centroids (distances equal to within 1e-4, far
    inside the estimate's error), tables of large values (the error bound grows with them), a
    centroid row with a value beyond fp16 and the padding rows of a sequence with fewer keys than
    lists (such rows take no part in the estimate: they cannot be the nearest), a single list,
    zero / huge / non-finite keys."""
    dev = _cuda()
    gen = torch.Generator().manual_seed(17)
    B, H, L, n = 2, 2, {"one_list": 1, "many_lists": 4096}.get(case, 200), 6000   # 4096: all 12 bits of a hint's list ids
    centres = torch.randn(B, H, L, 128, generator=gen)
    pick = torch.randint(0, L, (B, H, n), generator=gen)
    keys = torch.gather(centres, 2, pick.unsqueeze(-1).expand(-1, -1, -1, 128)) + 0.4 * torch.randn(B, H, n, 128, generator=gen)
    coarse = centres / centres.norm(dim=-1, keepdim=True)
    if case == "twin_lists":
        coarse[:, :, 100:150] = coarse[:, :, 0:50]                      # equal rows: the lower id must win
        coarse[:, :, 150:200] = coarse[:, :, 50:100] + 1e-5 * torch.randn(B, H, 50, 128, generator=gen)
    if case == "wide_tables":
        coarse = coarse * 37.0
    if case == "beyond_half_precision":
        coarse[:, :, 7, 3] = 5.0e4
    if case == "padded_lists":    # a sequence with fewer keys than lists: the unused rows hold the padding centroid
        coarse[:, :, 150:] = ops.DeviceIndex.PAD_CENTROID
        coarse[1, :, 3:] = ops.DeviceIndex.PAD_CENTROID
    if case in ("between_two_lists", "between_three_lists"):
        k = 2 if case == "between_two_lists" else 3
        near = torch.stack([torch.gather(coarse, 2, torch.randint(0, L, (B, H, n), generator=gen).unsqueeze(-1)
                                         .expand(-1, -1, -1, 128)) for _ in range(k)]).sum(0)
        keys = 5.0 * near + 1e-4 * torch.randn(B, H, n, 128, generator=gen)
    if case == "odd_keys":
        keys[:, :, 0] = 0.0
        keys[:, :, 1] = 1.0e-30
        keys[:, :, 2] = 1.0e30
        keys[:, :, 3, 5] = float("inf")
        keys[:, :, 4, 9] = float("nan")
        keys[:, :, 5] = coarse[:, :, 11] * 3.0                            # exactly on a centroid's ray
    keys = keys.to(dev)
    kv = ops.kv_contiguous(keys, torch.zeros_like(keys))
    got = []
    for bulk in (False, True):
        idx = ops.DeviceIndex(B, H, L, n + 64, dev)
        idx.coarse.copy_(coarse.reshape(B * H, L, 128))
        idx.codebooks.copy_(0.1 * torch.randn(B * H, 8, 16, 16, generator=torch.Generator().manual_seed(5)))
        idx.set_counts([n, n - 777])
        ops.encode(kv, idx, 0, [0, 0], [n, n - 777], bulk=bulk)
        torch.cuda.synchronize()
        got.append((u16(idx.list_ids), u32(idx.codes), idx.norms.cpu().numpy().view(np.uint32)))
    for b, cnt in enumerate([n, n - 777]):
        rows = slice(b * H, (b + 1) * H)
        for name, x, y in zip(("list ids", "codes", "norms"), got[0], got[1]):
            assert np.array_equal(x[rows, :cnt], y[rows, :cnt]), (case, b, name)
    if case in ("clustered", "wide_tables"):   # ... and the lists are the nearest ones (float64 check of a sample)
        lid = got[1][0][0, :512].astype(np.int64)
        d = keys[0, 0, :512].double().cpu()
        d = d / d.norm(dim=-1, keepdim=True)
        dist = torch.cdist(d, coarse[0, 0].double())
        best = dist.min(dim=1).values
        assert torch.all(dist[torch.arange(512), torch.from_numpy(lid)] <= best + 1e-5)


@pytest.mark.parametrize("k", [1, 5, 48, 512, 1000])
def test_nearest_rows_gives_the_nearest_centroid_of_every_direction(k):
    """pqhsa_nearest_rows (the coarse k-means' assignment step): for unit rows the answer is a
    nearest centroid by a float64 measurement (to the 1e-6 that fp32 distances can tell apart),
    equal centroid rows go to the lower index, and a row that is not unit is judged by its
    direction."""
    dev = _cuda()
    gen = torch.Generator().manual_seed(100 + k)
    p, r = 3, 3001
    centres = torch.randn(p, k, 128, generator=gen)
    centres = centres / centres.norm(dim=-1, keepdim=True) * (0.5 + 0.5 * torch.rand(p, k, 1, generator=gen))
    rows = torch.gather(centres, 1, torch.randint(0, k, (p, r), generator=gen).unsqueeze(-1).expand(-1, -1, 128))
    rows = rows + 0.2 * torch.randn(p, r, 128, generator=gen)
    rows = rows / rows.norm(dim=-1, keepdim=True)
    if k >= 5:
        centres[:, 4] = centres[:, 1]                    # equal rows: 1 wins over 4
    rows[:, 7] *= 37.0                                   # not unit: judged by its direction
    got = ops.nearest_rows(rows.to(dev), centres.to(dev)).cpu()
    unit = (rows / rows.norm(dim=-1, keepdim=True)).double()
    dist = torch.cdist(unit, centres.double()) ** 2
    best = dist.min(dim=2).values
    mine = torch.gather(dist, 2, got.unsqueeze(-1)).squeeze(-1)
    assert bool((mine <= best + 1e-6).all())
    assert int((got == 4).sum()) == 0 or k < 5
    fp32 = ((centres * centres).sum(-1).unsqueeze(1) - 2.0 * torch.bmm(unit.float(), centres.transpose(1, 2))).argmin(dim=2)
    if k >= 5:
        fp32[fp32 == 4] = 1                              # (a product matrix may round the twin columns apart)
    assert float((got == fp32).float().mean()) > 0.999


def test_nearest_codewords_gives_the_nearest_codeword_of_every_row():
    """pqhsa_nearest_codewords (the codebook k-means' assignment step): a nearest codeword by a
    float64 measurement for every row, the lower index among equal codewords, the fp32 product
    form's answer almost everywhere."""
    dev = _cuda()
    gen = torch.Generator().manual_seed(31)
    p, r = 5, 4099
    words = 0.2 * torch.randn(p, 16, 16, generator=gen)
    words[:, 9] = words[:, 2]                                        # equal codewords: 2 wins over 9
    rows = torch.gather(words, 1, torch.randint(0, 16, (p, r), generator=gen).unsqueeze(-1).expand(-1, -1, 16))
    rows = rows + 0.05 * torch.randn(p, r, 16, generator=gen)
    got = ops.nearest_codewords(rows.to(dev), words.to(dev)).cpu()
    dist = torch.cdist(rows.double(), words.double()) ** 2
    mine = torch.gather(dist, 2, got.unsqueeze(-1)).squeeze(-1)
    assert bool((mine <= dist.min(dim=2).values + 1e-9).all())
    assert int((got == 9).sum()) == 0
    fp32 = ((words * words).sum(-1).unsqueeze(1) - 2.0 * torch.bmm(rows, words.transpose(1, 2))).argmin(dim=2)
    fp32[fp32 == 9] = 2
    assert float((got == fp32).float().mean()) > 0.999


@pytest.mark.parametrize("k", [1, 3, 16, 17, 32, 36, 512, 600, 1024, 2000])
def test_nearest_from_products_is_the_elementwise_argmin(k):
    """pqhsa_nearest_from_products against the three torch ops it stands for, bit for bit: equal
    values (lowest index wins), +inf rows, NaNs (the first NaN wins, as in torch.argmin), and an
    output that is a column slice of a wider tensor."""
    dev = _cuda()
    gen = torch.Generator().manual_seed(k)
    p, r = 3, 1501
    dots = torch.randn(p, r, k, generator=gen)
    sq = torch.rand(p, k, generator=gen) * 2.0
    if k >= 3:
        dots[:, 5] = dots[:, 5, :1]                                 # whole rows of equal products ...
        sq[0] = sq[0, 0]                                            # ... and of equal norms: all values equal
        dots[1, 7, k // 2] = float("-inf")                          # value +inf in the middle
        dots[1, 8] = float("-inf")                                  # a row of +inf only
        dots[2, 9, k - 1] = float("nan")
        dots[2, 10, 1] = float("nan"); dots[2, 10, k - 1] = float("nan")
        dots[:, 11, k - 1] = dots[:, 11].max(dim=1).values + 1.0    # the minimum in the last place
    dots, sq = dots.to(dev), sq.to(dev)
    want = (sq.unsqueeze(1) - 2.0 * dots).argmin(dim=2)
    wide = torch.full((p, r + 9), -1, dtype=torch.int64, device=dev)
    ops.nearest_from_products(dots, sq, wide[:, 4 : 4 + r])
    torch.cuda.synchronize()
    assert torch.equal(wide[:, 4 : 4 + r], want)
    assert int((wide[:, :4] != -1).sum()) == 0 and int((wide[:, 4 + r :] != -1).sum()) == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_value_summaries_and_append_match_oracle(dtype):
    dev = _cuda()
    p = Problem(lens=[700], heads=2, lists=32, dtype=dtype, seed=5)
    idx = p.device_index(dev, finalize=False)       # appends go to the insertion-order tail
    kv = ops.kv_contiguous(*p.dense_kv())
    idx.vbar.zero_()
    n = p.n(0)
    # build summaries over the first n - 3 keys, then append 3 (one launch)
    idx.set_counts([n - 3])
    ops.value_summaries(kv, idx, p.sink)
    ops.encode_append(kv, idx, p.sink, [n - 3], [3])
    idx.set_counts([n])
    torch.cuda.synchronize()
    for h in range(p.H):
        ix = p.index[0, h]
        vals = p.values[0, h][p.sink : p.sink + n].numpy()
        sums, counts, vbar = fixed.value_summaries(vals[: n - 3], ix["list_ids"][: n - 3], p.L)
        for j in range(n - 3, n):
            fixed.value_append(vals[j], int(ix["list_ids"][j]), sums, counts, vbar)
        # untouched lists keep the mean of the build; touched ones were recomputed
        np.testing.assert_array_equal(idx.vcount[h].cpu().numpy(), counts)
        np.testing.assert_allclose(idx.vsum[h].cpu().numpy(), sums, rtol=0, atol=1e-5)
        np.testing.assert_allclose(idx.vbar[h].cpu().numpy(), vbar, rtol=0, atol=1e-6)
        assert np.array_equal(u32(idx.codes[h, n - 3 : n]), ix["codes"][n - 3 :])
        assert np.array_equal(u16(idx.list_ids[h, n - 3 : n]), ix["list_ids"][n - 3 :])


@pytest.mark.parametrize("groups", [1, 3, 4, 7])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_lut_build_and_scan_match_oracle_bitwise(groups, dtype):
    dev = _cuda()
    p = Problem(lens=[1500, 1111], heads=2, groups=groups, lists=40, dtype=dtype, seed=7)
    idx = p.device_index(dev)
    q = p.q_tensor()
    qnorm, lut, ls = ops.lut_build(q, idx, groups)
    logits = ops.lut_scan(idx, groups, qnorm, lut, ls, SCALE)
    torch.cuda.synchronize()
    for (b, h), ix in p.index.items():
        bh, n = b * p.H + h, p.n(b)
        oq, olut, ols = fixed.lut_build(p.queries[b, h].numpy(), ix["coarse"], ix["codebooks"])
        assert np.array_equal(qnorm[bh, :groups].cpu().numpy(), oq)
        assert np.array_equal(lut[bh, :, :, :groups].permute(2, 0, 1).cpu().numpy(), olut)
        assert np.array_equal(ls[bh, :, :groups].T.cpu().numpy(), ols)
        assert (lut[bh, :, :, groups:] == 0).all() and (ls[bh, :, groups:] == 0).all()
        want = fixed.scan(ix["codes"], ix["list_ids"], ix["norms"], olut, ols, oq, SCALE)
        got = logits[bh, :, :n].cpu().numpy()
        assert np.array_equal(got, want), (b, h, np.abs(got - want).max())


def test_lut_build_large_batch_takes_several_tiles_per_block():
    """With many streams the table-building launch gives a block several 64-list tiles in turn
    (so that it still fits the chip at once): same bits as the oracle, last partial tile included."""
    dev = _cuda()
    batch, heads, groups, lists = 30, 4, 4, 488      # 120 streams x (1 + 8 tiles) blocks would not fit at once
    idx = ops.DeviceIndex(batch, heads, lists, 64, dev)
    gen = torch.Generator(device="cpu").manual_seed(91)
    idx.coarse.copy_(torch.randn(idx.coarse.shape, generator=gen))
    idx.codebooks.copy_(0.3 * torch.randn(idx.codebooks.shape, generator=gen))
    q = torch.randn(batch, heads * groups, DIM, generator=gen)
    qnorm, lut, ls = ops.lut_build(q.to(dev), idx, groups)
    torch.cuda.synchronize()
    coarse, books = idx.coarse.cpu().numpy(), idx.codebooks.cpu().numpy()
    for bh in (0, 1, 57, 118, 119):
        b, h = divmod(bh, heads)
        oq, olut, ols = fixed.lut_build(q[b, h * groups : (h + 1) * groups].numpy(), coarse[bh], books[bh])
        assert np.array_equal(qnorm[bh, :groups].cpu().numpy(), oq), bh
        assert np.array_equal(lut[bh, :, :, :groups].permute(2, 0, 1).cpu().numpy(), olut), bh
        assert np.array_equal(ls[bh, :, :groups].T.cpu().numpy(), ols), bh


@pytest.mark.parametrize("stride_pad,offset", [(0, 0), (3, 0), (0, 1), (5, 3)])
def test_lut_scan_row_stride_and_alignment(stride_pad, offset):
    # The scan writes four neighbouring logits as one 16-byte store when the destination allows it;
    # an odd row stride or an unaligned base takes the element-wise path.  Both must give the
    # oracle's bits, and neither may touch a column at or past n.
    from pqhsa_release_amd import _lib

    dev = _cuda()
    groups = 4
    p = Problem(lens=[1501, 1110], heads=2, groups=groups, lists=40, dtype=torch.bfloat16, seed=17)
    idx = p.device_index(dev)
    qnorm, lut, ls = ops.lut_build(p.q_tensor(), idx, groups)
    bh, stride = idx.batch * idx.kv_heads, idx.n_cap + stride_pad
    buf = torch.full((bh * groups * stride + 8,), -7.0, dtype=torch.float32, device=dev)
    out = buf[offset : offset + bh * groups * stride]
    lib = _lib.load()
    _lib.check(lib.pqhsa_lut_scan(idx.ref(), groups, int(idx.n_max), qnorm.data_ptr(), lut.data_ptr(), ls.data_ptr(),
                                  float(SCALE), out.data_ptr(), stride, torch.cuda.current_stream().cuda_stream),
               "pqhsa_lut_scan")
    torch.cuda.synchronize()
    got_all = out.view(bh, groups, stride).cpu().numpy()
    for (b, h), ix in p.index.items():
        r, n = b * p.H + h, p.n(b)
        oq, olut, ols = fixed.lut_build(p.queries[b, h].numpy(), ix["coarse"], ix["codebooks"])
        want = fixed.scan(ix["codes"], ix["list_ids"], ix["norms"], olut, ols, oq, SCALE)
        assert np.array_equal(got_all[r, :, :n], want)
        assert (got_all[r, :, n:] == -7.0).all()
    assert (buf[:offset] == -7.0).all() and (buf[offset + bh * groups * stride :] == -7.0).all()


@pytest.mark.parametrize("stride", [5000, 5001, 5003])  # rows 16-byte aligned, and not
def test_topk_radix_on_logit_matrix_with_ties(stride):
    dev = _cuda()
    rng = np.random.default_rng(11)
    rows = 9
    logits = rng.standard_normal((rows, stride)).astype(np.float32)
    logits[1, :] = 0.5                                    # all equal: pure lowest-index rule
    logits[2, 100:400] = logits[2].max() + 1              # wide tie at the top
    logits[3, ::7] = np.sort(logits[3])[::-1][40]         # ties straddling the k boundary
    logits[4] = np.abs(logits[4]) * -1                    # all negative
    logits[5, :10] = [0.0, -0.0, 0.0, -0.0, 1.0, -0.0, 0.0, 2.0, -0.0, 0.0]
    logits[5, 10:] = -1.0
    n = [5000, 4097, 5000, 4999, 1, 12, 2500, 5000, 64]
    k = [100, 37, 150, 41, 1, 6, 2500, 0, 63]
    idx, val = ops.topk_radix(torch.from_numpy(logits).to(dev), n, k)
    torch.cuda.synchronize()
    idx, val = idx.cpu().numpy(), val.cpu().numpy()
    for r in range(rows):
        want_idx, _ = fixed.topk(logits[r, : n[r]], k[r])
        got = idx[r, : k[r]]
        assert np.array_equal(np.sort(got), np.sort(want_idx)), r      # exact set
        assert np.array_equal(val[r, : k[r]], logits[r, got]), r


@pytest.mark.parametrize("case", [
    dict(lens=[2048], heads=1, groups=1, lists=64, dtype=torch.float32, fraction=0.02, kv="dense"),
    dict(lens=[8192], heads=1, groups=1, lists=512, dtype=torch.float32, fraction=0.02, kv="dense"),   # cfg 0 in full
    dict(lens=[3000, 1800], heads=2, groups=4, lists=64, dtype=torch.bfloat16, fraction=0.02, kv="5d"),
    dict(lens=[2500, 1900, 700], heads=2, groups=4, lists=32, dtype=torch.bfloat16, fraction=0.05, kv="4d"),
    dict(lens=[2200], heads=2, groups=7, lists=48, dtype=torch.bfloat16, fraction=0.02, kv="5d"),
    dict(lens=[1500], heads=1, groups=2, lists=16, dtype=torch.float16, fraction=0.1, kv="dense"),
])
@pytest.mark.parametrize("general_path", [False, True, "fused"], ids=["short_context_kernel", "general", "general_one_launch"])
def test_decode_step_topk_bitexact_and_output_close(case, general_path):
    """All forms of the step against the oracle: the single kernel that serves short contexts
    (taken by default at these sizes), the general path (scan, selection and attention, each its own
    kernel where the shape allows) and the general path with those three in one launch."""
    dev = _cuda()
    p = Problem(lens=case["lens"], heads=case["heads"], groups=case["groups"], lists=case["lists"],
                dtype=case["dtype"], seed=13)
    idx = p.device_index(dev)
    if case["kv"] == "dense":
        kv = ops.kv_contiguous(*p.dense_kv())
    else:
        kv = ops.kv_paged(*p.paged_kv(case["kv"]))
    k_cap = ops.resolve_topk(p.n_max, case["fraction"], 0)
    ws = ops.DecodeWorkspace(idx, p.G, k_cap)
    # 16-bit K/V are read in place; the query/output pair is tried both in fp32 (the stated
    # 2e-3 max-abs bound applies as is) and in the cache dtype (the output is then rounded to
    # 8 or 11 significant bits, which alone costs up to 2^-9 relative)
    q_dtypes = [torch.float32] if case["dtype"] == torch.float32 else [torch.float32, case["dtype"]]
    for q_dtype in q_dtypes:
        q = p.q_tensor().to(q_dtype)
        out = torch.full_like(q, float("nan"))  # a row no workgroup folds would stay NaN
        ops.decode_step(q, out, kv, idx, p.G, p.seq_lens(), sink=p.sink, full_max=p.sink + p.local,
                        fraction=case["fraction"], topk=0, scale=SCALE, workspace=ws, **_path(general_path))
        torch.cuda.synchronize()
        tol = 1e-4 if case["dtype"] == torch.float32 else 2e-3
        rel = 0.0 if q_dtype == torch.float32 else (2.0 ** -8 if q_dtype == torch.bfloat16 else 2.0 ** -11)
        cnt = ws.topk_cnt.cpu().numpy().reshape(p.B, p.H, p.G)
        tidx = ws.topk_idx.cpu().numpy().reshape(p.B, p.H, p.G, -1)
        tval = ws.topk_val.cpu().numpy().reshape(p.B, p.H, p.G, -1)
        o = out.float().cpu().numpy().reshape(p.B, p.H, p.G, DIM)
        worst = 0.0
        for (b, h) in p.index:
            want_out, want_idx, logits = p.oracle_step(b, h, case["fraction"])
            k = want_idx.shape[1]
            for g in range(p.G):
                assert cnt[b, h, g] == k
                got = tidx[b, h, g, :k]
                assert np.array_equal(np.sort(got), np.sort(want_idx[g])), (b, h, g)  # bit-exact set
                assert np.array_equal(tval[b, h, g, :k], logits[g, got]), (b, h, g)  # and their logits
            err = np.abs(o[b, h] - want_out)
            assert (err <= tol + rel * np.abs(want_out)).all(), (b, h, q_dtype, err.max())
            worst = max(worst, float(err.max()))
        print(f"decode_step {case['dtype']} q={q_dtype}: max abs err {worst:.3e}")


def test_stand_alone_scan_list_mass_matches_the_logits():
    """pqhsa_lut_scan_mass: per-list sums of exp(logit - reference) in one pass over the index, against
    the same sums formed in float64 from the oracle's logits (the scan's logits are the oracle's bit
    for bit; the sums are float atomics, compared to 1e-5)."""
    dev = _cuda()
    p = Problem(lens=[5000, 2300], heads=2, groups=3, lists=32, seed=71)
    idx = p.device_index(dev)
    qnorm, lut, ls = ops.lut_build(p.q_tensor(), idx, p.G)
    gp = qnorm.shape[-1] if qnorm.ndim > 1 else qnorm.numel() // (p.B * p.H)
    ref = torch.zeros(p.B * p.H, gp, dtype=torch.float32, device=dev)
    want = {}
    for (b, h), ix in p.index.items():
        _, _, logits = p.oracle_step(b, h, 0.02)                      # [G, n]
        bh = b * p.H + h
        for g in range(p.G):
            ref[bh, g] = float(logits[g].max())
        lists = ix["list_ids"].astype(np.int64)
        w = np.exp(logits.astype(np.float64) - logits.max(axis=1, keepdims=True).astype(np.float64))
        m = np.zeros((p.L, p.G))
        for g in range(p.G):
            np.add.at(m[:, g], lists, w[g])
        want[bh] = m
    mass = ops.lut_scan_mass(idx, p.G, qnorm, lut, ls, SCALE, ref)
    torch.cuda.synchronize()
    got = mass.cpu().numpy()
    for bh, m in want.items():
        # (the weights of a wave's keys are summed per list as differences of one prefix sum over its
        # lanes: absolute accuracy about 1e-7 of the row's mass, which is what a softmax needs)
        for g in range(p.G):
            np.testing.assert_allclose(got[bh, :, g], m[:, g], rtol=1e-5, atol=5e-7 * m[:, g].sum())
        assert (got[bh, :, p.G:] == 0).all()                          # padded rows of the group carry nothing


@pytest.mark.parametrize("lens,groups,lists,block_keys,finalize", [
    ([5000, 2300], 3, 32, 1024, True),      # ragged: the short stream's last blocks are empty
    ([3001], 4, 64, 700, True),             # blocks that are no multiple of the workgroup, a ragged last one
    ([1800, 1800], 1, 16, 4096, False),     # one block per row, index in arrival order
    ([2600], 7, 40, 256, True),             # padded group
])
def test_stand_alone_scan_block_statistics_and_their_fold(lens, groups, lists, block_keys, finalize):
    """pqhsa_lut_scan_stats + pqhsa_block_reduce: per block of stored keys the largest logit (the
    oracle's, bit for bit) and the sum of exp(logit - maximum) (against float64 sums over the
    oracle's logits, 1e-5); folded, the row's maximum and its log-sum-exp over all indexed keys."""
    dev = _cuda()
    p = Problem(lens=lens, heads=2, groups=groups, lists=lists, seed=83)
    idx = p.device_index(dev, finalize=finalize)
    qnorm, lut, ls = ops.lut_build(p.q_tensor(), idx, p.G)
    bmax, bexp = ops.lut_scan_stats(idx, p.G, qnorm, lut, ls, SCALE, block_keys=block_keys)
    row_max, exp_sum = ops.block_reduce(bmax, bexp)
    torch.cuda.synchronize()
    blocks = -(-int(idx.n_max) // block_keys)
    assert tuple(bmax.shape) == (p.B * p.H, p.G, blocks)
    got_m, got_e = bmax.cpu().numpy(), bexp.cpu().numpy()
    got_rm, got_es = row_max.cpu().numpy(), exp_sum.cpu().numpy()
    pos = idx.pos.cpu().numpy()
    for (b, h) in p.index:
        bh, n = b * p.H + h, p.n(b)
        _, _, logits = p.oracle_step(b, h, 0.02)                      # [G, n] by retrieval-local index
        stored = logits[:, pos[bh, :n]]                               # ... and in the order of the stored keys
        for c in range(blocks):
            part = stored[:, c * block_keys : min(n, (c + 1) * block_keys)]
            if part.shape[1] == 0:
                assert (got_m[bh, :, c] == -np.inf).all() and (got_e[bh, :, c] == 0).all()
                continue
            top = part.max(axis=1)
            assert np.array_equal(got_m[bh, :, c], top)
            np.testing.assert_allclose(got_e[bh, :, c], np.exp(part.astype(np.float64) - top[:, None]).sum(axis=1), rtol=1e-5)
        top = stored.max(axis=1)
        assert np.array_equal(got_rm[bh], top)
        lse = top + np.log(np.exp(stored.astype(np.float64) - top[:, None]).sum(axis=1))
        np.testing.assert_allclose(got_rm[bh] + np.log(got_es[bh].astype(np.float64)), lse, rtol=0, atol=2e-5)


def test_block_reduce_of_rows_without_keys_and_of_many_blocks():
    dev = _cuda()
    rng = np.random.default_rng(5)
    bm = rng.standard_normal((6, 1000)).astype(np.float32) * 20
    be = (rng.random((6, 1000)) * 256 + 1).astype(np.float32)
    bm[1], be[1] = -np.inf, 0.0                                       # a row without keys
    bm[2, 3:], be[2, 3:] = -np.inf, 0.0                               # three blocks with keys
    bm[3, :] = bm[3, 0]                                               # equal maxima
    row_max, exp_sum = ops.block_reduce(torch.from_numpy(bm).to(dev), torch.from_numpy(be).to(dev))
    torch.cuda.synchronize()
    rm, es = row_max.cpu().numpy(), exp_sum.cpu().numpy()
    want_m = bm.max(axis=1)
    assert np.array_equal(rm, want_m)
    assert rm[1] == -np.inf and es[1] == 0.0
    with np.errstate(invalid="ignore"):
        w = np.where(np.isfinite(bm), be.astype(np.float64) * np.exp(bm.astype(np.float64) - want_m[:, None]), 0.0)
    keep = [0, 2, 3, 4, 5]
    np.testing.assert_allclose(es[keep], w.sum(axis=1)[keep], rtol=1e-5)


def test_decode_step_all_selected_equals_dense_attention():
    dev = _cuda()
    p = Problem(lens=[600], heads=1, groups=2, lists=16, seed=17)
    idx = p.device_index(dev)
    kv = ops.kv_contiguous(*p.dense_kv())
    q = p.q_tensor()
    out = torch.full_like(q, float("nan"))  # a row no workgroup folds would stay NaN
    ws = ops.DecodeWorkspace(idx, p.G, p.n_max)
    ops.decode_step(q, out, kv, idx, p.G, p.seq_lens(), sink=p.sink, full_max=p.sink + p.local, fraction=1.0,
                    topk=0, scale=SCALE, workspace=ws)
    k64, v64, q64 = p.keys[0, 0].double(), p.values[0, 0].double(), p.queries[0, 0].double()
    dense = torch.softmax((q64 @ k64.T) * SCALE, dim=-1) @ v64
    np.testing.assert_allclose(out[0].cpu().double().numpy(), dense.numpy(), rtol=1e-4, atol=1e-5)


def test_decode_step_degenerate_shapes():
    dev = _cuda()
    # no indexed keys at all (context shorter than sink + local): plain exact attention
    p = Problem(lens=[40], heads=1, groups=2, lists=8, seed=19)
    assert p.n(0) == 0
    idx = ops.DeviceIndex(1, 1, 8, 8, dev)
    idx.set_counts([0])
    kv = ops.kv_contiguous(*p.dense_kv())
    q = p.q_tensor()
    out = torch.full_like(q, float("nan"))
    ws = ops.DecodeWorkspace(idx, p.G, 1)
    ops.decode_step(q, out, kv, idx, p.G, p.seq_lens(), sink=p.sink, full_max=40, fraction=0.02, topk=0,
                    scale=SCALE, workspace=ws)
    k64, v64, q64 = p.keys[0, 0].double(), p.values[0, 0].double(), p.queries[0, 0].double()
    dense = torch.softmax((q64 @ k64.T) * SCALE, dim=-1) @ v64
    np.testing.assert_allclose(out[0].cpu().double().numpy(), dense.numpy(), rtol=1e-4, atol=1e-5)
    assert (ws.topk_cnt == 0).all()


@pytest.mark.parametrize("layout", ["5d", "4d"])
def test_paged_readers_match_contiguous_tensor(layout):
    dev = _cuda()
    p = Problem(lens=[333, 190], heads=3, lists=8, dtype=torch.bfloat16, seed=23)
    cache, table = p.paged_kv(layout)
    kv = ops.kv_paged(cache, table)
    for b in range(p.B):
        want_k = torch.stack([p.keys[b, h] for h in range(p.H)]).to(torch.bfloat16)
        want_v = torch.stack([p.values[b, h] for h in range(p.H)]).to(torch.bfloat16)
        k, v = ops.paged_gather_range(kv, b, 0, p.lens[b])
        assert torch.equal(k.cpu(), want_k) and torch.equal(v.cpu(), want_v)
        k, v = ops.paged_gather_range(kv, b, 37, 150)
        assert torch.equal(k.cpu(), want_k[:, 37:150]) and torch.equal(v.cpu(), want_v[:, 37:150])
        pos = torch.randint(0, p.lens[b], (p.H, 2, 11), generator=torch.Generator().manual_seed(b))
        k, v = ops.paged_gather_at(kv, b, pos.to(dev))
        for h in range(p.H):
            assert torch.equal(k[h].cpu(), want_k[h][pos[h]]) and torch.equal(v[h].cpu(), want_v[h][pos[h]])


def test_missing_or_bad_arguments_fail_loudly():
    dev = _cuda()
    p = Problem(lens=[300], heads=1, lists=8, seed=29)
    idx = p.device_index(dev)
    with pytest.raises(ValueError):
        ops.lut_build(torch.zeros(1, 1, 64, device=dev), idx, 1)            # wrong head dim
    with pytest.raises(ValueError):
        ops.kv_contiguous(torch.zeros(1, 1, 8, 128), torch.zeros(1, 1, 8, 128))   # CPU tensors
    with pytest.raises(ValueError):
        ops.lut_build(torch.zeros(1, 17, 128, device=dev), idx, 17)         # G too large


def _path(general_path):
    """Keyword arguments that pick the form of the step: False = the default (one kernel for short
    contexts), True = the general path, "fused" = the general path with scan, selection and
    attention in one launch (where the shape allows; else the flag changes nothing), "apart" = the
    general path with the tables and the threshold estimate as two launches."""
    return dict(general_path=bool(general_path), one_launch=general_path == "fused",
                separate_tables=general_path == "apart")


def _check_step(p, idx, kv, ws, fraction, tol=1e-4, general_path=True):
    """(The tests that use this are about the general path's estimate, candidate area and layouts:
    every form of it that the shape allows is run: tables and thresholds in one launch or two, and
    the one-launch scan + selection + attention.)"""
    runs = 1
    if general_path is True and ops.decode_step_launches(idx, p.G, ws, general_path=True, one_launch=True) == 3:
        runs += _check_step(p, idx, kv, ws, fraction, tol, "fused")
    if general_path is True and ops.decode_step_launches(idx, p.G, ws, general_path=True) == 4:
        runs += _check_step(p, idx, kv, ws, fraction, tol, "apart")
    q = p.q_tensor()
    out = torch.full_like(q, float("nan"))  # a row no workgroup folds would stay NaN
    ws.topk_idx.fill_(-1)
    ops.decode_step(q, out, kv, idx, p.G, p.seq_lens(), sink=p.sink, full_max=p.sink + p.local, fraction=fraction,
                    topk=0, scale=SCALE, workspace=ws, **_path(general_path))
    torch.cuda.synchronize()
    assert ws.fused_aborts() == 0
    tidx = ws.topk_idx.cpu().numpy().reshape(p.B, p.H, p.G, -1)
    o = out.float().cpu().numpy().reshape(p.B, p.H, p.G, DIM)
    for (b, h) in p.index:
        want_out, want_idx, _ = p.oracle_step(b, h, fraction)
        k = want_idx.shape[1]
        for g in range(p.G):
            assert np.array_equal(np.sort(tidx[b, h, g, :k]), np.sort(want_idx[g])), (b, h, g)
        assert np.abs(o[b, h] - want_out).max() <= tol, (b, h)
    return runs


@pytest.mark.parametrize("lens,heads", [([5000], 2), ([1500, 1300, 1700, 1200, 1600, 1400, 1100, 1800, 1250], 8)],
                         ids=["workgroup_per_row", "workgroup_per_row_pair"])
def test_threshold_estimate_on_heavily_tied_logits(lens, heads):
    """An index whose stored keys repeat five (code, list, norm) triples: a row's sampled logits take
    five values only, the histogram of the threshold estimate cannot separate them, and its
    bit-by-bit search takes over -- in both forms of the launch, a workgroup per query row and a
    workgroup per pair of rows (288 rows).  The selection is still the exact top-k, ties to the
    lowest index, and the candidates are whole groups of equal logits."""
    dev = _cuda()
    p = Problem(lens=lens, heads=heads, groups=4, lists=32, seed=67)
    for ix in p.index.values():
        pick = np.arange(ix["codes"].shape[0]) % 5
        for name in ("codes", "list_ids", "norms"):
            ix[name] = ix[name][pick].copy()
    idx = p.device_index(dev)
    kv = ops.kv_contiguous(*p.dense_kv())
    ws = ops.DecodeWorkspace(idx, p.G, ops.resolve_topk(p.n_max, 0.05, 0))
    assert ops.decode_step_launches(idx, p.G, ws, general_path=True) == 4
    assert _check_step(p, idx, kv, ws, 0.05) >= 2                 # (tables and thresholds in one launch, and apart)
    counts = ws.candidate_counts().cpu().numpy().reshape(p.B, p.H, -1)[:, :, : p.G]
    for b in range(p.B):
        assert (counts[b] >= p.n(b) // 5).all()                   # at least the whole group of the best logit


def test_decode_step_rescans_rows_when_the_sampled_threshold_keeps_too_few():
    """A sample made of the stream's best-scoring keys puts the threshold far too high: every row
    keeps fewer than k candidates, is re-scored in full by its selection workgroup, and the
    result is still the exact top-k with the right background."""
    dev = _cuda()
    p = Problem(lens=[20000], heads=1, groups=2, lists=32, seed=29)
    idx = p.device_index(dev)
    _, _, logits = p.oracle_step(0, 0, 0.02)
    ns = int(idx.s_n[0])
    best = np.argsort(-logits.max(axis=0), kind="stable")[:ns].copy()      # retrieval-local key indices
    codes, lists, norms = idx.by_key(0, p.n(0))
    pick = torch.from_numpy(best).to(dev)
    idx.s_codes[0, :ns], idx.s_list_ids[0, :ns], idx.s_norms[0, :ns] = codes[pick], lists[pick], norms[pick]
    ws = ops.DecodeWorkspace(idx, p.G, ops.resolve_topk(p.n_max, 0.02, 0))
    before = ws.rescans()
    runs = _check_step(p, idx, ops.kv_contiguous(*p.dense_kv()), ws, 0.02)
    assert ws.rescans() - before == p.G * runs, "both rows should have taken the full re-scan"
    assert int(ws.candidate_counts()[0, : p.G].max()) < ops.resolve_topk(p.n_max, 0.02, 0)


def test_decode_step_selects_from_a_full_pass_when_candidates_outgrow_their_area():
    """An index that was never sampled makes every key a candidate: far more than the bounded
    candidate area of the workspace holds (3 k + 2048 records per row).  Such rows are selected by
    passes over the stored keys themselves; top-k and output stay those of the oracle."""
    dev = _cuda()
    p = Problem(lens=[9000, 7000], heads=1, groups=3, lists=32, seed=33)
    raw = p.device_index(dev, finalize=False)
    k_cap = ops.resolve_topk(p.n_max, 0.02, 0)
    assert p.n(1) > 3 * k_cap + 2048
    ws = ops.DecodeWorkspace(raw, p.G, k_cap)
    runs = _check_step(p, raw, ops.kv_contiguous(*p.dense_kv()), ws, 0.02)
    assert ws.rescans() == p.B * p.H * p.G * runs
    assert int(ws.candidate_counts()[:, : p.G].min()) == p.n(1)   # the scan counted every key of the shorter row


def test_decode_step_with_device_lengths_beyond_the_host_bounds_exits_normally():
    """``full_max`` and ``n_max`` size the launch on the host; the lengths the kernels read live on
    the device.  When the device-side lengths run ahead of those bounds (a host mirror one step
    behind) the kernels cut the excess off instead of writing past the areas the launch sized:
    the step completes, its output is finite, the selection among the scanned keys is intact, and
    a correctly sized step afterwards gives the oracle's result."""
    dev = _cuda()
    p = Problem(lens=[6000, 4100], heads=2, groups=3, lists=32, seed=41)
    idx = p.device_index(dev)
    kv = ops.kv_contiguous(*p.dense_kv())
    k_cap = ops.resolve_topk(p.n_max, 0.03, 0)
    ws = ops.DecodeWorkspace(idx, p.G, k_cap)
    q = p.q_tensor()
    out = torch.full_like(q, float("nan"))  # a row no workgroup folds would stay NaN
    # one row more on the device than the host sized the attention launch for
    ops.decode_step(q, out, kv, idx, p.G, p.seq_lens(), sink=p.sink, full_max=p.sink + p.local - 1, fraction=0.03,
                    topk=0, scale=SCALE, workspace=ws, general_path=True)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    tidx = ws.topk_idx.cpu().numpy().reshape(p.B, p.H, p.G, -1)
    for (b, h) in p.index:
        _, want_idx, _ = p.oracle_step(b, h, 0.03)
        for g in range(p.G):
            assert np.array_equal(np.sort(tidx[b, h, g, : want_idx.shape[1]]), np.sort(want_idx[g])), (b, h, g)
    # a scan sized for fewer keys than the device-side counts say
    for general_path in (False, True, "fused"):   # (the single-kernel form clamps the same way)
        ops.decode_step(q, out, kv, idx, p.G, p.seq_lens(), sink=p.sink, full_max=p.sink + p.local - 1, fraction=0.03,
                        topk=0, scale=SCALE, workspace=ws, **_path(general_path))
        ops.decode_step(q, out, kv, idx, p.G, p.seq_lens(), sink=p.sink, full_max=p.sink + p.local, fraction=0.03,
                        topk=0, scale=SCALE, workspace=ws, n_max=p.n_max - 1500, **_path(general_path))
        torch.cuda.synchronize()
        assert torch.isfinite(out.float()).all()
    cnt = ws.topk_cnt.cpu().numpy()
    assert (cnt >= 0).all() and (cnt <= k_cap).all()
    sel = ws.topk_idx.cpu().numpy().reshape(p.B * p.H * p.G, -1)
    for r in range(sel.shape[0]):
        assert (sel[r, : cnt.reshape(-1)[r]] >= 0).all() and (sel[r, : cnt.reshape(-1)[r]] < p.n_max).all()
    _check_step(p, idx, kv, ws, 0.03)


def test_decode_step_on_unsorted_and_partly_sorted_layouts():
    """The same step over (i) an index that was never sorted or sampled (every key is a candidate),
    (ii) a sorted prefix followed by an insertion-order tail, as after appends."""
    dev = _cuda()
    p = Problem(lens=[3000, 2100], heads=2, groups=3, lists=32, seed=31)
    kv = ops.kv_contiguous(*p.dense_kv())
    raw = p.device_index(dev, finalize=False)
    ws = ops.DecodeWorkspace(raw, p.G, ops.resolve_topk(p.n_max, 0.05, 0))
    _check_step(p, raw, kv, ws, 0.05)
    counts = [p.n(b) for b in range(p.B)]
    part = p.device_index(dev, finalize=False)
    part.set_counts([c - 700 for c in counts])     # sort and sample the first keys only ...
    part.finalize_layout()
    part.set_counts(counts)                         # ... the last 700 stay in insertion order
    assert part.tail_max() == 700
    ws2 = ops.DecodeWorkspace(part, p.G, ops.resolve_topk(p.n_max, 0.05, 0))
    _check_step(p, part, kv, ws2, 0.05)
    assert ws2.rescans() == 0


@pytest.mark.parametrize("layout", ["dense", "5d", "4d"])
def test_gather_probe_reads_the_rows_it_is_given(layout):
    """The measurement kernel behind the scattered-row ceiling reads exactly the K and V rows at the
    listed token positions (same addressing as the attention kernel, block table included): the
    XOR of its checksums equals the XOR of every 32-bit word of those rows."""
    dev = _cuda()
    p = Problem(lens=[1500, 900], heads=2, groups=2, lists=16, dtype=torch.bfloat16 if layout != "dense" else torch.float32,
                seed=43)
    kv = ops.kv_contiguous(*p.dense_kv()) if layout == "dense" else ops.kv_paged(*p.paged_kv(layout))
    gen = torch.Generator().manual_seed(7)
    count = 777
    pos = torch.stack([torch.randint(0, p.lens[bh // p.H], (count,), generator=gen) for bh in range(p.B * p.H)])
    checks = ops.gather_probe(kv, pos.to(torch.int32).to(dev))
    torch.cuda.synchronize()
    got = 0
    for x in checks.cpu().numpy().view(np.uint32):
        got ^= int(x)
    keys, values = p.dense_kv()
    want = 0
    for bh in range(p.B * p.H):
        b, h = divmod(bh, p.H)
        for t in (keys, values):
            words = t[b, h][pos[bh].to(dev)].contiguous().view(torch.int32).cpu().numpy().view(np.uint32)
            want ^= int(np.bitwise_xor.reduce(words.reshape(-1)))
    assert got == want


def test_hybrid_attend_paged_alone_matches_oracle():
    """The stand-alone attention entry point, fed the oracle's own selection and per-list masses."""
    dev = _cuda()
    p = Problem(lens=[1500, 900], heads=2, groups=2, lists=16, dtype=torch.bfloat16, seed=37)
    idx = p.device_index(dev)
    kv = ops.kv_paged(*p.paged_kv("4d"))
    frac = 0.03
    k_cap = ops.resolve_topk(p.n_max, frac, 0)
    rows = p.B * p.H * p.G
    tidx = torch.full((rows, k_cap), 0, dtype=torch.int32)
    tval = torch.zeros(rows, k_cap)
    tcnt = torch.zeros(rows, dtype=torch.int32)
    mass = torch.zeros(rows, p.L)
    rmax = torch.zeros(rows)
    want = {}
    for (b, h), ix in p.index.items():
        out, sel, logits = p.oracle_step(b, h, frac)
        want[b, h] = out
        for g in range(p.G):
            r = (b * p.H + h) * p.G + g
            k = sel.shape[1]
            tidx[r, :k] = torch.from_numpy(sel[g].astype(np.int32))
            tval[r, :k] = torch.from_numpy(logits[g, sel[g]])
            tcnt[r] = k
            rmax[r] = float(logits[g].max())
            w = np.exp(logits[g].astype(np.float64) - float(logits[g].max()))
            mass[r] = torch.from_numpy(np.bincount(ix["list_ids"].astype(np.int64), weights=w, minlength=p.L)).float()
    q = p.q_tensor().float()
    out = torch.full_like(q, float("nan"))  # a row no workgroup folds would stay NaN
    ops.hybrid_attend_paged(q, out, kv, idx, p.G, p.seq_lens(), sink=p.sink, full_max=p.sink + p.local,
                            topk_idx=tidx.to(dev), topk_val=tval.to(dev), topk_cnt=tcnt.to(dev),
                            list_mass=mass.to(dev), row_max=rmax.to(dev), scale=SCALE)
    torch.cuda.synchronize()
    o = out.cpu().numpy().reshape(p.B, p.H, p.G, DIM)
    for (b, h), w in want.items():
        assert np.abs(o[b, h] - w).max() <= 2e-3, (b, h, np.abs(o[b, h] - w).max())


@pytest.mark.parametrize("cfg", [1, 2, 3, 4])
def test_full_size_step_properties_at_the_benchmark_shapes(cfg):
    """At the full configuration sizes (cfg 1: context 32 768, one sequence; cfg 2, the headline:
    context 131 072, batch 4; cfg 3: 16 sequences of 16 384 to 65 536 tokens in shuffled blocks;
    these with 8 KV heads, GQA 4; cfg 4: context 262 144, 4 KV heads, GQA 7; all bf16 paged) the
    oracle is too slow, so the
    step is checked through properties: the selected set is exactly the k best of the logits
    pqhsa_lut_scan writes for the same tables, nothing was re-scanned, and the output equals a
    dense torch attention in which unselected stored keys are replaced by their list's mean value
    under the approximate logits."""
    import bench

    dev = _cuda()
    layer = bench.Layer(cfg, 4242, torch.device(dev))
    layer.call.run(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    idx, G, H, B = layer.index, layer.G, layer.H, layer.B
    qnorm, lut, ls = ops.lut_build(layer.q, idx, G)
    logits = ops.lut_scan(idx, G, qnorm, lut, ls, 1.0 / np.sqrt(128.0))       # [BH, G, n_cap] by key index
    for b in range(B):                                                          # sequences differ in length at cfg 3
        n = layer.n[b]
        k = ops.resolve_topk(n, bench.FRACTION, 0)
        rows = slice(b * H, (b + 1) * H)
        tidx = layer.ws.topk_idx.view(B * H, G, -1)[rows, :, :k].to(torch.int64)
        tval = layer.ws.topk_val.view(B * H, G, -1)[rows, :, :k]
        lg = logits.view(B * H, G, -1)[rows, :, :n]
        assert torch.equal(torch.gather(lg, 2, tidx), tval), b                  # the selected logits, bit for bit
        kth = torch.topk(lg, k, dim=2).values[:, :, -1:]
        assert bool((tval >= kth).all()), b                                     # none below the k-th best
        assert bool((tidx.sort(dim=2).values.diff(dim=2) > 0).all()), b        # k distinct keys
    assert layer.ws.rescans() == 0
    # reference combination in fp64 on the device for one KV head of the last sequence
    b, h = B - 1, 3
    bh = b * H + h
    sel_idx, lg_h = tidx[h], lg[h]                      # of sequence B - 1, the loop's last
    kk, vv = ops.paged_gather_range(layer.kv, b, 0, layer.lens[b])
    K, V = kk[h].double(), vv[h].double()
    del kk, vv
    q = layer.q[b, h * G : (h + 1) * G].double()
    sink = bench.SINK
    sel = torch.zeros(G, n, dtype=torch.bool, device=dev)
    sel.scatter_(1, sel_idx, True)
    exact = (q @ K.T) / np.sqrt(128.0)
    _, lists, _ = idx.by_key(bh, n)
    lists = lists.to(torch.int64) & 0xFFFF
    m = torch.maximum(exact.max(dim=1).values, lg_h.double().max(dim=1).values)[:, None]
    w_exact = torch.exp(exact - m)
    w_exact[:, sink : sink + n] *= sel                                            # unselected stored keys leave the exact part
    w_bg = torch.exp(lg_h.double() - m) * (~sel)
    mass = torch.zeros(G, idx.num_lists, dtype=torch.float64, device=dev).index_add_(1, lists, w_bg)
    num = w_exact @ V + mass @ idx.vbar[bh].double()
    den = w_exact.sum(dim=1, keepdim=True) + mass.sum(dim=1, keepdim=True)
    want = (num / den).float()
    got = layer.out[b, h * G : (h + 1) * G].float()
    err = (got - want).abs()
    assert bool((err <= 2e-3 + 2.0 ** -8 * want.abs()).all()), float(err.max())
    # the same step with fp32 queries and output (K/V stay bf16 in their pages): the stated bound as
    # it is, with no allowance for a 16-bit output's own rounding
    q32 = layer.q.float()
    out32 = torch.full_like(q32, float("nan"))
    ops.decode_step(q32, out32, layer.kv, idx, G, layer.seq_lens, sink=sink, full_max=sink + bench.LOCAL,
                    fraction=bench.FRACTION, topk=0, scale=1.0 / np.sqrt(128.0), workspace=layer.ws)
    torch.cuda.synchronize()
    err32 = (out32[b, h * G : (h + 1) * G] - want).abs()
    assert float(err32.max()) <= 2e-3, float(err32.max())
    print(f"cfg {cfg}: max |out - dense reference| {float(err.max()):.2e} (bf16 q/out), {float(err32.max()):.2e} (fp32 q/out)")


def test_append_then_scan_at_the_long_context_shape():
    """cfg 4 as the benchmark runs it: context 262 144, 4 KV heads, GQA 7, bf16 pages, and every
    step appends one key per sequence (the one leaving the local window) before it scans.  After
    each of a few fused append + decode steps: the new key's norm, list and codes are those of the
    fixed-order oracle's encode of that row, the stored-key count moved, the selection is exactly
    the k best of the logits pqhsa_lut_scan writes over the grown index, and no row was re-scanned."""
    import bench
    from oracle import fixed

    dev = _cuda()
    steps = 3
    layer = bench.Layer(4, 777, torch.device(dev), room=steps + 1)
    idx, G, H, B = layer.index, layer.G, layer.H, layer.B
    stream = torch.cuda.current_stream().cuda_stream
    coarse, books = idx.coarse.cpu().numpy(), idx.codebooks.cpu().numpy()
    for t in range(1, steps + 1):
        layer.append_step(stream)
        torch.cuda.synchronize()
        for b in range(B):
            n_new = layer.n[b] + t
            assert int(idx.n_idx[b]) == n_new and idx.n_host[b] == n_new
            tok = bench.SINK + n_new - 1                       # the key that just left the local window
            kk, _ = ops.paged_gather_range(layer.kv, b, tok, tok + 1)
            for h in range(H):
                bh = b * H + h
                norms, lids, codes = fixed.encode(kk[h].float().cpu().numpy(), coarse[bh], books[bh])
                at = n_new - 1                                # appended keys sit at the end, in insertion order
                assert int(idx.pos[bh, at]) == at
                assert u32(idx.codes[bh, at : at + 1])[0] == codes[0], (t, bh)
                assert u16(idx.list_ids[bh, at : at + 1])[0] == lids[0], (t, bh)
                assert float(idx.norms[bh, at]) == float(norms[0]), (t, bh)
        qnorm, lut, ls = ops.lut_build(layer.q, idx, G)
        logits = ops.lut_scan(idx, G, qnorm, lut, ls, 1.0 / np.sqrt(128.0))
        for b in range(B):
            n = layer.n[b] + t
            k = ops.resolve_topk(n, bench.FRACTION, 0)
            rows = slice(b * H, (b + 1) * H)
            assert bool((layer.ws.topk_cnt.view(B * H, G)[rows] == k).all())
            tidx = layer.ws.topk_idx.view(B * H, G, -1)[rows, :, :k].to(torch.int64)
            tval = layer.ws.topk_val.view(B * H, G, -1)[rows, :, :k]
            lg = logits.view(B * H, G, -1)[rows, :, :n]
            assert torch.equal(torch.gather(lg, 2, tidx), tval), (t, b)
            want = torch.topk(lg, k, dim=2)
            assert torch.equal(tval.sort(dim=2, descending=True).values, want.values), (t, b)
            assert bool((tidx.sort(dim=2).values.diff(dim=2) > 0).all()), (t, b)
    assert layer.ws.rescans() == 0


@pytest.mark.parametrize("general_path", [False, True, "fused"], ids=["short_context_kernel", "general", "general_one_launch"])
def test_decode_step_graph_replays_match_eager_runs(general_path):
    """The step recorded into a HIP graph and replayed several times, with eager work and
    synchronisations between the replays: every replay gives the oracle's top-k sets and its
    outputs within 2e-3 for the query of that round, and what the eager step gives."""
    dev = _cuda()
    p = Problem(lens=[2600, 1900], heads=2, groups=4, lists=32, dtype=torch.bfloat16, seed=43)
    idx = p.device_index(dev)
    kv = ops.kv_paged(*p.paged_kv("5d"))
    q = p.q_tensor().float()
    out = torch.full_like(q, float("nan"))  # a row no workgroup folds would stay NaN
    ws = ops.DecodeWorkspace(idx, p.G, ops.resolve_topk(p.n_max, 0.03, 0))
    call = ops.DecodeCall(q, out, kv, idx, p.G, p.seq_lens(), sink=p.sink, full_max=p.sink + p.local,
                          fraction=0.03, topk=0, scale=SCALE, workspace=ws, **_path(general_path))
    call.capture()
    gen = torch.Generator(device="cpu").manual_seed(5)
    base = q.clone()
    for round_ in range(4):
        q.copy_((base + 0.3 * round_ * torch.randn(base.shape, generator=gen).to(dev)).to(p.dtype).float())
        call.run()
        torch.cuda.synchronize()
        want_out, want_idx = out.clone(), ws.topk_idx.clone().sort(dim=1).values
        out.fill_(float("nan"))
        ws.topk_idx.fill_(-1)
        junk = (torch.randn(512, 512, device=dev) @ torch.randn(512, 512, device=dev)).sum()   # unrelated eager work
        torch.cuda.synchronize()
        call.replay()
        torch.cuda.synchronize()
        assert torch.equal(ws.topk_idx.sort(dim=1).values, want_idx), round_
        np.testing.assert_allclose(out.cpu().numpy(), want_out.cpu().numpy(), atol=1e-5, err_msg=str(round_))
        assert torch.isfinite(junk)
        # ... and the replay against the fixed-order oracle on this pass's query
        qh = q.cpu().numpy().reshape(p.B, p.H, p.G, DIM)
        got_out = out.cpu().numpy().reshape(p.B, p.H, p.G, DIM)
        got_idx = ws.topk_idx.cpu().numpy().reshape(p.B, p.H, p.G, -1)
        for (b, h), ix in p.index.items():
            o_out, o_idx, _ = fixed.decode_step(qh[b, h], p.keys[b, h].numpy(), p.values[b, h].numpy(), ix, sink=p.sink,
                                                local=p.local, fraction=0.03, scale=SCALE)
            for g in range(p.G):
                assert np.array_equal(np.sort(got_idx[b, h, g, : o_idx.shape[1]]), np.sort(o_idx[g])), (round_, b, h, g)
            assert float(np.abs(got_out[b, h] - o_out).max()) <= 2e-3, (round_, b, h)


@pytest.mark.parametrize("lens, heads", [
    ([9000, 2100, 5200, 400], 2),                                   # packed launch: tiles with work first
    ([300 + (977 * i) % 2100 for i in range(66)], 1),               # over 64 sequences: tile-major launch
], ids=["packed", "tile_major"])
def test_ragged_batch_tile_hint_changes_no_result(lens, heads):
    """The mean-length hint only sizes the scan's tiles (a ragged batch is then launched with the
    tiles that hold work ahead of the empty ones, which leave at once): whatever it says, the
    top-k set is the oracle's and the outputs agree."""
    dev = _cuda()
    p = Problem(lens=lens, heads=heads, groups=4, lists=32, dtype=torch.bfloat16, seed=71)
    idx = p.device_index(dev)
    kv = ops.kv_paged(*p.paged_kv("5d"))
    q = p.q_tensor().float()
    k_cap = ops.resolve_topk(p.n_max, 0.03, 0)
    ws = ops.DecodeWorkspace(idx, p.G, k_cap)
    want = {(b, h): p.oracle_step(b, h, 0.03)[1] for (b, h) in p.index}
    first = None
    for hint in (None, 0, 1, 300, p.n_max, 10 ** 9):
        out = torch.full_like(q, float("nan"))  # a row no workgroup folds would stay NaN
        ws.topk_idx.fill_(-1)
        ops.decode_step(q, out, kv, idx, p.G, p.seq_lens(), sink=p.sink, full_max=p.sink + p.local, fraction=0.03,
                        topk=0, scale=SCALE, workspace=ws, general_path=True, n_mean=hint)
        torch.cuda.synchronize()
        tidx = ws.topk_idx.cpu().numpy().reshape(p.B, p.H, p.G, -1)
        for (b, h), want_idx in want.items():
            for g in range(p.G):
                assert np.array_equal(np.sort(tidx[b, h, g, : want_idx.shape[1]]), np.sort(want_idx[g])), (hint, b, h, g)
        if first is None:
            first = out.clone()
        np.testing.assert_allclose(out.cpu().numpy(), first.cpu().numpy(), atol=2e-6, rtol=1e-5, err_msg=str(hint))
    assert ws.rescans() == 0


@pytest.mark.parametrize("shape", [
    dict(steps=5, lens=[1805, 1505], heads=2, groups=4, lists=32, every=1),
    # 64 streams x 13 table blocks: the table-building launch gives a block two tiles of lists, and the
    # appended key's nearest list is found over the tiles' answers (a sample of the streams is checked)
    dict(steps=2, lens=[862, 852, 847, 842, 872, 882, 843, 854], heads=8, groups=2, lists=768, every=9),
    # the same steps with the tables and the threshold estimate as two launches (the appended key's
    # nearest list is then found by the table kernel's list blocks, as for "many_streams")
    dict(steps=5, lens=[1805, 1505], heads=2, groups=4, lists=32, every=1, apart=True),
    # streams that do not fill a round of eight, a padded group, lists that end inside a staged half
    dict(steps=3, lens=[1405, 1205, 1100], heads=3, groups=7, lists=300, every=2),
    # the steps after the first replayed from ONE HIP graph, captured with the launch shapes of the
    # final length: sequence lengths, key counts and the new keys are all read from device memory
    dict(steps=5, lens=[1805, 1505], heads=2, groups=4, lists=32, every=1, graph=True),
    # more than 256 query rows: two rows of a stream per workgroup, and the appending workgroups beside them
    dict(steps=2, lens=[862, 852, 847, 842, 872, 882, 843, 854, 866], heads=8, groups=4, lists=64, every=7),
], ids=["small", "many_streams", "small_two_launches", "ragged_groups", "graph_replay", "row_pairs"])
def test_fused_append_decode_steps_match_oracle_and_separate_append(shape):
    """pqhsa_append_decode_step over several steps: each step encodes the sequence's next key in
    the launch that builds the tables, attends over the grown index, and leaves the new count in
    device memory.  Checked against the oracle on the same prefix of the context."""
    dev = _cuda()
    steps = shape["steps"]
    p = Problem(lens=shape["lens"], heads=shape["heads"], groups=shape["groups"], lists=shape["lists"],
                dtype=torch.bfloat16, seed=47)
    lens0 = [ln - steps for ln in p.lens]
    n0 = [p.n(b) - steps for b in range(p.B)]
    kv = ops.kv_paged(*p.paged_kv("5d"))
    idx = p.device_index(dev, finalize=False)          # every key's codes are there, only the first n0 count
    idx.set_counts(n0)
    ops.value_summaries(kv, idx, p.sink)
    idx.finalize_layout()
    frac = 0.04
    ws = ops.DecodeWorkspace(idx, p.G, ops.resolve_topk(p.n_max, frac, 0))
    q = p.q_tensor().float()
    out = torch.full_like(q, float("nan"))  # a row no workgroup folds would stay NaN
    one = torch.ones(p.B, dtype=torch.int32, device=dev)
    seq = torch.tensor(lens0, dtype=torch.int32, device=dev)
    call = ops.DecodeCall(q, out, kv, idx, p.G, seq, sink=p.sink, full_max=p.sink + p.local, fraction=frac, topk=0,
                          scale=SCALE, workspace=ws, append_count=one, separate_tables=shape.get("apart", False))
    want_launches = 5 if shape.get("apart") or shape["lists"] > 512 else 4
    assert ops.decode_step_launches(idx, p.G, ws, appending=True, separate_tables=shape.get("apart", False)) == want_launches
    for t in range(1, steps + 1):
        seq.add_(1)
        if shape.get("graph"):
            if t == 1:
                call.n_max = max(n0) + steps     # the launch shapes of every later step
                call.run()                       # (eager: loads the kernels; its append is step 1)
            else:
                if t == 2:
                    call.capture(warm=False)     # records a step, runs nothing
                out.fill_(float("nan"))
                ws.topk_idx.fill_(-1)
                call.replay()
        else:
            call.n_max = max(n0) + t
            call.run()
        idx.note_appended([1] * p.B)
        torch.cuda.synchronize()
        assert idx.n_idx.cpu().tolist() == [n + t for n in n0]          # the step advanced the device-side counts
        tidx = ws.topk_idx.cpu().numpy().reshape(p.B, p.H, p.G, -1)
        o = out.cpu().numpy().reshape(p.B, p.H, p.G, DIM)
        for (b, h), ix in p.index.items():
            n, ln = n0[b] + t, lens0[b] + t
            bh = b * p.H + h
            codes, lists, norms = idx.by_key(bh, n)
            assert np.array_equal(u32(codes), ix["codes"][:n]) and np.array_equal(u16(lists), ix["list_ids"][:n])
            assert np.array_equal(norms.cpu().numpy(), ix["norms"][:n])
            if bh % shape["every"]:
                continue
            _, _, vbar = fixed.value_summaries(p.values[b, h][p.sink : p.sink + n].numpy(), ix["list_ids"][:n], p.L)
            np.testing.assert_allclose(idx.vbar[bh].cpu().numpy(), vbar, rtol=1e-6, atol=1e-6)
            part = {"coarse": ix["coarse"], "codebooks": ix["codebooks"], "codes": ix["codes"][:n],
                    "list_ids": ix["list_ids"][:n], "norms": ix["norms"][:n], "vbar": vbar}
            want_out, want_idx, _ = fixed.decode_step(p.queries[b, h].numpy(), p.keys[b, h][:ln].numpy(),
                                                      p.values[b, h][:ln].numpy(), part, sink=p.sink, local=p.local,
                                                      fraction=frac, scale=SCALE)
            for g in range(p.G):
                assert np.array_equal(np.sort(tidx[b, h, g, : want_idx.shape[1]]), np.sort(want_idx[g])), (t, b, h, g)
            assert np.abs(o[b, h] - want_out).max() <= 2e-3, (t, b, h)
    assert idx.tail_max() == steps and ws.rescans() == 0


def test_device_counts_ahead_of_the_host_stay_inside_k_cap():
    """If the device-side key count has moved past what the caller sized k_cap and n_max for (an
    append the host has not accounted for yet), the step selects k_cap keys instead of reading or
    writing past the top-k arrays."""
    dev = _cuda()
    p = Problem(lens=[3000], heads=1, groups=2, lists=16, seed=53)
    idx = p.device_index(dev)
    n = p.n(0)
    small = n - 400
    k_cap = ops.resolve_topk(small, 0.05, 0)                 # sized for fewer keys than the device holds
    assert ops.resolve_topk(n, 0.05, 0) > k_cap
    ws = ops.DecodeWorkspace(idx, p.G, k_cap)
    q = p.q_tensor()
    out = torch.full_like(q, float("nan"))  # a row no workgroup folds would stay NaN
    for general_path in (False, True, "fused"):
        ws.topk_cnt.zero_()
        ops.decode_step(q, out, ops.kv_contiguous(*p.dense_kv()), idx, p.G, p.seq_lens(), sink=p.sink,
                        full_max=p.sink + p.local, fraction=0.05, topk=0, scale=SCALE, workspace=ws, n_max=small,
                        **_path(general_path))
        torch.cuda.synchronize()
        assert ws.topk_cnt.cpu().tolist() == [k_cap] * p.G
        got = ws.topk_idx.cpu().numpy()
        assert ((got >= 0) & (got < n)).all() and bool(torch.isfinite(out).all())


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_decode_step_random_shapes_match_oracle(seed):
    """A seeded sweep over batch sizes, ragged lengths, group widths, list counts, dtypes, page
    layouts, selection fractions and sorted / insertion-order layouts: top-k sets bit-exact,
    outputs within the stated bound (plus the output's own rounding for 16-bit queries)."""
    import random

    dev = _cuda()
    rng = random.Random(seed)
    for case in range(6):
        lens = [rng.randint(300, rng.choice([3000, 12000, 30000])) for _ in range(rng.choice([1, 2, 3]))]
        heads, groups = rng.choice([1, 2]), rng.choice([1, 2, 3, 4, 5, 7, 8])
        lists = rng.choice([16, 32, 64, 128])
        dtype = rng.choice([torch.float32, torch.bfloat16, torch.float16])
        fraction = rng.choice([0.01, 0.02, 0.05, 0.1, 0.3])
        layout = rng.choice(["dense", "5d", "4d"])
        finalize = rng.random() < 0.75
        what = (seed, case, lens, heads, groups, lists, dtype, fraction, layout, finalize)
        p = Problem(lens=lens, heads=heads, groups=groups, lists=lists, dtype=dtype, seed=500 + 10 * seed + case)
        idx = p.device_index(dev, finalize=finalize)
        kv = ops.kv_contiguous(*p.dense_kv()) if layout == "dense" else ops.kv_paged(*p.paged_kv(layout))
        ws = ops.DecodeWorkspace(idx, p.G, ops.resolve_topk(p.n_max, fraction, 0))
        q = p.q_tensor()
        out = torch.full_like(q, float("nan"))  # a row no workgroup folds would stay NaN
        # the single kernel for short contexts where the shape fits it, or the general path in either form
        general_path = rng.choice([False, False, True, "fused"])
        what = what + (general_path,)
        ops.decode_step(q, out, kv, idx, p.G, p.seq_lens(), sink=p.sink, full_max=p.sink + p.local,
                        fraction=fraction, topk=0, scale=SCALE, workspace=ws, **_path(general_path))
        torch.cuda.synchronize()
        tidx = ws.topk_idx.cpu().numpy().reshape(p.B, p.H, p.G, -1)
        o = out.float().cpu().numpy().reshape(p.B, p.H, p.G, DIM)
        tol = 1e-4 if dtype == torch.float32 else 2e-3
        rel = {torch.float32: 0.0, torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[dtype]
        for (b, h) in p.index:
            want_out, want_idx, _ = p.oracle_step(b, h, fraction)
            k = want_idx.shape[1]
            for g in range(p.G):
                assert np.array_equal(np.sort(tidx[b, h, g, :k]), np.sort(want_idx[g])), (what, b, h, g)
            assert (np.abs(o[b, h] - want_out) <= tol + rel * np.abs(want_out)).all(), (what, b, h)
        if finalize and general_path:  # (an index that was never sampled makes every key a candidate: long rows then take the full pass)
            assert ws.rescans() == 0, what


def test_decode_step_batch_of_more_than_256_query_rows():
    """288 query rows (9 sequences x 8 KV heads x 4): the selection kernel then runs in the form
    that shares a compute unit between two workgroups, the launch that builds the tables and
    estimates the thresholds gives a workgroup two rows of a stream, and the short-context kernel
    does not apply.  A sample of the streams against the oracle, all rows for sane counts."""
    dev = _cuda()
    lens = [2400, 1300, 1900, 2100, 900, 1700, 2300, 1100, 1500]
    p = Problem(lens=lens, heads=8, groups=4, lists=32, dtype=torch.bfloat16, seed=83)
    idx = p.device_index(dev)
    kv = ops.kv_paged(*p.paged_kv("5d"))
    ws = ops.DecodeWorkspace(idx, p.G, ops.resolve_topk(p.n_max, 0.04, 0))
    q = p.q_tensor().float()
    out = torch.full_like(q, float("nan"))  # a row no workgroup folds would stay NaN
    ops.decode_step(q, out, kv, idx, p.G, p.seq_lens(), sink=p.sink, full_max=p.sink + p.local, fraction=0.04,
                    topk=0, scale=SCALE, workspace=ws)
    torch.cuda.synchronize()
    assert ops.decode_step_launches(idx, p.G, ws) == 4
    tidx = ws.topk_idx.cpu().numpy().reshape(p.B, p.H, p.G, -1)
    cnt = ws.topk_cnt.cpu().numpy().reshape(p.B, p.H, p.G)
    o = out.cpu().numpy().reshape(p.B, p.H, p.G, DIM)
    for b in range(p.B):
        assert (cnt[b] == ops.resolve_topk(p.n(b), 0.04, 0)).all(), b
    for i, (b, h) in enumerate(p.index):
        if i % 7:
            continue
        want_out, want_idx, _ = p.oracle_step(b, h, 0.04)
        for g in range(p.G):
            assert np.array_equal(np.sort(tidx[b, h, g, : want_idx.shape[1]]), np.sort(want_idx[g])), (b, h, g)
        assert np.abs(o[b, h] - want_out).max() <= 2e-3, (b, h)
    assert ws.rescans() == 0


@pytest.mark.parametrize("general_path", [False, True, "fused"], ids=["short_context_kernel", "general", "general_one_launch"])
@pytest.mark.parametrize("groups,lists,lens", [(16, 64, [2600]), (12, 256, [5000, 1700]), (9, 512, [7000])])
def test_decode_step_wide_groups_and_many_lists(groups, lists, lens, general_path):
    """Query groups of 9 to 16 rows (padded to 16 in the kernels) and list counts up to the
    headline configuration's 512, against the oracle."""
    dev = _cuda()
    p = Problem(lens=lens, heads=1, groups=groups, lists=lists, dtype=torch.bfloat16, seed=61)
    idx = p.device_index(dev)
    kv = ops.kv_paged(*p.paged_kv("5d"))
    ws = ops.DecodeWorkspace(idx, p.G, ops.resolve_topk(p.n_max, 0.05, 0))
    q = p.q_tensor().float()
    out = torch.full_like(q, float("nan"))  # a row no workgroup folds would stay NaN
    ops.decode_step(q, out, kv, idx, p.G, p.seq_lens(), sink=p.sink, full_max=p.sink + p.local, fraction=0.05,
                    topk=0, scale=SCALE, workspace=ws, **_path(general_path))
    torch.cuda.synchronize()
    tidx = ws.topk_idx.cpu().numpy().reshape(p.B, p.H, p.G, -1)
    o = out.cpu().numpy().reshape(p.B, p.H, p.G, DIM)
    for (b, h) in p.index:
        want_out, want_idx, _ = p.oracle_step(b, h, 0.05)
        k = want_idx.shape[1]
        for g in range(p.G):
            assert np.array_equal(np.sort(tidx[b, h, g, :k]), np.sort(want_idx[g])), (b, h, g)
        assert np.abs(o[b, h] - want_out).max() <= 2e-3, (b, h)


def test_topk_radix_on_tie_heavy_matrices():
    """Logit matrices made to stress the selection's tie handling: quantised values (long runs of
    equal logits on both sides of the k boundary), a handful of distinct values with both zeros,
    constants, denormal-range values; k from 0 to n.  The index set must be the oracle's."""
    dev = _cuda()
    rng = np.random.default_rng(23)
    for case, kind in enumerate(["quant1", "quant2", "few", "const", "mixed", "tiny", "quant1", "few"]):
        rows, stride = int(rng.integers(2, 7)), int(rng.choice([300, 5000, 30000]))
        x = rng.standard_normal((rows, stride)).astype(np.float32)
        if kind == "quant1":
            x = np.round(x, 1)
        elif kind == "quant2":
            x = np.round(x * 3) / 3
        elif kind == "few":
            x = rng.choice(np.array([-1.5, 0.0, -0.0, 2.25, 7.0], dtype=np.float32), size=(rows, stride))
        elif kind == "const":
            x[:] = 0.125
        elif kind == "mixed":
            x[:, ::3], x[:, 1::7] = np.float32(1.0), np.float32(-0.0)
        elif kind == "tiny":
            x *= np.float32(1e-30)
        n = [int(rng.integers(1, stride + 1)) for _ in range(rows)]
        k = [int(min(n[r], rng.choice([0, 1, 17, n[r] // 50 + 1, n[r] // 3 + 1, n[r]]))) for r in range(rows)]
        idx, val = ops.topk_radix(torch.from_numpy(x).to(dev), n, k)
        torch.cuda.synchronize()
        idx, val = idx.cpu().numpy(), val.cpu().numpy()
        for r in range(rows):
            want_idx, _ = fixed.topk(x[r, : n[r]], k[r])
            got = idx[r, : k[r]]
            assert np.array_equal(np.sort(got), np.sort(want_idx)), (case, kind, r, n[r], k[r])
            assert np.array_equal(val[r, : k[r]], x[r, got]), (case, kind, r)


def test_topk_radix_many_candidates_selected_from_memory():
    """More than 16 384 candidates per row (large k, or a k-th value shared by most of the row) are
    selected by passes over the candidates in memory: a 1024-way range split per pass, on the keys
    and then on the indices of the keys that tie.  Rows cover the whole float range (several
    splits), infinities, two-valued and constant rows (every candidate ties)."""
    dev = _cuda()
    rng = np.random.default_rng(29)
    stride = 70000
    wide = rng.integers(0, 2 ** 32, size=stride, dtype=np.uint64).astype(np.uint32).view(np.float32).copy()
    wide[np.isnan(wide)] = 0.0
    rows = [
        (np.full(stride, 0.125, np.float32), stride, 2000),                      # all equal: indices 0..k-1
        (np.full(stride, -np.inf, np.float32), 65537, 40000),
        (rng.choice(np.array([1.0, 2.0], np.float32), size=stride), stride, 50000),   # boundary inside the 1.0 ties
        (rng.standard_normal(stride).astype(np.float32), stride, stride // 3),
        (rng.standard_normal(stride).astype(np.float32), 60001, 60001),          # k = n
        (wide, stride, 30000),                                                    # bit patterns over the whole range
        (np.round(rng.standard_normal(stride), 1).astype(np.float32), stride, 35000),
        (np.where(rng.random(stride) < 0.9, np.float32(3.0), rng.standard_normal(stride).astype(np.float32)).astype(np.float32),
         stride, 100),                                                            # small k, k-th value shared by 90 % of the row
    ]
    # special values order by their bit patterns, as in the oracle: NaN above +inf, -inf lowest
    special = rng.standard_normal(stride).astype(np.float32)
    u = rng.random(stride)
    special[u < 0.05], special[(u >= 0.05) & (u < 0.10)], special[u > 0.80] = np.nan, np.inf, -np.inf
    rows += [(special, stride, 2000), (special, stride, 9000), (special, 69999, 60000)]
    x = np.stack([r[0] for r in rows])
    n, k = [r[1] for r in rows], [r[2] for r in rows]
    idx, val = ops.topk_radix(torch.from_numpy(x).to(dev), n, k)
    torch.cuda.synchronize()
    idx, val = idx.cpu().numpy(), val.cpu().numpy()
    for r in range(len(rows)):
        want_idx, _ = fixed.topk(x[r, : n[r]], k[r])
        got = idx[r, : k[r]]
        assert np.array_equal(np.sort(got), np.sort(want_idx)), (r, n[r], k[r])
        assert np.array_equal(val[r, : k[r]], x[r, got], equal_nan=True), r


TABLES_CASES = [
    # query rows of a padded group, list counts that end inside a tile / a phase, streams that do not fill a round of 8
    dict(lens=[20000], heads=2, groups=3, lists=64, dtype=torch.bfloat16),
    dict(lens=[17000, 9000, 30000], heads=3, groups=1, lists=200, dtype=torch.float16),
    dict(lens=[18000], heads=1, groups=7, lists=300, dtype=torch.float32),
    dict(lens=[17000, 17500], heads=4, groups=4, lists=512, dtype=torch.bfloat16),
    dict(lens=[20000], heads=1, groups=16, lists=16, dtype=torch.bfloat16),
    dict(lens=[2000, 700, 60, 1500], heads=2, groups=2, lists=40, dtype=torch.float32),   # (one sequence without indexed keys)
    # room for 170 000 keys per sequence: a sample of more than 4 096 keys per stream, eight per thread
    dict(lens=[20000, 12000], heads=1, groups=4, lists=128, dtype=torch.bfloat16, spare=150000),
    # more than 256 query rows: a workgroup takes two rows of a stream (whole groups, a group padded
    # from 7 to 8 rows whose last pair holds one row, a group of 3 whose last pair holds one)
    dict(lens=[2500, 1800, 2100, 900, 2300, 1500, 2600, 1200, 2000], heads=8, groups=4, lists=64, dtype=torch.bfloat16),
    dict(lens=[2400, 1700, 2900, 1300, 2000], heads=8, groups=7, lists=300, dtype=torch.float32),
    dict(lens=[2500, 1800, 2100, 900, 2300, 1500, 2600, 1200, 2000], heads=8, groups=3, lists=512, dtype=torch.float16),
]


@pytest.mark.parametrize("case", TABLES_CASES, ids=[str(i) for i in range(len(TABLES_CASES))])
def test_tables_and_thresholds_in_one_launch_match_the_two_launches(case):
    """A step without an append builds each query row's tables inside the row's threshold
    workgroup (four launches); the same step with the two kept apart (five) must leave the same
    tables and thresholds to the bit -- seen through the number of candidates every row's scan
    keeps -- and both must agree with the oracle."""
    dev = _cuda()
    p = Problem(lens=case["lens"], heads=case["heads"], groups=case["groups"], lists=case["lists"],
                dtype=case["dtype"], seed=131)
    idx = p.device_index(dev, spare=case.get("spare", 64))
    if "spare" in case:
        assert 4096 < idx.s_cap <= 8192
    kv = ops.kv_contiguous(*p.dense_kv())
    ws = ops.DecodeWorkspace(idx, p.G, ops.resolve_topk(p.n_max, 0.03, 0))
    assert ops.decode_step_launches(idx, p.G, ws, general_path=True) == 4
    assert ops.decode_step_launches(idx, p.G, ws, general_path=True, separate_tables=True) == 5
    q = p.q_tensor()
    # (the output has the query's type: half an ulp of it on top of the arithmetic's own tolerance)
    half_ulp = {torch.float32: 0.0, torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[case["dtype"]]
    tol = 1e-4 if case["dtype"] == torch.float32 else 2e-3
    seen = {}
    for apart in (True, False, False):
        out = torch.full_like(q, float("nan"))
        ws.topk_idx.fill_(-1)
        ws.topk_cnt.fill_(-1)
        ops.decode_step(q, out, kv, idx, p.G, p.seq_lens(), sink=p.sink, full_max=p.sink + p.local, fraction=0.03,
                        topk=0, scale=SCALE, workspace=ws, general_path=True, separate_tables=apart)
        torch.cuda.synchronize()
        counts = ws.candidate_counts().cpu().numpy().copy()
        tidx = ws.topk_idx.cpu().numpy().reshape(p.B, p.H, p.G, -1)
        o = out.float().cpu().numpy().reshape(p.B, p.H, p.G, DIM)
        if apart:
            seen = dict(counts=counts, out=o)
        else:
            assert np.array_equal(counts, seen["counts"])
            assert bool((np.abs(o - seen["out"]) <= 1e-5 + 2.0 * half_ulp * np.abs(o)).all())
        for (b, h) in p.index:
            if p.n(b) == 0:
                continue
            want_out, want_idx, _ = p.oracle_step(b, h, 0.03)
            k = want_idx.shape[1]
            for g in range(p.G):
                assert np.array_equal(np.sort(tidx[b, h, g, :k]), np.sort(want_idx[g])), (apart, b, h, g)
            assert bool((np.abs(o[b, h] - want_out) <= tol + half_ulp * np.abs(want_out)).all()), (apart, b, h)


def test_event_log_counts_steps_and_samples_them():
    """The per-kernel event log of the decode step: every step logged, one kernel only, and one
    step in three; the number of logged steps and which kernels carry a time."""
    import ctypes
    from pqhsa_release_amd import _lib

    dev = _cuda()
    lib = _lib.load()
    p = Problem(lens=[3000], heads=2, groups=4, lists=32, dtype=torch.bfloat16, seed=61)
    idx = p.device_index(dev)
    kv = ops.kv_paged(*p.paged_kv("5d"))
    ws = ops.DecodeWorkspace(idx, p.G, ops.resolve_topk(p.n_max, 0.02, 0))
    q = p.q_tensor()
    out = torch.full_like(q, float("nan"))  # a row no workgroup folds would stay NaN

    def steps(count, separate_tables=True):
        for _ in range(count):
            ops.decode_step(q, out, kv, idx, p.G, p.seq_lens(), sink=p.sink, full_max=p.sink + p.local,
                            fraction=0.02, topk=0, scale=SCALE, workspace=ws, general_path=True,
                            separate_tables=separate_tables)

    def collect():
        kms = (ctypes.c_float * 5)()
        seen = ctypes.c_int32(-1)
        _lib.check(lib.pqhsa_profile_collect(kms, ctypes.byref(seen)), "pqhsa_profile_collect")
        return seen.value, [float(v) for v in kms]

    _lib.check(lib.pqhsa_profile_enable(16), "enable")
    steps(5)
    seen, kms = collect()
    assert seen == 5 and all(0.0 < v < 50.0 for v in kms), (seen, kms)
    assert ops.decode_step_launches(idx, p.G, ws, general_path=True) == 4
    _lib.check(lib.pqhsa_profile_enable(16), "enable")
    steps(4, separate_tables=False)                # tables and thresholds in one launch: booked under the first slot
    seen, merged = collect()
    assert seen == 4 and all(0.0 < v < 50.0 for i, v in enumerate(merged) if i != 1), (seen, merged)
    assert 0.0 <= merged[1] < 50.0, (merged, kms)     # (an empty slot: the cost of recording an event)
    _lib.check(lib.pqhsa_profile_enable(16), "enable")
    _lib.check(lib.pqhsa_profile_only(4), "only")
    _lib.check(lib.pqhsa_profile_every(3), "every")
    steps(7)                                       # steps 0, 3 and 6 are logged
    seen, kms = collect()
    assert seen == 3 and kms[4] > 0.0 and all(v == 0.0 for i, v in enumerate(kms) if i != 4), (seen, kms)
    steps(2)                                       # the log is off again: nothing recorded, nothing to collect
    assert lib.pqhsa_profile_every(0) != 0 and b"stride" in lib.pqhsa_last_error()



def test_fold_of_sixty_four_partials_per_row_over_hundreds_of_launches():
    """The hand-over between the workgroups of a query row in the exact attention: every workgroup
    writes its partial result and a flag, and the one that finds all flags set folds the partials.
    Here each of 512 query rows (16 ragged sequences, 8 KV heads, groups of 4) attends over up to
    24 388 rows, which the launch cuts into the largest number of chunks it uses, 64 per query row
    (32 768 workgroups per launch; short sequences leave some of their chunks empty).  The stand-alone
    entry point is launched 300 times on one selection: every output must equal the first bit for
    bit (the fold adds the partials in chunk order whichever workgroup does it, so a partial read
    before it was complete, or a row folded twice or not at all, shows), and the first must equal a
    dense fp32 attention over the same rows."""
    import bench

    dev = _cuda()
    layer = bench.Layer(3, 977, torch.device(dev))
    B, H, G = layer.B, layer.H, layer.G
    rows = B * H * G
    k_cap = 24320
    full_max = bench.SINK + bench.LOCAL
    assert rows == 512 and (full_max + k_cap + 383) // 384 == 64
    gen = torch.Generator(device=dev).manual_seed(5)
    tidx = torch.zeros(rows, k_cap, dtype=torch.int32, device=dev)
    tcnt = torch.zeros(rows, dtype=torch.int32, device=dev)
    for b in range(B):
        n_b = layer.n[b]
        cnt = min(n_b, k_cap)
        for hg in range(H * G):
            r = b * H * G + hg
            tidx[r, :cnt] = torch.randperm(n_b, generator=gen, device=dev)[:cnt].to(torch.int32)
            tcnt[r] = cnt
    # no background: per-list masses of zero, and selected logits so low that nothing is taken off them
    tval = torch.full((rows, k_cap), -1e30, device=dev)
    mass = torch.zeros(rows, bench.LISTS, device=dev)
    rmax = torch.zeros(rows, device=dev)
    q = layer.q.float()
    scale = 1.0 / np.sqrt(128.0)

    def launch():
        out = torch.full_like(q, float("nan"))  # a row no workgroup folds would stay NaN
        ops.hybrid_attend_paged(q, out, layer.kv, layer.index, G, layer.seq_lens, sink=bench.SINK, full_max=full_max,
                                topk_idx=tidx, topk_val=tval, topk_cnt=tcnt, list_mass=mass, row_max=rmax, scale=scale)
        torch.cuda.synchronize()
        return out

    first = launch()
    assert bool(torch.isfinite(first).all())
    # dense attention over the same rows, for the shortest and the longest sequence and two more
    order = sorted(range(B), key=lambda b: layer.lens[b])
    for b in (order[0], order[-1], order[B // 2], order[1]):
        ln = layer.lens[b]
        for h, g in ((0, 0), (H - 1, G - 1), (3, 1)):
            r = (b * H + h) * G + g
            cnt = int(tcnt[r])
            pos = torch.cat([torch.arange(bench.SINK, device=dev), torch.arange(ln - bench.LOCAL, ln, device=dev),
                             bench.SINK + tidx[r, :cnt].long()])
            assert len(set(pos.tolist())) == pos.numel()
            keys, values = ops.paged_gather_at(layer.kv, b, pos.unsqueeze(0).expand(H, -1).contiguous())
            w = torch.softmax((keys[h].float() @ q[b, h * G + g]) * scale, dim=0)
            want = w @ values[h].float()
            err = float((first[b, h * G + g] - want).abs().max())
            assert err <= 2e-3, (b, h, g, err)
    for rep in range(300):
        again = launch()
        assert torch.equal(again, first), (rep, float((again - first).abs().max()))


def test_candidate_records_of_an_index_with_more_than_a_million_slots_per_sequence():
    """A candidate record names its key by stored position in 20 bits of one word; an index whose
    sequences have room for more than 2^20 keys keeps the records of (logit, retrieval-local index)
    with the list ids in a second array, read with the position map in the scan and selected without
    a look-up.  Same step, same oracle; the dense windows of the needle queries exercise the rows
    that write straight to memory in that form too."""
    dev = _cuda()
    p = Problem(lens=[20000, 9000], heads=2, groups=4, lists=32, seed=47)
    idx = p.device_index(dev, spare=(1 << 20))
    assert idx.n_cap > (1 << 20)
    kv = ops.kv_contiguous(*p.dense_kv())
    ws = ops.DecodeWorkspace(idx, p.G, ops.resolve_topk(p.n_max, 0.03, 0))
    assert ops.decode_step_launches(idx, p.G, ws, general_path=True, one_launch=True) == 5   # (no one-launch form either, and too large a sample for tables and thresholds in one launch)
    before = ws.rescans()
    assert _check_step(p, idx, kv, ws, 0.03) == 1
    assert ws.rescans() == before
