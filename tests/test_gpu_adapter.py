"""GPU tests of the drop-in boundary: adapters, sidecar and the vLLM decode hook, end to end
through the C ABI, against vectors recorded from the real reference (tests/golden/*.npz) and
against the fixed-order oracle run on the engine's own trained index."""

import math
import os
import types

import numpy as np
import pytest
import torch

from oracle import fixed
from oracle import torch_ref as tr
from tests.gpu_util import u16, u32

pytestmark = pytest.mark.gpu

DIM = 128
SCALE = 1.0 / math.sqrt(DIM)


def _cuda():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    return torch.device("cuda")


def _cfgs(lists, fraction, *, sink=4, local=64, strategy="incremental", interval=1):
    from pqhsa_release_amd.config import IVFPQConfig, SparseAttentionConfig

    ic = IVFPQConfig(num_lists=lists, nprobe=8, num_subspaces=8, num_bits=4, residual=True, coarse_max_iter=1,
                     pq_max_iter=2, kernel_backend="mi355x", direction_normalize=True, seed=0)
    ac = SparseAttentionConfig(sink_tokens=sink, local_window=local, retrieval_top_fraction=fraction,
                               exact_rerank=True, mode="hybrid", hybrid_value_mode="centroid",
                               index_update_interval=interval, index_update_strategy=strategy,
                               collect_attention_details=False)
    return ic, ac


def _load(golden_dir, name):
    fx = np.load(os.path.join(golden_dir, f"{name}.npz"))
    m = dict(zip(["ctx", "heads", "groups", "lists", "steps", "sink", "local"], (int(x) for x in fx["meta"])))
    m["fraction"] = float(fx["fraction"][0])
    return fx, m


def _words(packed_np):
    return tr.packed_to_words(torch.from_numpy(packed_np)).numpy().astype(np.uint32)


def _index_of(engine, bh, n):
    """Download one stream's index in the oracle's format."""
    idx = engine.index
    codes, lists, norms = idx.by_key(bh, n)          # stored list-sorted; the oracle wants key order
    return {"coarse": idx.coarse[bh].cpu().numpy(), "codebooks": idx.codebooks[bh].cpu().numpy(),
            "codes": u32(codes), "list_ids": u16(lists), "norms": norms.cpu().numpy(),
            "vbar": idx.vbar[bh].cpu().numpy()}


def _margin_ok(logits, got_idx, ref_idx):
    for g in range(logits.shape[0]):
        a, b = set(got_idx[g].tolist()), set(ref_idx[g].tolist())
        if a == b:
            continue
        kth = np.sort(logits[g])[::-1][len(ref_idx[g]) - 1]
        for i in a ^ b:
            assert abs(logits[g, i] - kth) <= 1e-5 * max(abs(kth), 1e-3), (g, i)


@pytest.mark.parametrize("name", ["ref_fp32_h1", "ref_bf16_gqa"])
def test_engine_reproduces_reference_vectors_with_the_reference_index(golden_dir, name):
    """The reference's trained index goes in (build_with_codebooks); packed codes, list ids, norms,
    top-k sets and attention outputs must come out as the reference recorded them, before and
    after per-step incremental appends."""
    dev = _cuda()
    from pqhsa_release_amd.attention import PQHSAEngine

    fx, m = _load(golden_dir, name)
    H, G, ctx, steps = m["heads"], m["groups"], m["ctx"], m["steps"]
    bf16 = name.endswith("gqa")
    kv_dtype = torch.bfloat16 if bf16 else torch.float32
    ic, ac = _cfgs(m["lists"], m["fraction"], sink=m["sink"], local=m["local"])
    keys = torch.from_numpy(fx["keys"]).to(dev, kv_dtype)[None]          # [1, H, ctx+steps, D]
    values = torch.from_numpy(fx["values"]).to(dev, kv_dtype)[None]
    eng = PQHSAEngine(ic, ac, batch=1, kv_heads=H, device=dev)
    eng.adopt(keys[:, :, :ctx], values[:, :, :ctx])
    eng.build([ctx], coarse=torch.from_numpy(fx["coarse"]), codebooks=torch.from_numpy(fx["codebooks"]))
    tol = 2e-3 if bf16 else 1e-4

    def check(tag, step):
        n = fx[f"{tag}_list_ids"].shape[1]
        assert eng.n(0) == n
        q = torch.from_numpy(fx["queries"][:, step]).reshape(1, H * G, DIM).to(dev)   # fp32 queries
        out = eng.forward(q, G)
        torch.cuda.synchronize()
        tidx, tval, tcnt = eng.last_topk(G)
        for h in range(H):
            ref_lists, ref_words = fx[f"{tag}_list_ids"][h], _words(fx[f"{tag}_packed"][h])
            codes_t, lists_t, norms_t = eng.index.by_key(h, n)
            lists, codes = u16(lists_t), u32(codes_t)
            # integer parity with the reference (these fixtures hold no argmin near-tie: the
            # fixed-order oracle reproduces them exactly too, tests/test_oracle_golden.py)
            assert np.array_equal(lists, ref_lists) and np.array_equal(codes, ref_words)
            np.testing.assert_allclose(norms_t.cpu().numpy(), fx[f"{tag}_norms"][h], rtol=1e-6)
            np.testing.assert_allclose(eng.index.vbar[h].cpu().numpy(), fx[f"{tag}_vbar"][h], atol=1e-5)
            k = fx[f"{tag}_topk_idx"].shape[2]
            got = tidx.reshape(H, G, -1)[h, :, :k].cpu().numpy()
            assert (tcnt.reshape(H, G)[h] == k).all()
            _margin_ok(fx[f"{tag}_scores"][h] * np.float32(SCALE), got, fx[f"{tag}_topk_idx"][h])
        err = (out[0].float().cpu().numpy() - fx[f"{tag}_output"]).__abs__().max()
        assert err <= tol, (tag, err)
        return err

    e0 = check("build", 0)
    for s in range(steps):
        pos = ctx + s
        eng.write_rows(keys[:, :, pos], values[:, :, pos])
        eng.advance(1)
    e1 = check("append", steps)
    print(f"{name}: max |out - reference| build {e0:.2e}, after {steps} appends {e1:.2e}")


def _problem(dev, *, batch=1, heads=2, groups=4, ctx=1500, extra=40, dtype=torch.bfloat16, seed=5):
    from pqhsa_release_amd.synth import make_layer

    k, v, _ = make_layer(ctx + extra, batch=batch, kv_heads=heads, groups=1, seed0=seed, dtype=dtype)
    gen = torch.Generator().manual_seed(seed + 1)
    first = min(100, k.shape[2] - (extra + 1) * groups)      # queries near some of the keys
    q = k[:, :, first:first + (extra + 1) * groups].float() + 0.2 * torch.randn(batch, heads, (extra + 1) * groups, DIM,
                                                                              generator=gen)
    q = q.reshape(batch, heads, extra + 1, groups, DIM).to(dtype)
    return k.to(dev), v.to(dev), q.to(dev)


def _oracle_check(eng, keys, values, q_step, groups, length, fraction, tol):
    """Run the fixed-order oracle on the engine's own index and compare top-k (exact) and output."""
    tidx, _, tcnt = eng.last_topk(groups)
    worst = 0.0
    outs = []
    for b in range(eng.B):
        for h in range(eng.H):
            bh, n = b * eng.H + h, eng.n(b)
            ix = _index_of(eng, bh, n)
            want_out, want_idx, _ = fixed.decode_step(q_step[b, h].float().cpu().numpy(),
                                                      keys[b, h, :length].float().cpu().numpy(),
                                                      values[b, h, :length].float().cpu().numpy(), ix,
                                                      sink=eng.sink, local=length - eng.sink - n,
                                                      fraction=fraction, scale=SCALE)
            k = want_idx.shape[1]
            got = tidx.reshape(eng.B, eng.H, groups, -1)[b, h, :, :k].cpu().numpy()
            for g in range(groups):
                assert np.array_equal(np.sort(got[g]), np.sort(want_idx[g])), (b, h, g)
            outs.append(want_out)
    return np.stack(outs).reshape(eng.B, eng.H * groups, DIM), worst


def test_gqa_adapter_decode_steps_match_oracle_on_its_own_index():
    dev = _cuda()
    from pqhsa_release_amd.attention import GQAIVFPQDecodeAttentionAdapter

    ctx, extra, H, G = 1500, 12, 2, 4
    keys, values, q = _problem(dev, heads=H, groups=G, ctx=ctx, extra=extra)
    ic, ac = _cfgs(64, 0.02)
    ad = GQAIVFPQDecodeAttentionAdapter(ic, ac, num_query_heads=H * G, num_key_value_heads=H)
    assert ad.build_cache(keys[:, :, :ctx], values[:, :, :ctx]) is ad
    assert ad.leading_shape == (1, H) and len(ad.streams) == H
    out = ad.forward(q[:, :, 0].reshape(1, H * G, DIM).float())
    assert out.context.shape == (1, H * G, DIM) and len(out.per_query) == G
    want, _ = _oracle_check(ad.engine, keys, values, q[:, :, 0], G, ctx, 0.02, 2e-3)
    assert np.abs(out.context.cpu().numpy() - want).max() <= 2e-3
    # decode_step appends, then attends (the new row is in the local window)
    for s in range(1, extra + 1):
        pos = ctx + s - 1
        res = ad.decode_step(q[:, :, s].reshape(1, H * G, 1, DIM).float(), keys[:, :, pos], values[:, :, pos : pos + 1])
        assert res.context.shape == (1, H * G, 1, DIM)
    assert ad.engine.n(0) == ctx + extra - 64 - 4 and ad.engine.index_adds == extra
    want, _ = _oracle_check(ad.engine, keys, values, q[:, :, extra], G, ctx + extra, 0.02, 2e-3)
    assert np.abs(res.context[:, :, 0].cpu().numpy() - want).max() <= 2e-3
    # appended keys were encoded exactly as a fresh encode of the same rows would
    n = ad.engine.n(0)
    for h in range(H):
        ix = _index_of(ad.engine, h, n)
        norms, lists, codes = fixed.encode(keys[0, h, 4 : 4 + n].float().cpu().numpy(), ix["coarse"], ix["codebooks"])
        assert np.array_equal(lists, ix["list_ids"]) and np.array_equal(codes, ix["codes"])
        assert np.array_equal(norms, ix["norms"])
    # bf16 queries in, bf16 context out
    res16 = ad.forward(q[:, :, extra].reshape(1, H * G, DIM))
    assert res16.context.dtype == torch.bfloat16
    assert np.abs(res16.context.float().cpu().numpy() - want).max() <= 2e-3 + 2.0 ** -8 * np.abs(want).max()


def test_engine_one_sequence_advances_across_a_capacity_growth():
    """Only one sequence of a batch advances, and its new key no longer fits the index: the step
    cannot append inside the decode launches and takes the separate path, which must start from
    the bookkeeping as it stood (the sequence that did not advance has nothing new to index).
    Counts, codes and the attention of both sequences are checked against the oracle."""
    dev = _cuda()
    from pqhsa_release_amd.attention import PQHSAEngine

    H, G, ctx, frac = 2, 2, 1100, 0.03
    keys, values, q = _problem(dev, batch=2, heads=H, groups=G, ctx=ctx, extra=4)
    ic, ac = _cfgs(32, frac)
    eng = PQHSAEngine(ic, ac, batch=2, kv_heads=H, device=dev, growth_margin=0)
    eng.bind_dense(keys.clone(), values.clone())              # rows beyond a sequence's length are simply not in use yet
    lens = [ctx, ctx - 40]
    eng.build(lens)
    n0 = [eng.n(0), eng.n(1)]
    assert eng.index.n_cap == n0[0], "the longest sequence fills the index exactly"
    for step in range(2):                                      # the first step grows the index, the second appends in-launch
        eng.advance(1, which=[0])
        lens[0] += 1
        out = eng.forward(q[:, :, step].reshape(2, H * G, DIM), G)
        torch.cuda.synchronize()
        assert eng.index.n_host == [n0[0] + step + 1, n0[1]] and eng.lens == lens
        tidx, _, _ = eng.last_topk(G)
        for b in range(2):
            for h in range(H):
                n = eng.n(b)
                ix = _index_of(eng, b * H + h, n)
                norms, lists, codes = fixed.encode(keys[b, h, 4 : 4 + n].float().cpu().numpy(), ix["coarse"], ix["codebooks"])
                assert np.array_equal(lists, ix["list_ids"]) and np.array_equal(codes, ix["codes"]), (step, b, h)
                want_out, want_idx, _ = fixed.decode_step(q[b, h, step].float().cpu().numpy(),
                                                          keys[b, h, : lens[b]].float().cpu().numpy(),
                                                          values[b, h, : lens[b]].float().cpu().numpy(), ix, sink=4,
                                                          local=lens[b] - 4 - n, fraction=frac, scale=SCALE)
                got = tidx.reshape(2, H, G, -1)[b, h, :, : want_idx.shape[1]].cpu().numpy()
                for g in range(G):
                    assert np.array_equal(np.sort(got[g]), np.sort(want_idx[g])), (step, b, h, g)
                err = np.abs(out[b, h * G : (h + 1) * G].float().cpu().numpy() - want_out).max()
                assert err <= 2e-3 + 2.0 ** -8 * np.abs(want_out).max(), (step, b, h, err)
    assert eng.index.n_cap > n0[0]


def test_plain_adapter_multi_query_and_state_round_trip():
    dev = _cuda()
    from pqhsa_release_amd.attention import IVFPQDecodeAttentionAdapter

    ctx, H, Q = 900, 2, 3
    keys, values, q = _problem(dev, batch=2, heads=H, groups=Q, ctx=ctx, extra=0, dtype=torch.float32, seed=9)
    ic, ac = _cfgs(32, 0.05)
    ad = IVFPQDecodeAttentionAdapter(ic, ac).build_cache(keys, values)
    queries = q[:, :, 0]                                            # [B, H, Q, D]
    res = ad.forward(queries)
    assert res.context.shape == (2, H, Q, DIM) and len(res.per_query) == Q
    assert res.per_query[0].per_stream[0].exact_retrieval_count == math.ceil((ctx - 68) * 0.05)
    want, _ = _oracle_check(ad.engine, keys, values, queries, Q, ctx, 0.05, 1e-4)
    assert np.abs(res.context.reshape(2, H * Q, DIM).cpu().numpy() - want).max() <= 1e-4
    single = ad.forward(queries[:, :, 0])                           # [B, H, D] -> [B, H, D]
    assert single.context.shape == (2, H, DIM)
    np.testing.assert_allclose(single.context.cpu().numpy(), res.context[:, :, 0].cpu().numpy(), atol=1e-5)
    state = ad.state_dict()
    clone = IVFPQDecodeAttentionAdapter.from_state_dict(state)
    again = clone.forward(queries)
    # same index, same selection; float sums may differ in the last bits (atomic accumulation order)
    np.testing.assert_allclose(again.context.cpu().numpy(), res.context.cpu().numpy(), atol=1e-5)
    assert clone.leading_shape == (2, H)


def test_all_tokens_selected_equals_dense_attention_through_the_adapter():
    dev = _cuda()
    from pqhsa_release_amd.attention import IVFPQDecodeAttentionAdapter

    keys, values, q = _problem(dev, heads=1, groups=1, ctx=400, extra=0, dtype=torch.float32, seed=21)
    ic, ac = _cfgs(8, 1.0, sink=2, local=5)
    ad = IVFPQDecodeAttentionAdapter(ic, ac).build_cache(keys, values)
    got = ad.forward(q[:, :, 0, 0]).context[0, 0].double().cpu()
    k64, v64, q64 = keys[0, 0].double().cpu(), values[0, 0].double().cpu(), q[0, 0, 0, 0].double().cpu()
    dense = torch.softmax((k64 @ q64) * SCALE, dim=0) @ v64
    np.testing.assert_allclose(got.numpy(), dense.numpy(), rtol=1e-4, atol=1e-5)


def test_deferred_strategy_flush_updates_codebooks_and_reencodes():
    dev = _cuda()
    from pqhsa_release_amd.attention import GQAIVFPQDecodeAttentionAdapter

    ctx, extra, H, G = 1200, 20, 2, 2
    keys, values, q = _problem(dev, heads=H, groups=G, ctx=ctx, extra=extra, seed=31)
    ic, ac = _cfgs(32, 0.02, strategy="deferred", interval=8)
    ad = GQAIVFPQDecodeAttentionAdapter(ic, ac, num_query_heads=H * G, num_key_value_heads=H)
    ad.build_cache(keys[:, :, :ctx], values[:, :, :ctx])
    n0 = ad.engine.n(0)
    coarse0 = ad.engine.index.coarse.clone()
    for s in range(extra):
        ad.append(keys[:, :, ctx + s], values[:, :, ctx + s])
    # deferred: nothing indexed yet, the pending rows stay exact in the local region
    assert ad.engine.n(0) == n0 and ad.engine.full_count(0) == 4 + 64 + extra and ad.engine.deferred_pending
    out = ad.forward(q[:, :, extra].reshape(1, H * G, DIM).float()).context
    want, _ = _oracle_check(ad.engine, keys, values, q[:, :, extra], G, ctx + extra, 0.02, 2e-3)
    assert np.abs(out.cpu().numpy() - want).max() <= 2e-3
    assert ad.apply_pending_index_update() == H and ad.apply_pending_index_update() == 0
    assert ad.engine.n(0) == n0 + extra and not torch.equal(coarse0, ad.engine.index.coarse)
    out = ad.forward(q[:, :, extra].reshape(1, H * G, DIM).float()).context
    want, _ = _oracle_check(ad.engine, keys, values, q[:, :, extra], G, ctx + extra, 0.02, 2e-3)
    assert np.abs(out.cpu().numpy() - want).max() <= 2e-3
    # after the flush every stored code is the encoding under the moved codebooks
    n = ad.engine.n(0)
    ix = _index_of(ad.engine, 1, n)
    _, lists, codes = fixed.encode(keys[0, 1, 4 : 4 + n].float().cpu().numpy(), ix["coarse"], ix["codebooks"])
    assert np.array_equal(lists, ix["list_ids"]) and np.array_equal(codes, ix["codes"])


@pytest.mark.parametrize("layout", ["5d", "4d"])
def test_vllm_hook_single_token_decode_over_a_paged_cache(layout, monkeypatch):
    dev = _cuda()
    from pqhsa_release_amd.vllm_backend import pq_hsa_decode_runtime as rt
    from pqhsa_release_amd.vllm_backend import pq_hsa_flashattn_wrap as wrap

    for k in list(os.environ):
        if k.startswith("PQ_HSA_"):
            monkeypatch.delenv(k)
    for k, v in {"PQ_HSA_ENABLE": "1", "PQ_HSA_NUM_LISTS": "64", "PQ_HSA_TOP_FRAC": "0.02", "PQ_HSA_LOCAL": "64",
                 "PQ_HSA_UPD_INTERVAL": "4", "PQ_HSA_FLUSH_INTERVAL": "4"}.items():
        monkeypatch.setenv(k, v)
    rt.reset_pq_hsa_runtime_stats()
    rt.reset_pq_hsa_layer_state()
    ctx, steps, H, G, bs = 1300, 9, 2, 4, 16
    keys, values, q = _problem(dev, heads=H, groups=G, ctx=ctx, extra=steps, seed=41)
    blocks = (ctx + steps + bs - 1) // bs
    table = torch.randperm(blocks + 4, generator=torch.Generator().manual_seed(1))[:blocks].to(torch.int32).to(dev)[None]
    if layout == "5d":
        cache = torch.zeros(2, blocks + 4, bs, H, DIM, dtype=torch.bfloat16, device=dev)
        kc, vc = cache[0], cache[1]
    else:
        cache = torch.zeros(blocks + 4, H, bs, 2 * DIM, dtype=torch.bfloat16, device=dev)
        kc, vc = tr.split_kv_cache(cache)
    pos = torch.arange(ctx, device=dev)
    kc[table[0, pos // bs].long(), pos % bs] = keys[0, :, :ctx].transpose(0, 1)
    vc[table[0, pos // bs].long(), pos % bs] = values[0, :, :ctx].transpose(0, 1)

    class Impl:
        scale, num_heads, num_kv_heads, kv_cache_dtype = SCALE, H * G, H, "auto"

        def forward(self, layer, query, key, value, kv_cache, attn_metadata, output=None, **extra):
            output.fill_(-7.0)
            return output

    wrap.wrap_forward(Impl)
    impl, layer = Impl(), types.SimpleNamespace(layer_name="layers.0.attn")
    try:
        for s in range(steps + 1):
            length = ctx + s
            slot = int(table[0, (length - 1) // bs]) * bs + (length - 1) % bs
            md = types.SimpleNamespace(max_query_len=1, num_actual_tokens=1, use_cascade=False, max_seq_len=length,
                                       seq_lens=torch.tensor([length], dtype=torch.int32, device=dev),
                                       block_table=table, slot_mapping=torch.tensor([slot], device=dev))
            k_new = keys[0, :, length - 1][None]                     # [1, H, D] this step's row
            v_new = values[0, :, length - 1][None]
            if layout == "4d":                                        # vLLM >= 0.10 writes the page itself
                kc[slot // bs, slot % bs] = k_new[0]
                vc[slot // bs, slot % bs] = v_new[0]
            out = torch.zeros(1, H * G, DIM, dtype=torch.bfloat16, device=dev)
            query = q[0, :, s].reshape(1, H * G, DIM)
            res = impl.forward(layer, query, k_new, v_new, cache, md, output=out)
            assert res is out and float(out.float().abs().max()) != 7.0
            eng = rt.state_for(impl, layer)["sidecar"].adapter.engine
            if s > 0 and s % 4 == 0:
                continue      # the hook flushed right after this forward: the index has moved on
            want, _ = _oracle_check(eng, keys, values, q[:, :, s], G, length, 0.02, 2e-3)
            err = np.abs(out.float().cpu().numpy() - want)
            assert (err <= 2e-3 + 2.0 ** -8 * np.abs(want)).all(), (s, err.max())
        assert rt.STATS["pq_build_calls"] == 1 and rt.STATS["pq_append_calls"] == steps
        assert rt.STATS["pq_flush_calls"] == steps // 4 and rt.STATS["sidecar"] == "GQASidecar"
        assert eng.keys_buf is None                                   # exact rows are read from the pages in place
        assert eng.n(0) == ctx + 8 - 64 - 4                           # two deferred flushes of 4 rows each
        # a prefill-shaped call goes to the wrapped original
        md.max_query_len = 5
        out = torch.zeros(1, H * G, DIM, dtype=torch.bfloat16, device=dev)
        impl.forward(layer, query, k_new, v_new, cache, md, output=out)
        assert float(out[0, 0, 0]) == -7.0
    finally:
        wrap.unwrap_forward(Impl)
        rt.reset_pq_hsa_layer_state()


def test_vllm_hook_extends_a_checkpointed_prefix_when_the_prompt_continues_it(monkeypatch):
    """PQ_HSA_PREFIX_EXTEND=1: the second request's prompt is the first one's followed by 150 more
    tokens.  The hook restores the checkpointed index and takes in only the added rows (no rebuild);
    the row of the first request's first decode token is overwritten by the new prompt.  Checked on
    the engine's own index: every stored code is the encoding of its key under the moved tables,
    top-k exact and output within tolerance of the oracle.  Parity with the reference's extend path
    is unpinned (its tests need vLLM); this pins the invariants."""
    dev = _cuda()
    from pqhsa_release_amd.vllm_backend import pq_hsa_decode_runtime as rt
    from pqhsa_release_amd.vllm_backend import pq_hsa_flashattn_wrap as wrap

    for k in list(os.environ):
        if k.startswith("PQ_HSA_"):
            monkeypatch.delenv(k)
    for k, v in {"PQ_HSA_ENABLE": "1", "PQ_HSA_NUM_LISTS": "64", "PQ_HSA_TOP_FRAC": "0.02", "PQ_HSA_LOCAL": "64",
                 "PQ_HSA_PREFIX_EXTEND": "1"}.items():
        monkeypatch.setenv(k, v)
    rt.reset_pq_hsa_runtime_stats()
    rt.reset_pq_hsa_layer_state()
    first, second, H, G, bs = 1300, 1450, 2, 4, 16      # sequence lengths at each request's first decode step
    keys, values, q = _problem(dev, heads=H, groups=G, ctx=second, extra=4, seed=43)
    other_k, other_v, _ = _problem(dev, heads=H, groups=G, ctx=200, extra=0, seed=44)   # the first request's own decode rows
    blocks = (second + 4 + bs - 1) // bs
    table = torch.randperm(blocks + 4, generator=torch.Generator().manual_seed(2))[:blocks].to(torch.int32).to(dev)[None]
    cache = torch.zeros(2, blocks + 4, bs, H, DIM, dtype=torch.bfloat16, device=dev)
    kc, vc = cache[0], cache[1]

    def write(lo, hi, k_src, v_src, src_lo):
        pos = torch.arange(lo, hi, device=dev)
        kc[table[0, pos // bs].long(), pos % bs] = k_src[0, :, src_lo : src_lo + hi - lo].transpose(0, 1)
        vc[table[0, pos // bs].long(), pos % bs] = v_src[0, :, src_lo : src_lo + hi - lo].transpose(0, 1)

    class Impl:
        scale, num_heads, num_kv_heads, kv_cache_dtype = SCALE, H * G, H, "auto"

        def forward(self, layer, query, key, value, kv_cache, attn_metadata, output=None, **extra):
            output.fill_(-7.0)
            return output

    prompt = list(range(first - 1))
    requests = {"r0": types.SimpleNamespace(prompt_token_ids=prompt)}
    runner = types.SimpleNamespace(input_batch=types.SimpleNamespace(req_ids=["r0"]), requests=requests)

    def decode(length, k_row, v_row, query):
        slot = int(table[0, (length - 1) // bs]) * bs + (length - 1) % bs
        md = types.SimpleNamespace(max_query_len=1, num_actual_tokens=1, use_cascade=False, max_seq_len=length,
                                   seq_lens=torch.tensor([length], dtype=torch.int32, device=dev),
                                   block_table=table, slot_mapping=torch.tensor([slot], device=dev), _pq_runner=runner)
        out = torch.zeros(1, H * G, DIM, dtype=torch.bfloat16, device=dev)
        impl.forward(layer, query, k_row, v_row, cache, md, output=out)
        assert float(out.float().abs().max()) != 7.0
        return out

    wrap.wrap_forward(Impl)
    impl, layer = Impl(), types.SimpleNamespace(layer_name="layers.0.attn")
    try:
        # first request: prompt rows, then three decode tokens of its own
        write(0, first - 1, keys, values, 0)
        for s in range(3):
            decode(first + s, other_k[0, :, s][None], other_v[0, :, s][None], q[0, :, 0].reshape(1, H * G, DIM))
        sc = rt.state_for(impl, layer)["sidecar"]
        assert rt.STATS["pq_build_calls"] == 1 and sc.prefix_checkpoint_length == first
        # second request: the same prompt and 150 more tokens, all prefilled into the pages
        requests["r0"] = types.SimpleNamespace(prompt_token_ids=prompt + [5] * (second - first))
        write(first - 1, second - 1, keys, values, first - 1)
        query = q[0, :, 1].reshape(1, H * G, DIM)
        out = decode(second, keys[0, :, second - 1][None], values[0, :, second - 1][None], query)
        assert rt.STATS["pq_build_calls"] == 1 and rt.STATS["prefix_extend_hits"] == 1
        assert rt.STATS["pq_extend_delta_tokens_total"] == second - first
        last = rt.STATS["pq_extend_last"]
        assert last["base_length"] == first and last["new_length"] == second and last["flush_applied_streams"] == H
        assert rt.state_for(impl, layer)["sidecar"] is sc and sc.prefix_checkpoint_length == second
        eng = sc.adapter.engine
        n = eng.n(0)
        assert n == second - 64 - 4 and eng.keys_buf is None
        want, _ = _oracle_check(eng, keys, values, q[:, :, 1], G, second, 0.02, 2e-3)
        err = np.abs(out.float().cpu().numpy() - want)
        assert (err <= 2e-3 + 2.0 ** -8 * np.abs(want)).all(), err.max()
        for h in range(H):
            ix = _index_of(eng, h, n)
            _, lists, codes = fixed.encode(keys[0, h, 4 : 4 + n].float().cpu().numpy(), ix["coarse"], ix["codebooks"])
            assert np.array_equal(lists, ix["list_ids"]) and np.array_equal(codes, ix["codes"])
        # and decoding goes on from there
        out = decode(second + 1, keys[0, :, second][None], values[0, :, second][None], q[0, :, 2].reshape(1, H * G, DIM))
        want, _ = _oracle_check(eng, keys, values, q[:, :, 2], G, second + 1, 0.02, 2e-3)
        err = np.abs(out.float().cpu().numpy() - want)
        assert (err <= 2e-3 + 2.0 ** -8 * np.abs(want)).all(), err.max()
        assert rt.STATS["pq_append_calls"] == 3 and rt.STATS["pq_build_calls"] == 1
    finally:
        wrap.unwrap_forward(Impl)
        rt.reset_pq_hsa_layer_state()


def _batch_hook(dev, monkeypatch, ctxs, steps, *, share_first_block=False, request_ids=False, lists="64"):
    """A paged cache holding one synthetic request per entry of ``ctxs`` and a ``run(fused, reqs_at)``
    that drives the wrapped forward for ``steps + 1`` decode steps over the requests ``reqs_at(step)``
    names, returning the outputs per step and the runtime's counters.  ``share_first_block``: the
    first two requests begin with the same 16 tokens and share their first physical block, as under
    vLLM's prefix caching.  ``request_ids``: the metadata carries a model runner with vLLM's
    request ids."""
    from pqhsa_release_amd.vllm_backend import pq_hsa_decode_runtime as rt
    from pqhsa_release_amd.vllm_backend import pq_hsa_flashattn_wrap as wrap

    H, G, bs = 2, 4, 16
    B = len(ctxs)
    probs = [_problem(dev, heads=H, groups=G, ctx=c, extra=steps, seed=50 + i) for i, c in enumerate(ctxs)]
    per_seq = (max(ctxs) + steps + bs - 1) // bs
    perm = torch.randperm(B * per_seq, generator=torch.Generator().manual_seed(3)).to(torch.int32).to(dev)
    table = perm.reshape(B, per_seq).contiguous()
    if share_first_block:
        probs[1][0][:, :, :bs] = probs[0][0][:, :, :bs]
        probs[1][1][:, :, :bs] = probs[0][1][:, :, :bs]
        table[1, 0] = table[0, 0]
    cache = torch.zeros(2, B * per_seq, bs, H, DIM, dtype=torch.bfloat16, device=dev)
    for b, (keys, values, _) in enumerate(probs):
        pos = torch.arange(ctxs[b], device=dev)
        cache[0][table[b, pos // bs].long(), pos % bs] = keys[0, :, : ctxs[b]].transpose(0, 1)
        cache[1][table[b, pos // bs].long(), pos % bs] = values[0, :, : ctxs[b]].transpose(0, 1)

    class Impl:
        scale, num_heads, num_kv_heads, kv_cache_dtype = SCALE, H * G, H, "auto"

        def forward(self, layer, query, key, value, kv_cache, attn_metadata, output=None, **extra):
            output.fill_(-7.0)
            return output

    def run(fused, reqs_at):
        for k in list(os.environ):
            if k.startswith("PQ_HSA_"):
                monkeypatch.delenv(k)
        for k, v in {"PQ_HSA_ENABLE": "1", "PQ_HSA_BATCH": "1", "PQ_HSA_BATCH_FUSED": fused, "PQ_HSA_NUM_LISTS": lists,
                     "PQ_HSA_TOP_FRAC": "0.02", "PQ_HSA_LOCAL": "64", "PQ_HSA_UPD_INTERVAL": "1",
                     "PQ_HSA_FLUSH_INTERVAL": "0"}.items():
            monkeypatch.setenv(k, v)
        rt.reset_pq_hsa_runtime_stats()
        rt.reset_pq_hsa_layer_state()
        kvc = cache.clone()
        wrap.wrap_forward(Impl)
        impl, layer = Impl(), types.SimpleNamespace(layer_name="layers.0.attn")
        outs = []
        try:
            for s in range(steps + 1):
                reqs = reqs_at(s)
                lens = [ctxs[b] + s for b in reqs]
                last = torch.tensor([ln - 1 for ln in lens], device=dev)
                tb = table[reqs].contiguous()
                slots = tb[torch.arange(len(reqs), device=dev), last // bs].long() * bs + last % bs
                md = types.SimpleNamespace(max_query_len=1, num_actual_tokens=len(reqs), use_cascade=False,
                                           max_seq_len=max(lens), block_table=tb, slot_mapping=slots,
                                           seq_lens=torch.tensor(lens, dtype=torch.int32, device=dev))
                if request_ids:
                    md._pq_runner = types.SimpleNamespace(
                        input_batch=types.SimpleNamespace(req_ids=[f"req-{b}" for b in reqs] + [None]), requests={})
                k_new = torch.cat([probs[b][0][:, :, ctxs[b] + s - 1] for b in reqs])      # [R, H, D]
                v_new = torch.cat([probs[b][1][:, :, ctxs[b] + s - 1] for b in reqs])
                query = torch.cat([probs[b][2][0, :, s].reshape(1, H * G, DIM) for b in reqs])
                out = torch.zeros(len(reqs), H * G, DIM, dtype=torch.bfloat16, device=dev)
                res = impl.forward(layer, query, k_new, v_new, kvc, md, output=out)
                assert res is out and float(out.float().abs().max()) != 7.0
                outs.append(out.float().cpu().numpy())
            return outs, dict(rt.STATS)
        finally:
            wrap.unwrap_forward(Impl)
            rt.reset_pq_hsa_layer_state()

    return run


def _close(a, b, what):
    # the same kernels on the same trained indexes: only bf16 rounding of the output differs
    assert np.abs(a - b).max() <= 2e-3 + 2.0 ** -7 * np.abs(b).max(), (what, np.abs(a - b).max())


def test_vllm_hook_batch_mode_one_engine_for_all_requests(monkeypatch):
    """PQ_HSA_BATCH=1: a ragged decode batch through the hook, once with one engine for the whole
    batch (the default: appends ride on the decode launches) and once with one sidecar per
    request (the reference's form); both must agree with each other step by step, and the
    batch must be rebuilt when a request leaves."""
    dev = _cuda()
    steps = 6
    run = _batch_hook(dev, monkeypatch, [1500, 900, 1203], steps)
    close = _close

    everyone = lambda s: [0, 1, 2]
    one_leaves = lambda s: [0, 1, 2] if s < 4 else [0, 2]
    one_joins = lambda s: [0, 1] if s < 3 else [0, 1, 2]
    rows_swap = lambda s: [0, 1, 2] if s < 3 else [2, 0, 1]

    fused, st_f = run("1", everyone)
    single, st_s = run("0", everyone)
    assert st_f["pq_batch_fused_steps"] == steps + 1 and st_f["pq_batch_group_builds"] == 1
    assert st_f["pq_batch_regroups"] == 0 and st_s["pq_batch_fused_steps"] == 0 and st_s["pq_build_calls"] == 3
    for s_, (a, b) in enumerate(zip(fused, single)):
        close(a, b, ("everyone", s_))

    # a request leaves: the group keeps the index rows of the two that stay (no rebuild); the
    # per-request form goes by batch row, so it rebuilds the request that moved up a row
    left, st_l = run("1", one_leaves)
    assert st_l["pq_batch_group_builds"] == 1 and st_l["pq_batch_regroups"] == 1 and st_l["pq_build_calls"] == 1
    for s_, a in enumerate(left):
        want = fused[s_] if s_ < 4 else fused[s_][[0, 2]]     # what the full batch gave for the same requests
        close(a, want, ("one leaves", s_))

    # a request joins: only the newcomer is built, at the step it appears, as its own sidecar would be
    joined, st_j = run("1", one_joins)
    single_j, _ = run("0", one_joins)
    assert st_j["pq_batch_group_builds"] == 1 and st_j["pq_batch_regroups"] == 1 and st_j["pq_build_calls"] == 2
    for s_, (a, b) in enumerate(zip(joined, single_j)):
        close(a, b, ("one joins", s_))

    # requests change rows: told apart by the blocks they own, their indexes move with them
    swapped, st_w = run("1", rows_swap)
    assert st_w["pq_batch_group_builds"] == 1 and st_w["pq_batch_regroups"] == 1 and st_w["pq_build_calls"] == 1
    for s_, a in enumerate(swapped):
        want = fused[s_] if s_ < 3 else fused[s_][[2, 0, 1]]
        close(a, want, ("rows swap", s_))


@pytest.mark.parametrize("request_ids", [False, True])
def test_vllm_hook_batch_mode_tells_apart_requests_that_share_their_first_block(monkeypatch, request_ids):
    """Two live requests with a common prompt prefix share their first physical block (vLLM's
    prefix caching).  When the batch rows are permuted each request must keep its own index: by
    vLLM's request ids when the metadata carries the runner, by the blocks a request alone owns
    otherwise.  Nothing is rebuilt, and every output is what the unpermuted batch gives."""
    dev = _cuda()
    steps = 5
    run = _batch_hook(dev, monkeypatch, [1100, 1100, 700], steps, share_first_block=True, request_ids=request_ids)
    base, st_b = run("1", lambda s: [0, 1, 2])
    assert st_b["pq_batch_group_builds"] == 1 and st_b["pq_batch_regroups"] == 0
    swapped, st_w = run("1", lambda s: [0, 1, 2] if s < 2 else [1, 0, 2])
    assert st_w["pq_batch_group_builds"] == 1 and st_w["pq_batch_regroups"] == 1 and st_w["pq_build_calls"] == 1
    for s_, a in enumerate(swapped):
        _close(a, base[s_] if s_ < 2 else base[s_][[1, 0, 2]], ("shared first block", s_))
    # requests 0 and 1 are equally long here: had they been confused, 1's queries would have run on 0's index
    assert np.abs(base[3][0] - base[3][1]).max() > 0.05


def test_vllm_hook_batch_mode_with_a_request_shorter_than_the_list_count(monkeypatch):
    """A request with fewer indexed keys than PQ_HSA_NUM_LISTS joins a running batch and leaves
    again.  Every stream keeps the list count it would have alone (the short one trains one list
    per key, the long ones all 64; unused table columns are padded), so the outputs are those of
    one sidecar per request, and the batch is regrouped, not rebuilt."""
    dev = _cuda()
    steps = 6
    ctxs = [1500, 110, 900]                    # 110 tokens: 42 keys to index with sink 4 and local window 64
    run = _batch_hook(dev, monkeypatch, ctxs, steps)
    comes_and_goes = lambda s: [0, 2] if s < 2 else ([0, 2, 1] if s < 5 else [0, 2])   # per-row sidecars keep rows 0, 1
    fused, st_f = run("1", comes_and_goes)
    single, _ = run("0", comes_and_goes)
    assert st_f["pq_batch_group_builds"] == 1 and st_f["pq_batch_regroups"] == 2 and st_f["pq_build_calls"] == 2
    for s_, (a, b) in enumerate(zip(fused, single)):
        _close(a, b, ("short request", s_))
    # and the whole batch built at once, short request included
    together, st_t = run("1", lambda s: [0, 1, 2])
    alone, _ = run("0", lambda s: [0, 1, 2])
    assert st_t["pq_batch_group_builds"] == 1 and st_t["pq_batch_regroups"] == 0
    for s_, (a, b) in enumerate(zip(together, alone)):
        _close(a, b, ("short request from the start", s_))


def test_deferred_flush_reproduces_the_reference_online_refresh(golden_dir):
    """The deferred strategy against vectors from the real reference: the reference's trained index
    goes in, keys are appended without touching it, and apply_pending_index_update must move the
    coarse centroids and PQ codewords to where the reference's online refresh moved them, re-encode
    every key as the reference did, rebuild the list means, and attend as the reference does before
    and after the flush."""
    dev = _cuda()
    from pqhsa_release_amd.attention import PQHSAEngine

    fx = np.load(os.path.join(golden_dir, "ref_deferred_flush.npz"))
    ctx, H, G, lists, added, sink, local = (int(x) for x in fx["meta"])
    fraction = float(fx["fraction"][0])
    ic, ac = _cfgs(lists, fraction, sink=sink, local=local, strategy="deferred", interval=8)
    assert ic.online_codebook_lr == float(fx["lr"][0])
    keys = torch.from_numpy(fx["keys"]).to(dev, torch.bfloat16)[None]
    values = torch.from_numpy(fx["values"]).to(dev, torch.bfloat16)[None]
    q = torch.from_numpy(fx["queries"]).reshape(1, H * G, DIM).to(dev)            # fp32 queries
    eng = PQHSAEngine(ic, ac, batch=1, kv_heads=H, device=dev)
    eng.adopt(keys[:, :, :ctx], values[:, :, :ctx])
    eng.build([ctx], coarse=torch.from_numpy(fx["build_coarse"]), codebooks=torch.from_numpy(fx["build_codebooks"]))
    n0 = eng.n(0)
    for s in range(added):
        eng.write_rows(keys[:, :, ctx + s], values[:, :, ctx + s])
        eng.advance(1)
    assert eng.n(0) == n0 and eng.deferred_pending
    out = eng.forward(q, G)
    assert float((out[0].cpu() - torch.from_numpy(fx["pending_output"])).abs().max()) <= 2e-3
    assert eng.apply_pending_index_update() and not eng.apply_pending_index_update()
    n = eng.n(0)
    assert n == fx["flush_list_ids"].shape[1] == n0 + added
    mismatched = 0
    for h in range(H):
        np.testing.assert_allclose(eng.index.coarse[h].cpu().numpy(), fx["flush_coarse"][h], rtol=0, atol=1e-6)
        np.testing.assert_allclose(eng.index.codebooks[h].cpu().numpy(), fx["flush_codebooks"][h], rtol=0, atol=1e-6)
        codes_t, lists_t, norms_t = eng.index.by_key(h, n)
        got_lists, got_codes = u16(lists_t), u32(codes_t)
        ref_lists, ref_codes = fx["flush_list_ids"][h], _words(fx["flush_packed"][h])
        np.testing.assert_allclose(norms_t.cpu().numpy(), fx["flush_norms"][h], rtol=1e-6)
        # the moved tables agree to 1e-6, not bit for bit (different summation order of the means):
        # a key may change list or codeword only where its two nearest candidates are a near-tie
        dirs = torch.from_numpy(fx["keys"][h, sink : sink + n])
        dirs = dirs / torch.linalg.vector_norm(dirs, dim=-1, keepdim=True)
        coarse = torch.from_numpy(fx["flush_coarse"][h])
        d2 = torch.cdist(dirs, coarse) ** 2
        for i in np.nonzero(got_lists != ref_lists)[0]:
            a, b = float(d2[i, int(got_lists[i])]), float(d2[i, int(ref_lists[i])])
            assert abs(a - b) <= 1e-5 * max(a, b), (h, i, a, b)
            mismatched += 1
        same_list = got_lists == ref_lists
        books = torch.from_numpy(fx["flush_codebooks"][h])
        resid = dirs - coarse[torch.from_numpy(ref_lists.astype(np.int64))]
        for i in np.nonzero((got_codes != ref_codes) & same_list)[0]:
            for m in range(8):
                cg, cr = (int(got_codes[i]) >> (4 * m)) & 15, (int(ref_codes[i]) >> (4 * m)) & 15
                if cg == cr:
                    continue
                sub = resid[i, 16 * m : 16 * m + 16]
                a, b = float(((sub - books[m, cg]) ** 2).sum()), float(((sub - books[m, cr]) ** 2).sum())
                assert abs(a - b) <= 1e-5 * max(a, b, 1e-6), (h, i, m, a, b)
            mismatched += 1
        np.testing.assert_allclose(eng.index.vbar[h].cpu().numpy(), fx["flush_vbar"][h], atol=2e-3 if mismatched else 1e-5)
    out = eng.forward(q, G)
    err = float((out[0].cpu() - torch.from_numpy(fx["flush_output"])).abs().max())
    assert err <= 2e-3, err
    print(f"deferred flush vs reference: {mismatched} near-tie keys of {H * n}, max |out - reference| {err:.2e}")


@pytest.mark.parametrize("name", ["ref_fp32_h1", "ref_bf16_gqa"])
def test_device_index_training_reproduces_the_reference_tables(golden_dir, name):
    """Index training on the device (pqhsa_release_amd.index.train: CPU-drawn seeds, Lloyd
    iterations as device products) against the tables the reference trained on the same keys with
    the same seed: within 1e-5, per stream and batched (reference: pq_hsa/index/ivfpq.py:84-140,
    pq.py:47-95)."""
    dev = _cuda()
    from pqhsa_release_amd.index.train import train_ivfpq, train_ivfpq_batched

    fx, m = _load(golden_dir, name)
    keys = torch.from_numpy(fx["keys"])[:, m["sink"]:m["ctx"] - m["local"]].to(dev)
    worst = 0.0
    for h in range(m["heads"]):
        coarse, books = train_ivfpq(keys[h], num_lists=m["lists"], coarse_iter=1, pq_iter=2, seed=0)
        worst = max(worst, float(np.abs(coarse.cpu().numpy() - fx["coarse"][h]).max()),
                    float(np.abs(books.cpu().numpy() - fx["codebooks"][h]).max()))
    coarse, books = train_ivfpq_batched(keys, num_lists=m["lists"], coarse_iter=1, pq_iter=2, seed=0)
    worst = max(worst, float(np.abs(coarse.cpu().numpy() - fx["coarse"]).max()),
                float(np.abs(books.cpu().numpy() - fx["codebooks"]).max()))
    print(f"{name}: max |trained table - reference| {worst:.2e}")
    assert worst <= 1e-5
