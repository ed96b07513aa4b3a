"""CPU tests of the host-side mirror of the reference interface: packing helpers, configuration
records, adapter error behaviour, the vLLM decode hook's gating / state machine / STATS (with
fake impl, metadata and sidecar objects, as the reference's own hook tests need a real vLLM)."""

import os
import types

import pytest
import torch

import pqhsa_release_amd as pkg
from pqhsa_release_amd.attention import GQAIVFPQDecodeAttentionAdapter, IVFPQDecodeAttentionAdapter
from pqhsa_release_amd.config import IVFPQConfig, SparseAttentionConfig, validate_for_kernels
from pqhsa_release_amd.vllm_backend import pq_hsa_decode_runtime as rt
from pqhsa_release_amd.vllm_backend import pq_hsa_flashattn_wrap as wrap
from pqhsa_release_amd.vllm_plugin import plugin
from pqhsa_release_amd.vllm_plugin.config import PQHSAConfig


def paper_cfgs():
    ic = IVFPQConfig(num_lists=64, num_subspaces=8, num_bits=4, coarse_max_iter=1, pq_max_iter=2,
                     direction_normalize=True, kernel_backend="mi355x")
    ac = SparseAttentionConfig(sink_tokens=4, local_window=64, retrieval_top_fraction=0.02, mode="hybrid",
                               hybrid_value_mode="centroid", collect_attention_details=False)
    return ic, ac


def test_packing_helpers_follow_reference_layout():
    codes = torch.tensor([[0, 1, 2, 3], [15, 14, 13, 12]])
    packed = pkg.pack_4bit_codes(codes)
    assert packed.dtype == torch.uint8 and packed.tolist() == [[0x10, 0x32], [0xEF, 0xCD]]
    assert torch.equal(pkg.unpack_4bit_codes(packed, 4), codes)
    odd = torch.tensor([[1, 2, 3], [4, 5, 6]])
    p = pkg.pack_4bit_codes(odd)
    assert p.shape == (2, 2) and torch.all((p[:, -1] >> 4) == 0)
    assert torch.equal(pkg.unpack_4bit_codes(p, 3), odd)
    with pytest.raises(ValueError, match=r"\[0, 15\]"):
        pkg.pack_4bit_codes(torch.tensor([[0, 16]]))
    with pytest.raises(ValueError):
        pkg.unpack_4bit_codes(packed, 7)


def test_config_defaults_match_reference_and_validation_is_loud():
    assert IVFPQConfig().num_lists == 256 and IVFPQConfig().num_bits == 8 and IVFPQConfig().eps == 1e-12
    ac = SparseAttentionConfig()
    assert (ac.mode, ac.hybrid_value_mode, ac.index_update_strategy, ac.retrieval_topk) == \
        ("sparse", "denominator", "incremental", 100)
    ic, ac = paper_cfgs()
    validate_for_kernels(ic, ac)
    for bad in (dict(num_bits=8), dict(num_subspaces=16), dict(direction_normalize=False), dict(rotation="random_orthogonal")):
        with pytest.raises(ValueError):
            validate_for_kernels(IVFPQConfig(**{**{n: getattr(ic, n) for n in ic.__slots__}, **bad}), ac)
    for bad in (dict(mode="sparse"), dict(hybrid_value_mode="full"), dict(exact_rerank=False), dict(retrieval_top_p=0.9),
                dict(retrieval_top_fraction=1.5), dict(index_update_strategy="sometimes"), dict(kv_storage="cpu")):
        with pytest.raises(ValueError):
            validate_for_kernels(ic, SparseAttentionConfig(**{**{n: getattr(ac, n) for n in ac.__slots__}, **bad}))


def test_adapters_raise_like_the_reference_before_build_and_on_bad_shapes():
    ic, ac = paper_cfgs()
    ad = IVFPQDecodeAttentionAdapter(ic, ac)
    with pytest.raises(RuntimeError):
        ad.forward(torch.zeros(1, 2, 128))
    with pytest.raises(RuntimeError):
        ad.leading_shape
    with pytest.raises(ValueError):
        ad.build_cache(torch.zeros(2, 100, 128), torch.zeros(2, 100, 128))
    with pytest.raises(RuntimeError, match="no CPU path"):
        ad.build_cache(torch.zeros(1, 2, 300, 128), torch.zeros(1, 2, 300, 128))      # CPU tensors
    with pytest.raises(ValueError):
        ad.decode_step(torch.zeros(1, 2, 128))                                         # append_kv without K/V
    with pytest.raises(ValueError, match="divisible"):
        GQAIVFPQDecodeAttentionAdapter(ic, ac, num_query_heads=7, num_key_value_heads=2)
    g = GQAIVFPQDecodeAttentionAdapter(ic, ac, num_query_heads=8, num_key_value_heads=2)
    assert g.num_key_value_groups == 4
    with pytest.raises(ValueError, match="KV heads"):
        g.build_cache(torch.zeros(1, 3, 300, 128), torch.zeros(1, 3, 300, 128))


def meta(seq_len=500, reqs=1, qlen=1, tokens=1, cascade=False):
    return types.SimpleNamespace(max_query_len=qlen, num_actual_tokens=tokens, use_cascade=cascade,
                                 seq_lens=torch.full((reqs,), seq_len, dtype=torch.int32), max_seq_len=seq_len,
                                 block_table=torch.zeros(reqs, 64, dtype=torch.int32),
                                 slot_mapping=torch.zeros(tokens, dtype=torch.int64))


@pytest.fixture
def clean_runtime(monkeypatch):
    for k in list(os.environ):
        if k.startswith("PQ_HSA_"):
            monkeypatch.delenv(k)
    rt.reset_pq_hsa_runtime_stats()
    rt.reset_pq_hsa_layer_state()
    yield
    rt.reset_pq_hsa_runtime_stats()
    rt.reset_pq_hsa_layer_state()


def test_should_pq_decode_gate_and_reject_reasons(clean_runtime, monkeypatch):
    assert rt.min_pq_seq() == 4 + 128 + 16
    assert rt.should_pq_decode(meta())
    assert not rt.should_pq_decode(None)
    assert not rt.should_pq_decode(meta(cascade=True))
    assert not rt.should_pq_decode(meta(qlen=2))
    assert not rt.should_pq_decode(meta(tokens=2))
    assert not rt.should_pq_decode(meta(reqs=2))
    assert not rt.should_pq_decode(meta(seq_len=100))
    assert rt.STATS["reject"] == {"no_metadata": 1, "cascade": 1, "max_query_len!=1": 1, "num_actual_tokens!=1": 1,
                                  "num_reqs!=1": 1, "seq_too_short": 1}
    monkeypatch.setenv("PQ_HSA_BATCH", "1")
    assert rt.should_pq_decode(meta(reqs=3, tokens=3))
    assert not rt.should_pq_decode(meta(reqs=3, tokens=2))
    monkeypatch.setenv("PQ_HSA_LOCAL", "64")
    assert rt.min_pq_seq() == 84


class FakeSidecar:
    built = 0

    def __init__(self, icfg, acfg, *, num_query_heads, num_kv_heads):
        self.icfg, self.acfg, self.hq, self.hkv = icfg, acfg, num_query_heads, num_kv_heads
        self.length, self.appended, self.flushed, self.fail = 0, 0, 0, False
        self._ckpt = None

    batched_heads_active = True
    cuda_graph_active = False

    @property
    def prefix_checkpoint_length(self):
        return self._ckpt

    def build_cache(self, keys, values):
        FakeSidecar.built += 1
        self.length = keys.shape[2]
        return self

    def set_paged_kv_context(self, kv_cache, attn_metadata, seq_idx=0):
        self.paged = (kv_cache, seq_idx)

    def append(self, k, v):
        assert k.shape == (1, self.hkv, 128)
        self.appended += 1
        self.length += 1

    def forward(self, q):
        if self.fail:
            raise RuntimeError("boom")
        return torch.full((1, self.hq, 128), float(self.length))

    def apply_pending_index_update(self):
        self.flushed += 1
        return 1

    def checkpoint_prefix(self):
        self._ckpt = self.length

    def restore_prefix(self, k, v, *, kv_cache=None, attn_metadata=None, seq_idx=0):
        self.length = self._ckpt
        return True


@pytest.fixture
def fake_stack(clean_runtime, monkeypatch):
    FakeSidecar.built = 0
    monkeypatch.setattr(rt, "sidecar_cls", lambda: FakeSidecar)
    monkeypatch.setattr(rt, "gather_flashattn_kv",
                        lambda kv, md, i=0: (torch.zeros(1, 2, int(md.max_seq_len), 128),
                                             torch.zeros(1, 2, int(md.max_seq_len), 128), int(md.max_seq_len)))
    impl = types.SimpleNamespace(scale=0.088, num_heads=8, num_kv_heads=2, kv_cache_dtype="auto")
    layer = types.SimpleNamespace(layer_name="model.layers.0.self_attn.attn")
    kv_cache = torch.zeros(64, 2, 16, 256)         # 4-D layout: nothing to write in the hook
    return impl, layer, kv_cache


def step(impl, layer, kv_cache, seq_len, dense_value=-1.0):
    q, k, v = torch.zeros(1, 8, 128), torch.zeros(1, 2, 128), torch.zeros(1, 2, 128)
    out = torch.zeros(1, 8, 128)
    res = rt.pq_or_dense_forward(impl, layer, q, k, v, kv_cache, meta(seq_len), out,
                                 lambda: torch.full((1, 8, 128), dense_value))
    return res


def test_hook_state_machine_build_append_flush_rebuild(fake_stack, monkeypatch):
    impl, layer, kv_cache = fake_stack
    # disabled: dense path, nothing built
    assert float(step(impl, layer, kv_cache, 500)[0, 0, 0]) == -1.0
    assert rt.STATS["dense_fa_calls"] == 1 and FakeSidecar.built == 0
    monkeypatch.setenv("PQ_HSA_ENABLE", "1")
    monkeypatch.setenv("PQ_HSA_FLUSH_INTERVAL", "2")
    assert float(step(impl, layer, kv_cache, 500)[0, 0, 0]) == 500.0              # first step builds
    sc = rt.state_for(impl, layer)["sidecar"]
    assert isinstance(sc, FakeSidecar) and sc.acfg.scale == pytest.approx(0.088) and sc.acfg.mode == "hybrid"
    assert sc.icfg.num_lists == 512 and sc.acfg.index_update_strategy == "deferred"
    assert rt.STATS["pq_build_calls"] == 1 and rt.STATS["prefix_persist_misses"] == 1
    assert rt.STATS["prefix_miss_reasons"] == {"no_adapter": 1}
    assert float(step(impl, layer, kv_cache, 501)[0, 0, 0]) == 501.0              # sequential: append
    assert float(step(impl, layer, kv_cache, 502)[0, 0, 0]) == 502.0
    assert sc.appended == 2 and sc.flushed == 1 and rt.STATS["pq_flush_calls"] == 1
    assert rt.STATS["pq_append_calls"] == 2 and rt.STATS["pq_decode_calls"] == 3
    assert float(step(impl, layer, kv_cache, 700)[0, 0, 0]) == 700.0              # non-sequential: rebuild
    assert FakeSidecar.built == 2 and rt.STATS["prefix_miss_reasons"]["no_prefix_key"] == 1
    # short sequence falls through to dense and records why
    assert float(step(impl, layer, kv_cache, 100)[0, 0, 0]) == -1.0
    assert rt.STATS["reject"]["seq_too_short"] == 1


def test_hook_error_convention_reraise_or_dense_fallback(fake_stack, monkeypatch):
    impl, layer, kv_cache = fake_stack
    monkeypatch.setenv("PQ_HSA_ENABLE", "1")
    step(impl, layer, kv_cache, 500)
    rt.state_for(impl, layer)["sidecar"].fail = True
    with pytest.raises(RuntimeError, match="boom"):
        step(impl, layer, kv_cache, 501)
    assert rt.STATS["last_error"] == "RuntimeError: boom" and rt.STATS["dense_fallback_calls"] == 1
    monkeypatch.setenv("PQ_HSA_FALLBACK", "1")
    rt.state_for(impl, layer)["seq_len"] = 501
    assert float(step(impl, layer, kv_cache, 502)[0, 0, 0]) == -1.0
    assert rt.STATS["dense_fallback_calls"] == 2


def test_prefix_checkpoint_restore_on_same_prompt(fake_stack, monkeypatch):
    impl, layer, kv_cache = fake_stack
    monkeypatch.setenv("PQ_HSA_ENABLE", "1")
    runner = types.SimpleNamespace(input_batch=types.SimpleNamespace(req_ids=["r0"]),
                                   requests={"r0": types.SimpleNamespace(prompt_token_ids=list(range(499)))})

    def go(seq_len):
        md = meta(seq_len)
        md._pq_runner = runner
        out = torch.zeros(1, 8, 128)
        return rt.pq_or_dense_forward(impl, layer, torch.zeros(1, 8, 128), torch.zeros(1, 2, 128),
                                      torch.zeros(1, 2, 128), kv_cache, md, out, lambda: out)

    go(500)
    go(501)
    assert float(go(500)[0, 0, 0]) == 500.0           # same prompt again: restored, not rebuilt
    assert FakeSidecar.built == 1 and rt.STATS["prefix_persist_hits"] == 1


def test_prefix_extend_when_the_prompt_continues_the_checkpointed_one(fake_stack, monkeypatch):
    # reasons and counters as in the reference's runtime (pq_hsa_decode_runtime.py:431-488, 574-618)
    impl, layer, kv_cache = fake_stack
    monkeypatch.setenv("PQ_HSA_ENABLE", "1")
    requests = {"r0": types.SimpleNamespace(prompt_token_ids=list(range(499)))}
    runner = types.SimpleNamespace(input_batch=types.SimpleNamespace(req_ids=["r0"]), requests=requests)
    calls = []

    def extend_prefix(self, k, v, *, kv_cache, attn_metadata, seq_idx=0, new_length):
        calls.append((self._ckpt, new_length))
        if self.fail:
            return None
        self.length = new_length
        return {"base_length": self._ckpt, "new_length": new_length}

    monkeypatch.setattr(FakeSidecar, "extend_prefix", extend_prefix, raising=False)

    def go(seq_len):
        md = meta(seq_len)
        md._pq_runner = runner
        out = torch.zeros(1, 8, 128)
        return rt.pq_or_dense_forward(impl, layer, torch.zeros(1, 8, 128), torch.zeros(1, 2, 128),
                                      torch.zeros(1, 2, 128), kv_cache, md, out, lambda: out)

    go(500)                                             # prompt of 499 tokens + the first decode token
    go(501)
    # next turn: the old prompt, what was generated, and 100 more tokens; switch still off -> rebuild
    requests["r0"] = types.SimpleNamespace(prompt_token_ids=list(range(499)) + [7] * 101)
    go(601)
    assert FakeSidecar.built == 2 and calls == [] and rt.STATS["prefix_extend_hits"] == 0
    monkeypatch.setenv("PQ_HSA_PREFIX_EXTEND", "1")
    requests["r0"] = types.SimpleNamespace(prompt_token_ids=list(range(499)) + [7] * 101 + [9] * 50)
    assert float(go(651)[0, 0, 0]) == 651.0
    assert FakeSidecar.built == 2 and calls == [(601, 651)]
    assert rt.STATS["prefix_extend_hits"] == 1 and rt.STATS["pq_extend_delta_tokens_total"] == 50
    assert rt.STATS["pq_extend_last"]["new_length"] == 651
    sc = rt.state_for(impl, layer)["sidecar"]
    assert sc.prefix_checkpoint_length == 651           # re-armed for the turn after
    go(652)
    # a prompt that does not start with the checkpointed one
    requests["r0"] = types.SimpleNamespace(prompt_token_ids=[1] * 700)
    go(701)
    assert FakeSidecar.built == 3 and rt.STATS["prefix_extend_rejects"] == {"prefix_digest_mismatch": 1}
    # more than PQ_HSA_PREFIX_EXTEND_MAX_FRAC of the new length would be new
    requests["r0"] = types.SimpleNamespace(prompt_token_ids=[1] * 700 + [2] * 900)
    go(1601)
    assert FakeSidecar.built == 4 and rt.STATS["prefix_extend_rejects"]["delta_too_large"] == 1
    # the sidecar may decline (returns None): rebuild, and say why
    requests["r0"] = types.SimpleNamespace(prompt_token_ids=[1] * 700 + [2] * 900 + [3] * 10)
    rt.state_for(impl, layer)["sidecar"].fail = True
    monkeypatch.setattr(FakeSidecar, "forward", lambda self, q: torch.full((1, self.hq, 128), float(self.length)))
    go(1611)
    assert FakeSidecar.built == 5 and rt.STATS["prefix_extend_rejects"]["adapter_declined"] == 1
    # the pure matcher: remaining reasons
    md = meta(800)
    assert rt.prefix_extend_match(md, None, 500, 800)[:2] == (False, "no_checkpoint")
    assert rt.prefix_extend_match(md, (499, b"x"), 502, 800)[:2] == (False, "checkpoint_inconsistent")
    assert rt.prefix_extend_match(md, (799, b"x"), 800, 800)[:2] == (False, "not_longer")
    assert rt.prefix_extend_match(md, (499, b"x"), 500, 800)[:2] == (False, "no_runner")
    md._pq_runner = types.SimpleNamespace(input_batch=types.SimpleNamespace(req_ids=["r0"]),
                                          requests={"r0": types.SimpleNamespace(prompt_token_ids=[0] * 5)})
    assert rt.prefix_extend_match(md, (499, b"x"), 500, 800)[:2] == (False, "prompt_len_mismatch")


def test_copy_ctx_and_as_decode_qkv():
    out = torch.zeros(2, 8, 128, dtype=torch.bfloat16)
    rt.copy_ctx(out, torch.ones(1, 8 * 128), 1)
    assert float(out[0].sum()) == 8 * 128 and float(out[1].sum()) == 0
    assert rt.as_decode_qkv(torch.zeros(3, 8, 128)).shape == (1, 8, 128)
    assert rt.as_decode_qkv(torch.zeros(3, 128)).shape == (1, 1, 128)
    with pytest.raises(ValueError):
        rt.as_decode_qkv(torch.zeros(128))


def test_write_kv_to_cache_uses_the_slot_mapping():
    cache = torch.zeros(2, 5, 16, 2, 128)
    md = types.SimpleNamespace(slot_mapping=torch.tensor([37]))
    rt.write_kv_to_cache(torch.ones(1, 2, 128), 2 * torch.ones(1, 2, 128), cache, md)
    assert float(cache[0, 2, 5].sum()) == 256 and float(cache[1, 2, 5].sum()) == 512 and float(cache.sum()) == 768


def test_plugin_is_a_noop_unless_enabled_and_config_env_round_trip(clean_runtime, monkeypatch):
    class Impl:
        def forward(self, layer, query, key, value, kv_cache, attn_metadata, output=None, **extra):
            return "dense"

    monkeypatch.delenv("PQ_HSA_VLLM", raising=False)
    plugin.vllm_general_plugin()
    assert plugin.install(impl_cls=Impl) == {"installed": False, "reason": "PQ_HSA_VLLM!=1"}
    assert not getattr(Impl.forward, "_pq_hsa_wrapped", False)
    monkeypatch.setenv("PQ_HSA_VLLM", "1")
    monkeypatch.setenv("PQ_HSA_TOP_FRAC", "0.02")
    res = plugin.install(impl_cls=Impl)
    assert res["installed"] and res["config"]["top_fraction"] == 0.02
    assert "PQ_HSA_TOP_FRAC" not in res["env_defaults_written"]       # explicit value wins
    assert os.environ["PQ_HSA_ENABLE"] == "1" and os.environ["PQ_HSA_LOCAL"] == "128"
    assert os.environ["PQ_HSA_CUDA_SPLITS"] == "8"                     # H20 switches accepted as no-ops
    assert getattr(Impl.forward, "_pq_hsa_wrapped", False)
    assert not wrap.wrap_forward(Impl)                                 # idempotent
    # prefill-like metadata goes to the original forward
    assert Impl().forward(None, None, None, None, None, meta(qlen=7, tokens=7)) == "dense"
    wrap.unwrap_forward(Impl)
    assert not getattr(Impl.forward, "_pq_hsa_wrapped", False)
    cfg = PQHSAConfig(top_fraction=0.05, local_window=64, batch=True)
    env = cfg.as_env()
    assert env["PQ_HSA_TOP_FRAC"] == "0.05" and env["PQ_HSA_LOCAL"] == "64" and env["PQ_HSA_BATCH"] == "1"
    for k in list(os.environ):
        if k.startswith("PQ_HSA_"):
            monkeypatch.delenv(k)
    cfg.apply_env_defaults()
    back = PQHSAConfig.from_env()
    assert (back.top_fraction, back.local_window, back.batch) == (0.05, 64, True)


def test_batched_index_training_equals_the_per_stream_procedure():
    """Streams of one length train together (batched matrix products); with the shared seed the
    result is what one train_ivfpq call per stream gives, including the paths for fewer vectors
    than clusters and for clusters left empty (each stream then draws from its own generator)."""
    from pqhsa_release_amd.index.train import train_ivfpq, train_ivfpq_batched

    gen = torch.Generator().manual_seed(5)
    centers = torch.randn(4, 24, 128, generator=gen)
    pick = torch.randint(0, 24, (4, 1500), generator=gen)
    keys = centers[torch.arange(4)[:, None], pick] + 0.3 * torch.randn(4, 1500, 128, generator=gen)
    for k, lists in ((keys, 32), (keys[:, :12], 32)):   # 12 keys: fewer than the 16 codewords
        coarse, books = train_ivfpq_batched(k, num_lists=lists, coarse_iter=2, pq_iter=3, seed=11)
        assert coarse.shape == (4, min(lists, k.shape[1]), 128) and books.shape == (4, 8, 16, 16)
        for s in range(4):
            c1, b1 = train_ivfpq(k[s], num_lists=lists, coarse_iter=2, pq_iter=3, seed=11)
            torch.testing.assert_close(coarse[s], c1, rtol=0, atol=1e-6)
            torch.testing.assert_close(books[s], b1, rtol=0, atol=1e-6)
    with pytest.raises(ValueError):
        train_ivfpq_batched(keys[:, :0], num_lists=8)


def test_batch_mode_per_request_sidecars(fake_stack, monkeypatch):
    """PQ_HSA_BATCH=1 with PQ_HSA_BATCH_FUSED=0: one sidecar per request, built on first sight,
    appended to while the request advances by one token, rebuilt when it does not."""
    impl, layer, kv_cache = fake_stack
    monkeypatch.setenv("PQ_HSA_ENABLE", "1")
    monkeypatch.setenv("PQ_HSA_BATCH", "1")
    monkeypatch.setenv("PQ_HSA_BATCH_FUSED", "0")

    def batch_step(lens):
        n = len(lens)
        md = meta(seq_len=max(lens), reqs=n, tokens=n)
        md.seq_lens = torch.tensor(lens, dtype=torch.int32)
        out = torch.zeros(n, 8, 128)
        q, k, v = torch.zeros(n, 8, 128), torch.zeros(n, 2, 128), torch.zeros(n, 2, 128)
        return rt.pq_or_dense_forward(impl, layer, q, k, v, kv_cache, md, out, lambda: torch.full((n, 8, 128), -1.0))

    monkeypatch.setattr(rt, "gather_flashattn_kv",
                        lambda kv, md, i=0: (torch.zeros(1, 2, int(md.seq_lens[i]), 128),
                                             torch.zeros(1, 2, int(md.seq_lens[i]), 128), int(md.seq_lens[i])))
    res = batch_step([500, 300, 400])
    assert [float(res[r, 0, 0]) for r in range(3)] == [500.0, 300.0, 400.0] and FakeSidecar.built == 3
    res = batch_step([501, 301, 401])
    assert [float(res[r, 0, 0]) for r in range(3)] == [501.0, 301.0, 401.0] and FakeSidecar.built == 3
    res = batch_step([502, 350])                      # request 1 is a different one now, request 2 left
    assert [float(res[r, 0, 0]) for r in range(2)] == [502.0, 350.0] and FakeSidecar.built == 4
    assert sorted(rt.state_for(impl, layer)["batch"]) == [0, 1]
    assert rt.STATS["pq_batch_steps"] == 3 and rt.STATS["pq_batch_reqs_total"] == 8
    assert rt.STATS["pq_batch_fused_steps"] == 0


def test_device_index_regroup_copies_rows_and_counts():
    """Regrouping picks sequences out of existing indexes: rows, per-list tables, sampled subsets
    and counts follow the sequence; capacity grows to what the caller asks for."""
    from pqhsa_release_amd import ops

    gen = torch.Generator().manual_seed(3)
    def filled(batch, n_cap, counts):
        ix = ops.DeviceIndex(batch, 2, 8, n_cap, "cpu")
        for name in ("codes", "list_ids", "norms", "pos", "coarse", "codebooks", "vbar", "vsum", "vcount",
                     "s_codes", "s_list_ids", "s_norms"):
            t = getattr(ix, name)
            t.copy_((torch.rand(t.shape, generator=gen) * 100).to(t.dtype))
        ix.s_n.copy_(torch.tensor([c // 2 for c in counts], dtype=torch.int32))
        ix.n_sorted_host = [c // 3 for c in counts]
        ix.set_counts(counts)
        return ix

    a, b = filled(3, 64, [40, 10, 64]), filled(1, 200, [150])
    new = ops.DeviceIndex.regroup([(a, 2), (b, 0), (a, 0)], n_cap=100)
    assert new.batch == 3 and new.n_cap >= 150 and new.n_host == [64, 150, 40]
    assert new.n_sorted_host == [21, 50, 13] and new.s_n.tolist() == [32, 75, 20]
    assert new.n_idx.tolist() == [64, 150, 40]
    for dst, (src, seq, n) in enumerate([(a, 2, 64), (b, 0, 150), (a, 0, 40)]):
        rows_new, rows_old = slice(2 * dst, 2 * dst + 2), slice(2 * seq, 2 * seq + 2)
        for name in ("codes", "list_ids", "norms", "pos"):
            assert torch.equal(getattr(new, name)[rows_new, :n], getattr(src, name)[rows_old, :n]), name
        for name in ("coarse", "codebooks", "vbar", "vsum", "vcount"):
            assert torch.equal(getattr(new, name)[rows_new], getattr(src, name)[rows_old]), name
        keep = min(src.s_cap, new.s_cap)
        assert torch.equal(new.s_codes[rows_new, :keep], src.s_codes[rows_old, :keep])
    with pytest.raises(ValueError):
        ops.DeviceIndex.regroup([(a, 0), (ops.DeviceIndex(1, 4, 8, 16, "cpu"), 0)], n_cap=16)


def test_sampled_subset_positions_are_one_per_stratum():
    """DeviceIndex._sample_positions: ascending, distinct, inside [0, n), one per stratum of the
    list-ordered keys; the heads of a sequence share them, sequences and seeds do not."""
    from pqhsa_release_amd.ops import DeviceIndex

    holder = types.SimpleNamespace(device=torch.device("cpu"))
    seqs = torch.tensor([[0], [0], [1]])
    for n, ns in ((131004, 8192), (5000, 1024), (1000, 1000), (4097, 4096)):
        pos = DeviceIndex._sample_positions(holder, n, ns, 0, seqs)
        assert pos.shape == (3, ns) and int(pos.min()) >= 0 and int(pos.max()) < n
        assert bool((pos[:, 1:] > pos[:, :-1]).all())
        i = torch.arange(ns)
        assert bool((pos >= i * n // ns).all()) and bool((pos < (i + 1) * n // ns).all())
        assert torch.equal(pos[0], pos[1])
        if n >= 2 * ns:   # strata of one key leave no choice
            assert not torch.equal(pos[0], pos[2])
            assert not torch.equal(pos[0], DeviceIndex._sample_positions(holder, n, ns, 1, seqs)[0])
    # the places inside the strata are spread: no half of a stratum is favoured
    pos = DeviceIndex._sample_positions(holder, 1 << 20, 8192, 3, seqs[:1])[0]
    inside = (pos - torch.arange(8192) * 128).float() / 128.0
    assert 0.45 < float(inside.mean()) < 0.55 and float(inside.std()) > 0.25


def test_ema_rows_moves_the_rows_that_got_vectors_and_no_others():
    """_ema_rows (the table move of the deferred flush): row j becomes (1 - lr) row + lr * mean of
    the vectors assigned to j; rows without vectors keep their bits (pq.py:117-173)."""
    from pqhsa_release_amd.attention.engine import _ema_rows

    gen = torch.Generator().manual_seed(9)
    table = torch.randn(40, 16, generator=gen)
    vectors = torch.randn(300, 16, generator=gen)
    assign = torch.randint(0, 40, (300,), generator=gen)
    assign[assign == 7] = 8                       # row 7 gets nothing
    before = table.clone()
    _ema_rows(table, vectors, assign, 0.25, 1e-12)
    for j in range(40):
        mine = vectors[assign == j]
        if mine.shape[0] == 0:
            assert torch.equal(table[j], before[j])
        else:
            want = 0.75 * before[j] + 0.25 * (mine.sum(0) / mine.shape[0])
            torch.testing.assert_close(table[j], want, rtol=0, atol=1e-6)
    assert torch.equal(table[7], before[7])


def test_bench_passes_counter_traffic_on_only_for_the_kernels_it_was_measured_on(tmp_path, monkeypatch):
    """bench.py's roofline objects carry the HBM bytes per launch from the committed counter runs only
    while the kernel sources are the ones the counters were taken on (a digest in the file)."""
    import json

    import bench

    digest = bench.kernel_sources_digest()
    assert len(digest) == 64 and digest == bench.kernel_sources_digest()
    rec = {"commit": "abc1234", "sources_sha256": digest, "bytes_per_launch": {"attend": 123, "scan_emit": 45}}
    path = tmp_path / "decode_step_cfg{cfg}_hbm_traffic.json"
    (tmp_path / "decode_step_cfg7_hbm_traffic.json").write_text(json.dumps(rec))
    monkeypatch.setattr(bench, "TRAFFIC_FILE", str(path))
    assert bench.measured_traffic(7, "attend") == (123, "abc1234")
    assert bench.measured_traffic(7, "scan_emit") == (45, "abc1234")
    assert bench.measured_traffic(7, "lut_build") == (None, None)          # no figure for this kernel
    assert bench.measured_traffic(8, "attend") == (None, None)             # no file for this configuration
    rec["sources_sha256"] = "0" * 64                                        # measured on other kernels
    (tmp_path / "decode_step_cfg7_hbm_traffic.json").write_text(json.dumps(rec))
    assert bench.measured_traffic(7, "attend") == (None, "abc1234")
