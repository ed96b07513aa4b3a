"""Configuration records of the PQ-HSA decode path.

Field names and defaults follow the reference's ``IVFPQConfig``
(pq_hsa/index/ivfpq.py:83-101) and ``SparseAttentionConfig``
(pq_hsa/attention/sparse_attention.py:14-37) so that existing call sites construct them
unchanged.  The MI355X kernels implement the decode hot path only — hybrid mode with the
per-list centroid background, all-PQ top-k, exact rerank, 8 x 4-bit residual PQ on the
direction-normalised keys — and ``validate_for_kernels`` says so loudly for anything else.
"""

from __future__ import annotations

from dataclasses import dataclass

ALLOWED_KERNEL_BACKENDS = frozenset({"auto", "torch", "triton", "h20", "mi355x"})


@dataclass(slots=True)
class IVFPQConfig:
    num_lists: int = 256
    nprobe: int = 8
    num_subspaces: int = 16
    num_bits: int = 8
    residual: bool = True
    coarse_max_iter: int = 30
    pq_max_iter: int = 25
    pack_codes: bool = True
    topk_block_size: int | None = None
    kernel_backend: str = "auto"
    rotation: str = "none"
    direction_normalize: bool = False
    online_codebook_lr: float = 0.05
    seed: int = 0
    eps: float = 1e-12


@dataclass(slots=True)
class SparseAttentionConfig:
    sink_tokens: int = 0
    local_window: int = 0
    retrieval_topk: int = 100
    retrieval_top_fraction: float | None = None
    retrieval_top_p: float | None = None
    retrieval_top_p_scope: str = "retrieval"
    nprobe: int | None = None
    candidate_budget: int | None = None
    exact_rerank: bool = True
    scale: float | None = None
    mode: str = "sparse"
    hybrid_value_mode: str = "denominator"
    hybrid_topk_source: str = "all_pq"
    hybrid_denominator_source: str = "all_pq"
    index_update_interval: int = 1
    index_update_strategy: str = "incremental"
    codebook_refresh_interval: int | None = None
    kv_storage: str = "device"
    pin_offloaded_kv: bool = False
    prefetch_full_kv: bool = False
    collect_attention_details: bool = True
    profile_attention_components: bool = False


def validate_for_kernels(index_config: IVFPQConfig, attention_config: SparseAttentionConfig) -> None:
    """Reject configurations outside the path the HIP kernels implement (``ValueError``, the
    reference's convention for configuration mismatches, sparse_attention.py:98-163)."""
    ic, ac = index_config, attention_config
    if ic.kernel_backend not in ALLOWED_KERNEL_BACKENDS:
        raise ValueError("kernel_backend must be 'auto', 'torch', 'triton', 'h20' or 'mi355x'")
    if ic.num_subspaces != 8 or ic.num_bits != 4:
        raise ValueError("the MI355X kernels implement 8 subspaces x 4 bits; got "
                         f"{ic.num_subspaces} x {ic.num_bits}")
    if not ic.residual or not ic.direction_normalize or ic.rotation != "none" or not ic.pack_codes:
        raise ValueError("the MI355X kernels need residual=True, direction_normalize=True, rotation='none', "
                         "pack_codes=True")
    if ic.num_lists < 1 or ic.num_lists > 4096:
        raise ValueError("num_lists must be in [1, 4096]")
    if ac.mode != "hybrid" or ac.hybrid_value_mode != "centroid":
        raise ValueError("the MI355X kernels implement mode='hybrid' with hybrid_value_mode='centroid'")
    if ac.hybrid_topk_source != "all_pq" or ac.hybrid_denominator_source != "all_pq":
        raise ValueError("the MI355X kernels implement hybrid_topk_source = hybrid_denominator_source = 'all_pq'")
    if not ac.exact_rerank:
        raise ValueError("the MI355X kernels implement exact_rerank=True")
    if ac.retrieval_top_p is not None:
        raise ValueError("retrieval_top_p is not implemented by the MI355X kernels")
    if ac.retrieval_top_fraction is not None and not (0.0 < ac.retrieval_top_fraction <= 1.0):
        raise ValueError("retrieval_top_fraction must be in (0, 1]")
    if ac.sink_tokens < 0 or ac.local_window < 0:
        raise ValueError("sink_tokens and local_window must be non-negative")
    if ac.index_update_interval <= 0:
        raise ValueError("index_update_interval must be positive")
    if ac.index_update_strategy not in {"incremental", "online", "rebuild", "deferred"}:
        raise ValueError("index_update_strategy must be 'incremental', 'online', 'rebuild', or 'deferred'")
    if ac.codebook_refresh_interval is not None:
        raise ValueError("codebook_refresh_interval is not implemented by the MI355X path")
    if ac.kv_storage != "device":
        raise ValueError("kv_storage must be 'device' (CPU offload is outside the decode kernel path)")
