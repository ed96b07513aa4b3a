"""Install the PQ-HSA decode hook over ``FlashAttentionImpl.forward``.

Same monkey-patch as the reference's benchmarks/vllm_backend/pq_hsa_flashattn_wrap.py:41-97: the
wrapped ``forward(self, layer, query, key, value, kv_cache, attn_metadata, output=None, **extra)``
hands single-token decode steps to ``pq_or_dense_forward`` and everything else to the original.
``wrap_forward`` works on any class with that signature (vLLM itself is only imported by
``install_pq_hsa_flashattn_backend``).
"""

from __future__ import annotations

from . import pq_hsa_decode_runtime as runtime


def wrap_forward(impl_cls) -> bool:
    """Patch ``impl_cls.forward`` in place; returns False when it is already wrapped."""
    orig = impl_cls.forward
    if getattr(orig, "_pq_hsa_wrapped", False):
        return False

    def forward(self, layer, query, key, value, kv_cache, attn_metadata, output=None, **extra):
        def dense():
            return orig(self, layer, query, key, value, kv_cache, attn_metadata, output=output, **extra)

        return runtime.pq_or_dense_forward(self, layer, query, key, value, kv_cache, attn_metadata, output, dense)

    forward._pq_hsa_wrapped = True  # type: ignore[attr-defined]
    forward._pq_hsa_original = orig  # type: ignore[attr-defined]
    impl_cls.forward = forward
    runtime.STATS["installed"] = True
    runtime.STATS["backend"] = "flashattn_wrap"
    return True


def unwrap_forward(impl_cls) -> None:
    orig = getattr(impl_cls.forward, "_pq_hsa_original", None)
    if orig is not None:
        impl_cls.forward = orig
        runtime.STATS["installed"] = False


def install_pq_hsa_flashattn_backend() -> bool:
    try:
        from vllm.v1.attention.backends.flash_attn import FlashAttentionImpl
    except ImportError as exc:  # vLLM is not part of this package
        raise RuntimeError("vLLM is not importable: cannot wrap FlashAttentionImpl.forward") from exc
    return wrap_forward(FlashAttentionImpl)
