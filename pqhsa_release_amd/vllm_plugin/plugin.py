"""``vllm.general_plugins`` entry point (pq_hsa_vllm/src/pq_hsa_vllm/plugin.py:57-97 of the
reference): a no-op unless ``PQ_HSA_VLLM=1``; otherwise applies the config's environment
defaults and wraps ``FlashAttentionImpl.forward``.  Register it as
``pq_hsa_vllm = "pqhsa_release_amd.vllm_plugin.plugin:vllm_general_plugin"``."""

from __future__ import annotations

import os
from typing import Any, Optional

from .config import PQHSAConfig

_INSTALLED = False


def enabled() -> bool:
    return os.environ.get("PQ_HSA_VLLM", "0") == "1"


def install(rank: Optional[int] = None, *, force: bool = False, config: Optional[PQHSAConfig] = None,
            impl_cls=None) -> dict[str, Any]:
    """Idempotent per process.  ``impl_cls`` lets a caller wrap an attention implementation class
    other than vLLM's (any class with the FlashAttentionImpl.forward signature)."""
    global _INSTALLED
    if not force and not enabled():
        return {"installed": False, "reason": "PQ_HSA_VLLM!=1"}
    cfg = config or PQHSAConfig.from_env()
    written = cfg.apply_env_defaults()
    from ..vllm_backend import pq_hsa_flashattn_wrap as wrap

    if impl_cls is not None:
        wrap.wrap_forward(impl_cls)
    else:
        wrap.install_pq_hsa_flashattn_backend()
    _INSTALLED = True
    return {"installed": True, "rank": rank, "config": cfg.asdict(), "env_defaults_written": sorted(written)}


def vllm_general_plugin() -> None:
    if not enabled():
        return
    install()


__all__ = ["vllm_general_plugin", "install", "enabled", "PQHSAConfig"]
