"""MI355X-native PQ-HSA single-token decode attention (hand-written HIP kernels behind a C ABI)."""

from .config import IVFPQConfig, SparseAttentionConfig  # noqa: F401
from .index.packing import pack_4bit_codes, unpack_4bit_codes  # noqa: F401

__all__ = ["IVFPQConfig", "SparseAttentionConfig", "pack_4bit_codes", "unpack_4bit_codes"]
