from .decode_adapter import (  # noqa: F401
    DecodeAttentionOutput,
    GQAIVFPQDecodeAttentionAdapter,
    IVFPQDecodeAttentionAdapter,
    MultiHeadAttentionOutput,
)
from .engine import PQHSAEngine  # noqa: F401
