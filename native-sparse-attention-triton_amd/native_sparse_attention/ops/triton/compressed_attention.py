"""Import path of the reference's ops/triton/compressed_attention.py:538-1292; the names below are this package's gfx950 implementations
(no Triton is involved: only the module path is kept so that existing imports resolve)."""
from ..compressed_attention import (  # noqa: F401
    compressed_attention,
    _compressed_attention_fwd,
    _compressed_attention_bwd,
)

__all__ = ["compressed_attention", "_compressed_attention_fwd", "_compressed_attention_bwd"]
