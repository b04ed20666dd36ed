"""Import path of the reference's ops/triton/flash_attention.py:563-935; the names below are this package's gfx950 implementations
(no Triton is involved: only the module path is kept so that existing imports resolve)."""
from ..flash_attention import (  # noqa: F401
    flash_attention_varlen,
    _flash_attention_fwd,
    _flash_attention_bwd,
)

__all__ = ["flash_attention_varlen", "_flash_attention_fwd", "_flash_attention_bwd"]
