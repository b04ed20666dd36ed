"""Import path of the reference's ops/triton/flash_attention_decode.py:142-217; the names below are this package's gfx950 implementations
(no Triton is involved: only the module path is kept so that existing imports resolve)."""
from ..decode import (  # noqa: F401
    flash_attention_decode,
)

__all__ = ["flash_attention_decode"]
