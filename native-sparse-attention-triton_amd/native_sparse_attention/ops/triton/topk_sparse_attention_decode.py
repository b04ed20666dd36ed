"""Import path of the reference's ops/triton/topk_sparse_attention_decode.py:151-237; the names below are this package's gfx950 implementations
(no Triton is involved: only the module path is kept so that existing imports resolve)."""
from ..decode import (  # noqa: F401
    topk_sparse_attention_decode,
)

__all__ = ["topk_sparse_attention_decode"]
