"""Import path of the reference's ops/triton/topk_sparse_attention.py:828-1217; the names below are this package's gfx950 implementations
(no Triton is involved: only the module path is kept so that existing imports resolve)."""
from ..topk_sparse_attention import (  # noqa: F401
    topk_sparse_attention,
    _topk_sparse_attention_fwd,
    _topk_sparse_attention_bwd,
)

__all__ = ["topk_sparse_attention", "_topk_sparse_attention_fwd", "_topk_sparse_attention_bwd"]
