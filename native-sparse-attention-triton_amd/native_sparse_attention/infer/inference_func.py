"""Import path of the reference's per-branch inference functions (infer/inference_func.py:27-202): compress_infer,
compressed_attention_infer, topk_sparse_attention_infer and sliding_window_attention_infer, with the reference's
argument order.  They live next to nsa_infer in nsa_inference.py; this module only keeps the old path resolving."""
from .nsa_inference import (  # noqa: F401
    compress_infer,
    compressed_attention_infer,
    sliding_window_attention_infer,
    topk_sparse_attention_infer,
)

__all__ = ["compress_infer", "compressed_attention_infer", "topk_sparse_attention_infer", "sliding_window_attention_infer"]
