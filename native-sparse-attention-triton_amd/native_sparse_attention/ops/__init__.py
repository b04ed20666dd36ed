"""Drop-in operator surface of native_sparse_attention.ops, backed by libnsa_hip.so."""
from .topk_sparse_attention import topk_sparse_attention  # noqa: F401

__all__ = [
    "topk_sparse_attention",
]
