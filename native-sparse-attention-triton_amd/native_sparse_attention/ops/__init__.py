"""Drop-in operator surface of native_sparse_attention.ops, backed by libnsa_hip.so."""
from .weighted_pool import avgpool_compress, weightedpool_compress  # noqa: F401
from .topk_sparse_attention import topk_sparse_attention  # noqa: F401

__all__ = [
    "avgpool_compress",
    "weightedpool_compress",
    "topk_sparse_attention",
]
