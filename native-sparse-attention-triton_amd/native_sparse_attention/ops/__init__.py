"""Drop-in operator surface of native_sparse_attention.ops, backed by libnsa_hip.so."""
from .weighted_pool import avgpool_compress, weightedpool_compress  # noqa: F401
from .linear_compress import linear_compress  # noqa: F401
from .flash_attention import flash_attention_varlen  # noqa: F401
from .compressed_attention import compressed_attention  # noqa: F401
from .topk_sparse_attention import topk_sparse_attention  # noqa: F401
from .decode import (  # noqa: F401
    compressed_attention_decode,
    flash_attention_decode,
    topk_sparse_attention_decode,
)

__all__ = [
    "avgpool_compress",
    "weightedpool_compress",
    "linear_compress",
    "flash_attention_varlen",
    "compressed_attention",
    "topk_sparse_attention",
    "flash_attention_decode",
    "compressed_attention_decode",
    "topk_sparse_attention_decode",
]
