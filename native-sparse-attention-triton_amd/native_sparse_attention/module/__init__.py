from .kv_cache import NSACache  # noqa: F401
from .rope import RopeConfig, RotaryEmbedding  # noqa: F401
from .native_sparse_attention import NativeSparseAttention  # noqa: F401

__all__ = ["NativeSparseAttention", "RotaryEmbedding", "RopeConfig", "NSACache"]
