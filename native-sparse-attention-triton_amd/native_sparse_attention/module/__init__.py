from .kv_cache import KVCache, NSACache  # noqa: F401
from .rope import RopeConfig, RotaryEmbedding  # noqa: F401
from .self_attention import SelfAttention  # noqa: F401
from .native_sparse_attention import NativeSparseAttention  # noqa: F401

__all__ = ["SelfAttention", "NativeSparseAttention", "RotaryEmbedding", "RopeConfig", "NSACache", "KVCache"]
