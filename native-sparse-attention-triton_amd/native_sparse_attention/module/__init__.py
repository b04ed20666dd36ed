from .kv_cache import NSACache  # noqa: F401
