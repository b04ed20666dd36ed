"""Import path of the reference's ops/triton/weighted_pool.py:301-363; the names below are this package's gfx950 implementations
(no Triton is involved: only the module path is kept so that existing imports resolve)."""
from ..weighted_pool import (  # noqa: F401
    weightedpool_compress,
    avgpool_compress,
)

__all__ = ["weightedpool_compress", "avgpool_compress"]
