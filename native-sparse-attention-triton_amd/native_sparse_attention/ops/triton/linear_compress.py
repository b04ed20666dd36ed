"""Import path of the reference's ops/triton/linear_compress.py:497-525; the names below are this package's gfx950 implementations
(no Triton is involved: only the module path is kept so that existing imports resolve)."""
from ..linear_compress import (  # noqa: F401
    linear_compress,
)

__all__ = ["linear_compress"]
