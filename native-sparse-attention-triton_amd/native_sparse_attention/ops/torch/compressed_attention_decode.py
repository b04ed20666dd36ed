"""Import path of the reference's ops/torch/compressed_attention_decode.py:65-193; the name below is this package's gfx950
implementation (same arguments and results; only the module path is kept so that existing imports resolve)."""
from ..decode import (  # noqa: F401
    compressed_attention_decode,
)

__all__ = ["compressed_attention_decode"]
