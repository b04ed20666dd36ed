from ..utils import get_compressed_seqlens  # noqa: F401
