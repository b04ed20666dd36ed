from .nsa_inference import nsa_infer  # noqa: F401
from .decode_graph import NSADecodeGraph  # noqa: F401
