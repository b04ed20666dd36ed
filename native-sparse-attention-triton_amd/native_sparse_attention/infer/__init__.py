from .nsa_inference import nsa_infer  # noqa: F401
