from .toy_llama import ToyLlama, ToyLlamaConfig, ToyLlamaLayer  # noqa: F401
from .toy_nsa_llama import FFN, InferenceConfig, RMSNorm, ToyNSALlama, ToyNSALlamaConfig, ToyNSALlamaLayer  # noqa: F401

__all__ = ["ToyLlamaConfig", "ToyNSALlamaConfig", "InferenceConfig", "ToyLlama", "ToyNSALlama"]
