from .toy_nsa_llama import FFN, InferenceConfig, RMSNorm, ToyNSALlama, ToyNSALlamaConfig, ToyNSALlamaLayer  # noqa: F401

__all__ = ["ToyNSALlamaConfig", "InferenceConfig", "ToyNSALlama"]
