"""The dense twin of ToyNSALlama: same decoder with SelfAttention layers and plain KV caches.  Counterpart of
native_sparse_attention/model/toy_llama.py:22-240 of the reference (same config fields, module and parameter names)."""
from dataclasses import dataclass, field
from typing import List, Optional

import torch
import torch.nn as nn

from ..module import KVCache, RopeConfig, SelfAttention
from .toy_nsa_llama import FFN, InferenceConfig, RMSNorm, _llama3_scaling


@dataclass
class ToyLlamaConfig:
    vocab_size: int = 128288
    max_position_embeddings: int = 131072
    hidden_size: int = 4096
    intermediate_size: int = 14336
    num_hidden_layers: int = 32
    num_attention_heads: int = 32
    num_key_value_heads: int = 2
    head_dim: int = 128
    rope_theta: float = 500000.0
    rope_scaling: dict = field(default_factory=_llama3_scaling)


class ToyLlamaLayer(nn.Module):
    def __init__(self, hidden_size: int, intermediate_size: int, num_q_heads: int, num_kv_heads: int, head_dim: int,
                 rope_config: RopeConfig, rope_device: str = "cuda"):
        super().__init__()
        self.attn_norm = RMSNorm(hidden_size)
        self.self_attn = SelfAttention(hidden_size, num_q_heads, num_kv_heads, head_dim, rope_config, rope_device)
        self.ffn_norm = RMSNorm(hidden_size)
        self.ffn = FFN(hidden_size, intermediate_size)

    def forward(self, x, cu_seqlens):
        x = x + self.self_attn(self.attn_norm(x), cu_seqlens)
        return x + self.ffn(self.ffn_norm(x))

    @torch.no_grad()
    def inference(self, x, cu_seqlens, step, kv_cache):
        x = x + self.self_attn.inference(self.attn_norm(x), cu_seqlens, step, kv_cache)
        return x + self.ffn(self.ffn_norm(x))


class ToyLlama(nn.Module):
    def __init__(self, config: ToyLlamaConfig, inference_config: Optional[InferenceConfig] = None, device: str = "cuda"):
        super().__init__()
        self.config = c = config
        self.embedding = nn.Embedding(c.vocab_size, c.hidden_size)
        self.rope_config = RopeConfig(c.max_position_embeddings, c.head_dim, c.rope_theta, c.rope_scaling)
        self.layers = nn.ModuleList([
            ToyLlamaLayer(c.hidden_size, c.intermediate_size, c.num_attention_heads, c.num_key_value_heads, c.head_dim,
                          RopeConfig(c.max_position_embeddings, c.head_dim, c.rope_theta, c.rope_scaling), rope_device=device)
            for _ in range(c.num_hidden_layers)])
        self.norm = RMSNorm(c.hidden_size)
        self.lm_head = nn.Linear(c.hidden_size, c.vocab_size, bias=False)
        self.inference_config = inference_config
        self.kv_cache: Optional[List[KVCache]] = None
        self._device = device

    def forward(self, input_ids: torch.LongTensor, cu_seqlens: torch.LongTensor):
        x = self.embedding(input_ids).to(torch.bfloat16)
        for layer in self.layers:
            x = layer(x, cu_seqlens)
        return self.lm_head(self.norm(x)).to(torch.float32)

    @torch.no_grad()
    def inference(self, input_ids: torch.LongTensor, cu_seqlens: torch.LongTensor, step: int):
        if self.kv_cache is None:
            ic, c = self.inference_config, self.config
            self.kv_cache = [KVCache(ic.max_batch_size, ic.max_length, c.num_key_value_heads, c.head_dim, torch.bfloat16, self._device)
                             for _ in range(c.num_hidden_layers)]
        x = self.embedding(input_ids).to(torch.bfloat16)
        for layer, cache in zip(self.layers, self.kv_cache):
            x = layer.inference(x, cu_seqlens, step, cache)
        x = self.norm(x)
        if step == 0:
            x = x[cu_seqlens[1:].long() - 1]
        return self.lm_head(x).to(torch.float32)

    def generate(self, input_ids: torch.LongTensor, cu_seqlens: torch.LongTensor, max_new_tokens: int = -1):
        if max_new_tokens <= 0:
            max_new_tokens = self.inference_config.max_new_tokens
        out = []
        for step in range(max_new_tokens):
            input_ids = torch.argmax(self.inference(input_ids, cu_seqlens, step), dim=-1)
            out.append(input_ids)
        return torch.stack(out, dim=1)
