"""A small Llama-style decoder whose attention is the NativeSparseAttention layer: embedding, pre-norm
blocks (RMSNorm -> NSA -> residual, RMSNorm -> SwiGLU FFN -> residual), final norm and LM head, with a
training `forward`, a cached `inference` step and greedy `generate`.

Counterpart of native_sparse_attention/model/toy_nsa_llama.py:22-277 of the reference (same config
fields, module and parameter names, call signatures), built on this package's layer, cache and kernels.
"""
from dataclasses import dataclass, field
from typing import List, Optional

import torch
import torch.nn as nn

from ..module import NativeSparseAttention, NSACache, RopeConfig


def _llama3_scaling():
    return {"factor": 8.0, "high_freq_factor": 4.0, "low_freq_factor": 1.0, "original_max_position_embeddings": 8192,
            "rope_type": "llama3"}


@dataclass
class ToyNSALlamaConfig:
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
    compress_type: str = "weightedpool"
    kernel_size: int = 32
    kernel_stride: int = 16
    block_size: int = 64
    topk: int = 16
    init_blocks: int = 1
    local_blocks: int = 2
    window_size: int = 512


@dataclass
class InferenceConfig:
    max_batch_size: int = 32
    max_length: int = 8192
    max_new_tokens: int = 128


class RMSNorm(nn.Module):
    """weight * x / sqrt(mean(x^2) + eps), statistics in fp32 (toy_nsa_llama.py:65-76)."""

    def __init__(self, hidden_size: int, eps: float = 1e-6):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size))
        self.variance_epsilon = eps

    def forward(self, hidden_states: torch.Tensor):
        x32 = hidden_states.to(torch.float32)
        x32 = x32 * torch.rsqrt(x32.pow(2).mean(-1, keepdim=True) + self.variance_epsilon)
        return self.weight * x32.to(hidden_states.dtype)


class FFN(nn.Module):
    """down(silu(gate(x)) * up(x)) (toy_nsa_llama.py:79-91)."""

    def __init__(self, hidden_size: int, intermediate_size: int):
        super().__init__()
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.gate_proj = nn.Linear(hidden_size, intermediate_size, bias=False)
        self.up_proj = nn.Linear(hidden_size, intermediate_size, bias=False)
        self.down_proj = nn.Linear(intermediate_size, hidden_size, bias=False)
        self.act_fn = nn.SiLU()

    def forward(self, x):
        return self.down_proj(self.act_fn(self.gate_proj(x)) * self.up_proj(x))


class ToyNSALlamaLayer(nn.Module):
    def __init__(self, hidden_size: int, intermediate_size: int, num_q_heads: int, num_kv_heads: int, head_dim: int,
                 compress_type: str, kernel_size: int, kernel_stride: int, block_size: int, topk: int, init_blocks: int,
                 local_blocks: int, window_size: int, rope_config: RopeConfig, rope_device: str = "cuda"):
        super().__init__()
        self.attn_norm = RMSNorm(hidden_size)
        self.nsa = NativeSparseAttention(
            compress_type=compress_type, hidden_size=hidden_size, num_q_heads=num_q_heads, num_kv_heads=num_kv_heads,
            head_dim=head_dim, kernel_size=kernel_size, kernel_stride=kernel_stride, block_size=block_size, topk=topk,
            init_blocks=init_blocks, local_blocks=local_blocks, window_size=window_size, rope_config=rope_config,
            rope_device=rope_device)
        self.ffn_norm = RMSNorm(hidden_size)
        self.ffn = FFN(hidden_size, intermediate_size)

    def forward(self, x, cu_seqlens):
        x = x + self.nsa(self.attn_norm(x), cu_seqlens)
        return x + self.ffn(self.ffn_norm(x))

    @torch.no_grad()
    def inference(self, x, cu_seqlens, step, kv_cache):
        x = x + self.nsa.inference(self.attn_norm(x), cu_seqlens, step, kv_cache)
        return x + self.ffn(self.ffn_norm(x))


class ToyNSALlama(nn.Module):
    def __init__(self, config: ToyNSALlamaConfig, inference_config: Optional[InferenceConfig] = None, device: str = "cuda"):
        super().__init__()
        self.config = config
        c = config
        self.embedding = nn.Embedding(c.vocab_size, c.hidden_size)
        self.rope_config = RopeConfig(c.max_position_embeddings, c.head_dim, c.rope_theta, c.rope_scaling)
        self.layers = nn.ModuleList([
            ToyNSALlamaLayer(c.hidden_size, c.intermediate_size, c.num_attention_heads, c.num_key_value_heads, c.head_dim,
                             c.compress_type, c.kernel_size, c.kernel_stride, c.block_size, c.topk, c.init_blocks, c.local_blocks,
                             c.window_size, RopeConfig(c.max_position_embeddings, c.head_dim, c.rope_theta, c.rope_scaling),
                             rope_device=device)
            for _ in range(c.num_hidden_layers)])
        self.norm = RMSNorm(c.hidden_size)
        self.lm_head = nn.Linear(c.hidden_size, c.vocab_size, bias=False)
        self.inference_config = inference_config
        self.kv_cache: Optional[List[NSACache]] = None
        self._device = device

    def forward(self, input_ids: torch.LongTensor, cu_seqlens: torch.LongTensor):
        """input_ids [total_len] (varlen, sequences back to back), cu_seqlens [batch + 1] -> logits fp32 [total_len, vocab]."""
        x = self.embedding(input_ids).to(torch.bfloat16)
        for layer in self.layers:
            x = layer(x, cu_seqlens)
        return self.lm_head(self.norm(x)).to(torch.float32)

    @torch.no_grad()
    def inference(self, input_ids: torch.LongTensor, cu_seqlens: torch.LongTensor, step: int):
        """step 0: input_ids [total_len] is the prompt batch; step > 0: input_ids [batch], one new token per sequence.
        Returns the logits of the last position of every sequence, fp32 [batch, vocab]."""
        if self.kv_cache is None:
            ic, c = self.inference_config, self.config
            self.kv_cache = [NSACache(ic.max_batch_size, ic.max_length, c.num_key_value_heads, c.head_dim, c.kernel_size,
                                      c.kernel_stride, c.window_size, torch.bfloat16, self._device)
                             for _ in range(c.num_hidden_layers)]
        x = self.embedding(input_ids).to(torch.bfloat16)
        for layer, cache in zip(self.layers, self.kv_cache):
            x = layer.inference(x, cu_seqlens, step, cache)
        x = self.norm(x)
        if step == 0:
            x = x[cu_seqlens[1:].long() - 1]
        return self.lm_head(x).to(torch.float32)

    def generate(self, input_ids: torch.LongTensor, cu_seqlens: torch.LongTensor, max_new_tokens: int = -1):
        """Greedy decoding; returns the new tokens [batch, max_new_tokens]."""
        if max_new_tokens <= 0:
            max_new_tokens = self.inference_config.max_new_tokens
        out = []
        for step in range(max_new_tokens):
            input_ids = torch.argmax(self.inference(input_ids, cu_seqlens, step), dim=-1)
            out.append(input_ids)
        return torch.stack(out, dim=1)
