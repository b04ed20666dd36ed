"""Dense causal self-attention layer with rotary embedding and a KV cache: the baseline the reference compares the
sparse layer with.  Counterpart of native_sparse_attention/module/self_attention.py:22-175 (same constructor,
parameter names and calls); the attention itself runs on this package's flash_attention_varlen and
flash_attention_decode instead of the third-party flash-attn kernels the reference imports."""
import torch

from ..ops import flash_attention_decode, flash_attention_varlen
from .kv_cache import KVCache
from .rope import RopeConfig, RotaryEmbedding


class SelfAttention(torch.nn.Module):
    def __init__(self, hidden_size: int, num_q_heads: int, num_kv_heads: int, head_dim: int, rope_config: RopeConfig,
                 rope_device: str = "cuda"):
        super().__init__()
        self.hidden_size, self.num_q_heads, self.num_kv_heads, self.head_dim = hidden_size, num_q_heads, num_kv_heads, head_dim
        self.rope_config = rope_config
        assert self.head_dim == self.rope_config.head_dim
        self.proj_q = torch.nn.Linear(hidden_size, num_q_heads * head_dim, bias=False)
        self.proj_k = torch.nn.Linear(hidden_size, num_kv_heads * head_dim, bias=False)
        self.proj_v = torch.nn.Linear(hidden_size, num_kv_heads * head_dim, bias=False)
        self.proj_o = torch.nn.Linear(num_q_heads * head_dim, hidden_size, bias=False)
        self.rope = RotaryEmbedding(rope_config, device=rope_device)
        self.init_params()

    def init_params(self):
        for p in self.parameters():
            torch.nn.init.xavier_uniform_(p)

    def _qkv(self, x):
        return (self.proj_q(x).view(-1, self.num_q_heads, self.head_dim), self.proj_k(x).view(-1, self.num_kv_heads, self.head_dim),
                self.proj_v(x).view(-1, self.num_kv_heads, self.head_dim))

    def forward(self, x: torch.Tensor, cu_seqlens: torch.Tensor):
        """x [total_len, hidden_size] (bf16/fp16), cu_seqlens [batch + 1] -> [total_len, hidden_size]."""
        assert x.dtype == torch.bfloat16 or x.dtype == torch.float16
        assert x.shape[-1] == self.hidden_size
        cu_seqlens = cu_seqlens.to(torch.int32)
        q, k, v = self._qkv(x)
        q, k = self.rope(q, cu_seqlens), self.rope(k, cu_seqlens)
        out = flash_attention_varlen(q, k, v, cu_seqlens, cu_seqlens, 0, 0, causal=True)
        return self.proj_o(out.reshape(-1, self.num_q_heads * self.head_dim))

    @torch.no_grad()
    def inference(self, x: torch.Tensor, cu_seqlens: torch.Tensor, step: int, cache: KVCache):
        """step == 0: prefill of x [total_len, hidden]; step > 0: one new token per sequence, x [batch, hidden]."""
        assert x.dtype == torch.bfloat16 or x.dtype == torch.float16
        assert x.shape[-1] == self.hidden_size and step >= 0
        cu_seqlens = cu_seqlens.to(torch.int32)
        batch = cu_seqlens.shape[0] - 1
        assert x.shape[0] == (cu_seqlens[-1] if step == 0 else batch)
        q, k, v = self._qkv(x)
        if step == 0:
            q, k = self.rope(q, cu_seqlens, step), self.rope(k, cu_seqlens, step)
            cache.reset()
            cache.update_kv(cu_seqlens, step, k, v)
            out = flash_attention_varlen(q, k, v, cu_seqlens, cu_seqlens, 0, 0, causal=True)
        else:
            # the new token's position is the cache length, read on the device
            q, k = self.rope.rotate_at(q, cache.kv_len[:batch]), self.rope.rotate_at(k, cache.kv_len[:batch])
            cache.update_kv(cu_seqlens, step, k, v)
            out = flash_attention_decode(q, cache.kv_cache[0, :batch], cache.kv_cache[1, :batch], cache.kv_len[:batch])
        return self.proj_o(out.reshape(-1, self.num_q_heads * self.head_dim))
