"""Native sparse attention layer: projections, key/value compression, the three attention branches and
the gated sum, for training (`forward`) and cached inference (`inference`).

Counterpart of native_sparse_attention/module/native_sparse_attention.py:45-287 of the reference, with the
same constructor arguments, parameter names and call signatures, so that a state dict moves across
unchanged.  The sliding-window branch, which the reference hands to the third-party
flash_attn_varlen_func (:213-223), runs on this package's own window kernels.
"""
import torch

from ..infer import nsa_infer
from ..ops import avgpool_compress, compressed_attention, linear_compress, topk_sparse_attention, weightedpool_compress
from ..ops.gated_sum import gated_sum
from ..ops.sliding_window import sliding_window_attention_varlen
from .kv_cache import NSACache
from .rope import RopeConfig, RotaryEmbedding

COMPRESS_TYPE_TO_FUNC = {
    "avgpool": avgpool_compress,
    "weightedpool": weightedpool_compress,
    "linear": linear_compress,
}

COMPRESS_TYPE_TO_WEIGHT = {
    "avgpool": lambda num_heads, head_dim, kernel_size: None,
    "weightedpool": lambda num_heads, head_dim, kernel_size: torch.nn.Parameter(torch.zeros(num_heads, kernel_size)),
    "linear": lambda num_heads, head_dim, kernel_size: torch.nn.Parameter(torch.zeros(num_heads, head_dim * kernel_size, head_dim)),
}


class NativeSparseAttention(torch.nn.Module):
    """Arguments as in the reference (native_sparse_attention.py:45-81): compress_type in
    {'linear', 'avgpool', 'weightedpool'}; block_size / topk / init_blocks / local_blocks steer the
    selected branch, window_size the sliding-window branch; rope_device is where inv_freq lives."""

    def __init__(self, compress_type: str, hidden_size: int, num_q_heads: int, num_kv_heads: int, head_dim: int, kernel_size: int,
                 kernel_stride: int, block_size: int, topk: int, init_blocks: int, local_blocks: int, window_size: int,
                 rope_config: RopeConfig, rope_device: str = "cuda"):
        super().__init__()
        self.compress_type = compress_type
        self.hidden_size = hidden_size
        self.num_q_heads = num_q_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.kernel_size = kernel_size
        self.kernel_stride = kernel_stride
        self.block_size = block_size
        self.topk = topk
        self.init_blocks = init_blocks
        self.local_blocks = local_blocks
        self.window_size = window_size
        self.rope_config = rope_config
        assert self.head_dim == self.rope_config.head_dim

        self.proj_q = torch.nn.Linear(hidden_size, num_q_heads * head_dim, bias=False)
        self.proj_k = torch.nn.Linear(hidden_size, num_kv_heads * head_dim, bias=False)
        self.proj_v = torch.nn.Linear(hidden_size, num_kv_heads * head_dim, bias=False)
        self.proj_o = torch.nn.Linear(num_q_heads * head_dim, hidden_size, bias=False)

        self.compress_func = COMPRESS_TYPE_TO_FUNC[compress_type]
        self.compress_key = COMPRESS_TYPE_TO_WEIGHT[compress_type](num_kv_heads, head_dim, kernel_size)
        self.compress_value = COMPRESS_TYPE_TO_WEIGHT[compress_type](num_kv_heads, head_dim, kernel_size)
        self.intra_block_pe = torch.nn.Parameter(torch.zeros(num_kv_heads, kernel_size, head_dim))

        self.gate = torch.nn.Sequential(torch.nn.Linear(hidden_size, num_q_heads * 3, bias=False), torch.nn.Sigmoid())
        self.rope = RotaryEmbedding(rope_config, device=rope_device)
        self.init_params()

    def init_params(self):
        for p in self.parameters():
            if len(p.shape) > 1:
                torch.nn.init.xavier_uniform_(p)

    def forward(self, x: torch.Tensor, cu_seqlens: torch.Tensor):
        """x [total_len, hidden_size] (bf16/fp16), cu_seqlens [batch + 1] -> [total_len, hidden_size]."""
        assert x.dtype == torch.bfloat16 or x.dtype == torch.float16
        assert x.shape[-1] == self.hidden_size
        cu_seqlens = cu_seqlens.to(torch.int32)
        seqlens = cu_seqlens[1:] - cu_seqlens[:-1]

        q = self.proj_q(x).view(-1, self.num_q_heads, self.head_dim)
        k = self.proj_k(x).view(-1, self.num_kv_heads, self.head_dim)
        v = self.proj_v(x).view(-1, self.num_kv_heads, self.head_dim)

        # keys and values are compressed before the rotary embedding (:172-188)
        compressed_k, compressed_cu_seqlens = self.compress_func(k, self.compress_key, cu_seqlens, self.kernel_size, self.kernel_stride,
                                                                 self.intra_block_pe)
        # the values compress to the same rows as the keys: no second device read for the output shape
        if self.compress_func in (avgpool_compress, weightedpool_compress, linear_compress):
            compressed_v, _ = self.compress_func(v, self.compress_value, cu_seqlens, self.kernel_size, self.kernel_stride, None,
                                                 known_total=compressed_k.shape[0], known_y_cu=compressed_cu_seqlens)
        else:
            compressed_v, _ = self.compress_func(v, self.compress_value, cu_seqlens, self.kernel_size, self.kernel_stride, None)

        q = self.rope(q, cu_seqlens)
        compressed_k = self.rope(compressed_k, compressed_cu_seqlens, stride=self.kernel_stride)

        compressed_seqlens = compressed_cu_seqlens[1:] - compressed_cu_seqlens[:-1]
        # the two maxima the reference reads back one by one (:197-198), in one device read
        max_seqlen, max_compressed = torch.stack((seqlens.max(), compressed_seqlens.max())).tolist()
        compressed_attn_output, topk_idx = compressed_attention(
            q, compressed_k, compressed_v, self.kernel_size, self.kernel_stride, self.block_size, self.topk, cu_seqlens,
            compressed_cu_seqlens, max_seqlen, max_compressed, None, self.init_blocks, self.local_blocks)

        k = self.rope(k, cu_seqlens)
        sparse_attn_output = topk_sparse_attention(q, k, v, topk_idx, self.block_size, cu_seqlens, None)
        sliding_attn_output = sliding_window_attention_varlen(q, k, v, cu_seqlens, self.window_size)

        gate = self.gate(x).view(-1, self.num_q_heads, 3)
        # gate[..., 0:1] * compressed + gate[..., 1:2] * sparse + gate[..., 2:3] * sliding (:228-232), one kernel each way
        attn_output = gated_sum(gate, compressed_attn_output, sparse_attn_output, sliding_attn_output)
        return self.proj_o(attn_output.reshape(-1, self.num_q_heads * self.head_dim))

    @torch.no_grad()
    def inference(self, x: torch.Tensor, cu_seqlens: torch.Tensor, step: int, cache: NSACache):
        """step == 0: prefill of x [total_len, hidden]; step > 0: one new token per sequence, x [batch, hidden]."""
        assert x.dtype == torch.bfloat16 or x.dtype == torch.float16
        assert x.shape[-1] == self.hidden_size
        cu_seqlens = cu_seqlens.to(torch.int32)
        assert step >= 0
        if step == 0:
            assert x.shape[0] == cu_seqlens[-1]
        else:
            assert x.shape[0] == cu_seqlens.shape[0] - 1
        q = self.proj_q(x).view(-1, self.num_q_heads, self.head_dim)
        k = self.proj_k(x).view(-1, self.num_kv_heads, self.head_dim)
        v = self.proj_v(x).view(-1, self.num_kv_heads, self.head_dim)
        gate = self.gate(x).view(-1, self.num_q_heads, 3)
        output = nsa_infer(cu_seqlens, step, q, k, v, gate, self.rope, cache, [self.compress_key, self.compress_value],
                           [self.compress_func, self.compress_func], self.intra_block_pe, self.kernel_size, self.kernel_stride,
                           self.block_size, self.topk, self.init_blocks, self.local_blocks, self.window_size)
        return self.proj_o(output.reshape(-1, self.num_q_heads * self.head_dim))
