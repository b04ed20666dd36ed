"""compressed_attention: same signature and checks as the reference operator
(native_sparse_attention/ops/triton/compressed_attention.py:783-848, 1182-1331), on the gfx950 kernels.
The block selection is one fused kernel; the dense [Hkv, T, Tc] score tensor of the reference is
never built, so there is no sequence-length threshold and `parallel_topk_compute` has no effect."""
import math
import warnings
from typing import Optional, Tuple, Union

import torch

from .. import _lib
from .utils import last_dim_contiguous, pad_head_dim


def _compressed_attention_fwd(q, k, v, kernel_size, kernel_stride, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, sm_scale):
    assert k.dtype == q.dtype and v.dtype == q.dtype
    assert cu_seqlens_q.dtype == torch.int32 and cu_seqlens_k.dtype == torch.int32
    q_len, num_q_heads, head_dim = q.shape
    k_len, num_k_heads, _ = k.shape
    v_len, num_v_heads, _ = v.shape
    batch = cu_seqlens_q.shape[0] - 1
    assert k_len == v_len and q_len > k_len
    assert num_k_heads == num_v_heads and num_q_heads % num_k_heads == 0
    q, k, v = map(last_dim_contiguous, (q, k, v))
    o = torch.zeros_like(q, memory_format=torch.contiguous_format)
    lse = torch.full((num_q_heads, q_len), -torch.inf, dtype=torch.float32, device=q.device)
    lib = _lib.load()
    strides = _lib.host_i64([q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1), o.stride(0), o.stride(1)])
    rc = lib.nsa_cmp_attn_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(), cu_seqlens_q.data_ptr(),
                              cu_seqlens_k.data_ptr(), q_len, k_len, batch, num_q_heads, num_k_heads, head_dim, kernel_size,
                              kernel_stride, strides, sm_scale, _lib.dtype_code(q), _lib.stream_ptr(q))
    _lib.check(rc, "nsa_cmp_attn_fwd")
    return o, lse


def _compressed_attention_bwd(o, do, lse, q, k, v, kernel_size, kernel_stride, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, sm_scale):
    q_len, num_q_heads, head_dim = q.shape
    k_len, num_k_heads, _ = k.shape
    batch = cu_seqlens_q.shape[0] - 1
    q, k, v, o, do = map(last_dim_contiguous, (q, k, v, o, do))
    dq = torch.empty((q_len, num_q_heads, head_dim), dtype=q.dtype, device=q.device)
    dk = torch.empty((k_len, num_k_heads, head_dim), dtype=q.dtype, device=q.device)
    dv = torch.empty((k_len, num_k_heads, head_dim), dtype=q.dtype, device=q.device)
    lib = _lib.load()
    ws = _lib.workspace(lib.nsa_cmp_attn_bwd_workspace_bytes(q_len, k_len, batch, num_q_heads, num_k_heads, head_dim), q.device)
    strides = _lib.host_i64([q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1), o.stride(0), o.stride(1),
                             do.stride(0), do.stride(1), dq.stride(0), dq.stride(1), dk.stride(0), dk.stride(1), dv.stride(0), dv.stride(1)])
    rc = lib.nsa_cmp_attn_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), do.data_ptr(), lse.data_ptr(), dq.data_ptr(),
                              dk.data_ptr(), dv.data_ptr(), cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), q_len, k_len, batch,
                              num_q_heads, num_k_heads, head_dim, kernel_size, kernel_stride, strides, sm_scale,
                              _lib.dtype_code(q), ws.data_ptr(), ws.numel(), _lib.stream_ptr(q))
    _lib.check(rc, "nsa_cmp_attn_bwd")
    return dq, dk, dv


def _select_blocks(q, k, lse, kernel_size, kernel_stride, block_size, k_out, cu_seqlens_q, cu_seqlens_k, max_seqlen_q,
                   init_blocks, local_blocks, sm_scale):
    q_len, num_q_heads, head_dim = q.shape
    k_len, num_k_heads, _ = k.shape
    batch = cu_seqlens_q.shape[0] - 1
    q, k = map(last_dim_contiguous, (q, k))
    idx = torch.empty(num_k_heads, q_len, k_out, dtype=torch.int32, device=q.device)
    lib = _lib.load()
    strides = _lib.host_i64([q.stride(0), q.stride(1), k.stride(0), k.stride(1), 0, 0, idx.stride(0), idx.stride(1), idx.stride(2)])
    rc = lib.nsa_cmp_attn_select(q.data_ptr(), k.data_ptr(), lse.data_ptr(), cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(),
                                 idx.data_ptr(), q_len, k_len, batch, num_q_heads, num_k_heads, head_dim, kernel_size, kernel_stride,
                                 block_size, k_out, max_seqlen_q, init_blocks, local_blocks, strides, sm_scale,
                                 _lib.dtype_code(q), _lib.stream_ptr(q))
    _lib.check(rc, "nsa_cmp_attn_select")
    return idx


class CompressedAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, kernel_size, kernel_stride, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, sm_scale=None):
        assert q.dtype == torch.bfloat16 or q.dtype == torch.float16
        assert q.dtype == k.dtype and k.dtype == v.dtype
        assert cu_seqlens_q.dtype == torch.int32 and cu_seqlens_k.dtype == torch.int32
        if sm_scale is None:
            sm_scale = 1 / math.sqrt(q.shape[-1])
        o, lse = _compressed_attention_fwd(q, k, v, kernel_size, kernel_stride, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, sm_scale)
        ctx.save_for_backward(q, k, v, o, lse, cu_seqlens_q, cu_seqlens_k)
        ctx.sm_scale, ctx.kernel_size, ctx.kernel_stride = sm_scale, kernel_size, kernel_stride
        ctx.max_seqlen_q, ctx.max_seqlen_k = max_seqlen_q, max_seqlen_k
        ctx.mark_non_differentiable(lse)
        return o, lse

    @staticmethod
    def backward(ctx, do, *args):
        q, k, v, o, lse, cu_seqlens_q, cu_seqlens_k = ctx.saved_tensors
        dq, dk, dv = _compressed_attention_bwd(o, do, lse, q, k, v, ctx.kernel_size, ctx.kernel_stride, cu_seqlens_q, cu_seqlens_k,
                                               ctx.max_seqlen_q, ctx.max_seqlen_k, ctx.sm_scale)
        return dq, dk, dv, None, None, None, None, None, None, None


def compressed_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    kernel_size: int,
    kernel_stride: int,
    block_size: int,
    topk: int,
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_k: torch.Tensor,
    max_seqlen_q: int = None,
    max_seqlen_k: int = None,
    sm_scale: float = None,
    init_blocks: int = 1,
    local_blocks: int = 2,
    parallel_topk_compute: Union[str, bool] = "auto",
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Attention between queries and compressed keys/values, plus the block ids for topk_sparse_attention.

    q: [total_q_len, num_q_heads, head_dim]; k, v: [total_kv_len, num_kv_heads, head_dim] (compressed);
    returns (attn_output [total_q_len, num_q_heads, head_dim],
    topk_idx int32 [num_kv_heads, total_q_len, min(topk, ceil(max_seqlen_q / block_size))]), or
    (attn_output, None) with a warning when topk <= 0.
    """
    if max_seqlen_q is None:
        max_seqlen_q = (cu_seqlens_q[1:] - cu_seqlens_q[:-1]).max().item()
    if max_seqlen_k is None:
        max_seqlen_k = (cu_seqlens_k[1:] - cu_seqlens_k[:-1]).max().item()
    d = q.shape[-1]
    if sm_scale is None:
        sm_scale = 1 / math.sqrt(d)
    q, k, v = pad_head_dim(q, k, v)
    attn_output, lse = CompressedAttention.apply(
        q, k, v, kernel_size, kernel_stride, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, sm_scale)
    out = attn_output if attn_output.shape[-1] == d else attn_output[..., :d].contiguous()
    if topk <= 0:
        warnings.warn("topk <= 0, returned topk_idx will be None")
        return out, None
    assert topk >= init_blocks + local_blocks
    assert block_size % kernel_size == 0 and kernel_size % kernel_stride == 0
    with torch.no_grad():
        k_out = min(topk, math.ceil(max_seqlen_q / block_size))
        topk_idx = _select_blocks(q.detach(), k.detach(), lse, kernel_size, kernel_stride, block_size, k_out, cu_seqlens_q,
                                  cu_seqlens_k, max_seqlen_q, init_blocks, local_blocks, sm_scale)
    return out, topk_idx
