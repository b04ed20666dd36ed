"""topk_sparse_attention: same signature and checks as the reference operator
(native_sparse_attention/ops/triton/topk_sparse_attention.py:1112-1217), running on the gfx950 kernels."""
import math
from typing import Optional

import torch

from .. import _lib
from .utils import pad_head_dim


def _last_dim_contiguous(t: torch.Tensor) -> torch.Tensor:
    return t if t.stride(-1) == 1 else t.contiguous()


def _topk_sparse_attention_fwd(q, k, v, topk_idx, block_size, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, sm_scale,
                               workspace=None, phases=3, out=None):
    """Returns (o [T,Hq,D], lse fp32 [Hq,T] in base-2 units); mirrors _topk_sparse_attention_fwd (:828-909).

    workspace / phases / out let a profiler re-run one pass on buffers a previous call filled."""
    assert k.dtype == q.dtype and v.dtype == q.dtype
    assert cu_seqlens_q.dtype == torch.int32 and cu_seqlens_k.dtype == torch.int32
    assert block_size in {32, 64, 128, 256}
    q_len, num_q_heads, head_dim = q.shape
    k_len, num_k_heads, _ = k.shape
    v_len, num_v_heads, _ = v.shape
    batch = cu_seqlens_q.shape[0] - 1
    assert q_len == k_len and k_len == v_len
    topk = topk_idx.shape[-1]
    assert topk_idx.shape[0] == num_k_heads and topk_idx.shape[1] == q_len
    assert num_k_heads == num_v_heads and num_q_heads % num_k_heads == 0
    q, k, v = map(_last_dim_contiguous, (q, k, v))
    if out is None:
        o = torch.empty((q_len, num_q_heads, head_dim), dtype=q.dtype, device=q.device)
        lse = torch.empty((num_q_heads, q_len), dtype=torch.float32, device=q.device)
    else:
        o, lse = out
    lib = _lib.load()
    ws = workspace
    if ws is None:
        ws = _lib.workspace(lib.nsa_topk_attn_fwd_workspace_bytes(q_len, batch, num_k_heads, head_dim), q.device)
    rc = lib.nsa_topk_attn_fwd(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), topk_idx.data_ptr(), o.data_ptr(), lse.data_ptr(),
        cu_seqlens_q.data_ptr(), q_len, batch, num_q_heads, num_k_heads, head_dim, topk, block_size,
        q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1),
        topk_idx.stride(0), topk_idx.stride(1), topk_idx.stride(2), o.stride(0), o.stride(1),
        sm_scale, _lib.dtype_code(q), ws.data_ptr(), ws.numel(), phases, _lib.stream_ptr(q),
    )
    _lib.check(rc, "nsa_topk_attn_fwd")
    return o, lse


def _topk_sparse_attention_bwd(o, do, lse, q, k, v, topk_idx, block_size, cu_seqlens_q, cu_seqlens_k,
                               max_seqlen_q, max_seqlen_k, sm_scale, return_reverse_index=False, workspace=None, phases=7, out=None):
    """Returns (dq, dk, dv); mirrors _topk_sparse_attention_bwd (:912-1109)."""
    assert block_size in {32, 64, 128, 256}
    q_len, num_q_heads, head_dim = q.shape
    num_k_heads = k.shape[1]
    batch = cu_seqlens_q.shape[0] - 1
    topk = topk_idx.shape[-1]
    q, k, v, o, do = map(_last_dim_contiguous, (q, k, v, o, do))
    if out is None:
        dq = torch.empty((q_len, num_q_heads, head_dim), dtype=q.dtype, device=q.device)
        dk = torch.empty((q_len, num_k_heads, head_dim), dtype=q.dtype, device=q.device)
        dv = torch.empty((q_len, num_k_heads, head_dim), dtype=q.dtype, device=q.device)
    else:
        dq, dk, dv = out
    lib = _lib.load()
    ws = workspace
    if ws is None:
        ws = _lib.workspace(
            lib.nsa_topk_attn_bwd_workspace_bytes(q_len, batch, num_q_heads, num_k_heads, head_dim, topk, block_size), q.device)
    strides = _lib.host_i64(
        [q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1), o.stride(0), o.stride(1),
         do.stride(0), do.stride(1), topk_idx.stride(0), topk_idx.stride(1), topk_idx.stride(2),
         dq.stride(0), dq.stride(1), dk.stride(0), dk.stride(1), dv.stride(0), dv.stride(1)])
    seg_off = queries = None
    if return_reverse_index:
        n_seg = lib.nsa_topk_reverse_index_segments(q_len, batch, num_k_heads, block_size)
        seg_off = torch.empty(n_seg + 1, dtype=torch.int32, device=q.device)
        pieces = 4 if block_size == 256 else 1  # the index of 256-key blocks is kept per 64-key piece
        queries = torch.empty(pieces * num_k_heads * q_len * topk, dtype=torch.int32, device=q.device)
    rc = lib.nsa_topk_attn_bwd(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), do.data_ptr(), lse.data_ptr(), topk_idx.data_ptr(),
        cu_seqlens_q.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), q_len, batch, num_q_heads, num_k_heads,
        head_dim, topk, block_size, strides, sm_scale, _lib.dtype_code(q), ws.data_ptr(), ws.numel(),
        seg_off.data_ptr() if return_reverse_index else None, queries.data_ptr() if return_reverse_index else None,
        phases, _lib.stream_ptr(q),
    )
    _lib.check(rc, "nsa_topk_attn_bwd")
    if return_reverse_index:
        return dq, dk, dv, seg_off, queries
    return dq, dk, dv


class TopkSparseAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, topk_idx, block_size, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, sm_scale=None):
        assert q.dtype == torch.bfloat16 or q.dtype == torch.float16
        assert q.dtype == k.dtype and k.dtype == v.dtype
        assert topk_idx.dtype == torch.int32
        assert cu_seqlens_q.dtype == torch.int32 and cu_seqlens_k.dtype == torch.int32
        if sm_scale is None:
            sm_scale = 1 / math.sqrt(q.shape[-1])
        o, lse = _topk_sparse_attention_fwd(
            q, k, v, topk_idx, block_size, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, sm_scale)
        ctx.save_for_backward(q, k, v, o, lse, cu_seqlens_q, cu_seqlens_k, topk_idx)
        ctx.sm_scale, ctx.block_size = sm_scale, block_size
        ctx.max_seqlen_q, ctx.max_seqlen_k = max_seqlen_q, max_seqlen_k
        return o

    @staticmethod
    def backward(ctx, do, *args):
        q, k, v, o, lse, cu_seqlens_q, cu_seqlens_k, topk_idx = ctx.saved_tensors
        dq, dk, dv = _topk_sparse_attention_bwd(
            o, do, lse, q, k, v, topk_idx, ctx.block_size, cu_seqlens_q, cu_seqlens_k,
            ctx.max_seqlen_q, ctx.max_seqlen_k, ctx.sm_scale)
        return dq, dk, dv, None, None, None, None, None, None, None


def topk_sparse_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    topk_idx: torch.Tensor,
    block_size: int,
    cu_seqlens: torch.Tensor,
    softmax_scale: Optional[float] = None,
) -> torch.Tensor:
    """Block-sparse GQA attention, varlen layout.

    Args:
        q: [total_len, num_q_heads, head_dim]; k, v: [total_len, num_kv_heads, head_dim] (bf16/fp16)
        topk_idx: int32 [num_kv_heads, total_len, topk], per-sequence block ids, -1 = padding
        block_size: key/value block size (32, 64, 128 or 256)
        cu_seqlens: int32 [batch + 1]
        softmax_scale: defaults to 1/sqrt(head_dim)
    Returns: [total_len, num_q_heads, head_dim]

    The kernels walk the token range directly, so unlike the reference wrapper (:1205) no
    host synchronisation is needed to learn the longest sequence.
    """
    d = q.shape[-1]
    if softmax_scale is None:
        softmax_scale = 1 / math.sqrt(d)
    q, k, v = pad_head_dim(q, k, v)
    o = TopkSparseAttention.apply(q, k, v, topk_idx, block_size, cu_seqlens, cu_seqlens, None, None, softmax_scale)
    return o if o.shape[-1] == d else o[..., :d].contiguous()
