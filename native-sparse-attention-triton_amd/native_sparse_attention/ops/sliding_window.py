"""Causal sliding-window varlen attention, forward and backward, for the window branch.

The reference calls the third-party flash_attn_varlen_func(..., causal=True, window_size=(W, -1))
here (native_sparse_attention/module/native_sparse_attention.py:213-223 in training,
native_sparse_attention/infer/inference_func.py:180-190 in prefill); this is the in-repo counterpart."""
import math
from typing import Optional

import torch

from .. import _lib
from .utils import last_dim_contiguous, pad_head_dim


def _window_fwd(q, k, v, cu_seqlens, window_size, sm_scale):
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    o = torch.zeros_like(q, memory_format=torch.contiguous_format)
    lse = torch.empty(Hq, T, dtype=torch.float32, device=q.device)
    strides = _lib.host_i64([q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1), o.stride(0), o.stride(1)])
    rc = _lib.load().nsa_window_attn_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(), cu_seqlens.data_ptr(),
                                         T, cu_seqlens.shape[0] - 1, Hq, Hkv, D, window_size, strides, sm_scale,
                                         _lib.dtype_code(q), _lib.stream_ptr(q))
    _lib.check(rc, "nsa_window_attn_fwd")
    return o, lse


def _window_bwd(q, k, v, o, lse, do, cu_seqlens, window_size, sm_scale):
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    B = cu_seqlens.shape[0] - 1
    do = last_dim_contiguous(do)
    dq = torch.zeros_like(q, memory_format=torch.contiguous_format)
    dk = torch.zeros_like(k, memory_format=torch.contiguous_format)
    dv = torch.zeros_like(v, memory_format=torch.contiguous_format)
    lib = _lib.load()
    ws = _lib.workspace(lib.nsa_window_attn_bwd_workspace_bytes(T, B, Hq, Hkv, D), q.device)
    strides = _lib.host_i64([q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1), o.stride(0), o.stride(1),
                             do.stride(0), do.stride(1), dq.stride(0), dq.stride(1), dk.stride(0), dk.stride(1), dv.stride(0), dv.stride(1)])
    rc = lib.nsa_window_attn_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), do.data_ptr(), lse.data_ptr(), dq.data_ptr(),
                                 dk.data_ptr(), dv.data_ptr(), cu_seqlens.data_ptr(), T, B, Hq, Hkv, D, window_size, strides, sm_scale,
                                 _lib.dtype_code(q), ws.data_ptr(), ws.numel(), _lib.stream_ptr(q))
    _lib.check(rc, "nsa_window_attn_bwd")
    return dq, dk, dv


class SlidingWindowAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens, window_size, sm_scale):
        q, k, v = map(last_dim_contiguous, (q, k, v))
        o, lse = _window_fwd(q, k, v, cu_seqlens, window_size, sm_scale)
        ctx.save_for_backward(q, k, v, o, lse, cu_seqlens)
        ctx.window_size, ctx.sm_scale = window_size, sm_scale
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, lse, cu_seqlens = ctx.saved_tensors
        dq, dk, dv = _window_bwd(q, k, v, o, lse, do, cu_seqlens, ctx.window_size, ctx.sm_scale)
        return dq, dk, dv, None, None, None


def sliding_window_attention_varlen(q, k, v, cu_seqlens, window_size: int, sm_scale: Optional[float] = None) -> torch.Tensor:
    """q [T,Hq,D], k/v [T,Hkv,D]; position i sees keys j of its own sequence with i - window_size <= j <= i.
    Gradients flow to q, k and v."""
    assert q.dtype == torch.bfloat16 or q.dtype == torch.float16
    assert k.dtype == q.dtype and v.dtype == q.dtype and cu_seqlens.dtype == torch.int32
    assert k.shape[0] == q.shape[0] and v.shape == k.shape and q.shape[1] % k.shape[1] == 0 and window_size >= 0
    d = q.shape[-1]
    if sm_scale is None:
        sm_scale = 1 / math.sqrt(d)
    q, k, v = pad_head_dim(q, k, v)   # head size between the built ones: zero columns appended
    o = SlidingWindowAttention.apply(q, k, v, cu_seqlens, int(window_size), float(sm_scale))
    return o if o.shape[-1] == d else o[..., :d].contiguous()
