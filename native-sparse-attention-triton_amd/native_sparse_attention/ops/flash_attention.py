"""Dense varlen attention, same call as the reference's flash_attention_varlen
(native_sparse_attention/ops/triton/flash_attention.py:895-935), on the tile kernels of this package."""
import math
from typing import Optional

import torch

from .. import _lib
from .utils import last_dim_contiguous, pad_head_dim


def _flash_attention_fwd(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, causal, sm_scale, gqa_interleave=False):
    """Forward pass alone, as the reference's helper of the same name (ops/triton/flash_attention.py:563-642): returns
    (o, lse).  lse is fp32 [Hq, total_q] in base-2 units (only _flash_attention_bwd reads it)."""
    assert not gqa_interleave, "interleaved GQA is handled by flash_attention_varlen (a head permutation around this call)"
    q, k, v = map(last_dim_contiguous, (q, k, v))
    Tq, Hq, D = q.shape
    Tk, Hkv, _ = k.shape
    B = cu_seqlens_q.shape[0] - 1
    o = torch.zeros_like(q, memory_format=torch.contiguous_format)
    lse = torch.empty(Hq, Tq, dtype=torch.float32, device=q.device)
    strides = _lib.host_i64([q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1), o.stride(0), o.stride(1)])
    rc = _lib.load().nsa_flash_attn_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(), cu_seqlens_q.data_ptr(),
                                        cu_seqlens_k.data_ptr(), Tq, Tk, B, Hq, Hkv, D, int(causal), strides, sm_scale,
                                        _lib.dtype_code(q), _lib.stream_ptr(q))
    _lib.check(rc, "nsa_flash_attn_fwd")
    return o, lse


def _flash_attention_bwd(o, do, lse, q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, causal, sm_scale,
                         gqa_interleave=False):
    """Backward pass alone (ops/triton/flash_attention.py:645-892 of the reference): returns (dq, dk, dv)."""
    assert not gqa_interleave, "interleaved GQA is handled by flash_attention_varlen (a head permutation around this call)"
    q, k, v, o, do = map(last_dim_contiguous, (q, k, v, o, do))
    Tq, Hq, D = q.shape
    Tk, Hkv, _ = k.shape
    B = cu_seqlens_q.shape[0] - 1
    dq = torch.zeros_like(q, memory_format=torch.contiguous_format)
    dk = torch.zeros_like(k, memory_format=torch.contiguous_format)
    dv = torch.zeros_like(v, memory_format=torch.contiguous_format)
    lib = _lib.load()
    ws = _lib.workspace(lib.nsa_flash_attn_bwd_workspace_bytes(Tq, Tk, B, Hq, Hkv, D), q.device)
    strides = _lib.host_i64([q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1), o.stride(0), o.stride(1),
                             do.stride(0), do.stride(1), dq.stride(0), dq.stride(1), dk.stride(0), dk.stride(1), dv.stride(0), dv.stride(1)])
    rc = lib.nsa_flash_attn_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), do.data_ptr(), lse.data_ptr(), dq.data_ptr(),
                                dk.data_ptr(), dv.data_ptr(), cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), Tq, Tk, B, Hq, Hkv, D,
                                int(causal), strides, sm_scale, _lib.dtype_code(q), ws.data_ptr(), ws.numel(), _lib.stream_ptr(q))
    _lib.check(rc, "nsa_flash_attn_bwd")
    return dq, dk, dv


class FlashAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens_q, cu_seqlens_k, causal, sm_scale):
        q, k, v = map(last_dim_contiguous, (q, k, v))
        o, lse = _flash_attention_fwd(q, k, v, cu_seqlens_q, cu_seqlens_k, 0, 0, causal, sm_scale)
        ctx.save_for_backward(q, k, v, o, lse, cu_seqlens_q, cu_seqlens_k)
        ctx.causal, ctx.sm_scale = causal, sm_scale
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, lse, cu_q, cu_k = ctx.saved_tensors
        dq, dk, dv = _flash_attention_bwd(o, do, lse, q, k, v, cu_q, cu_k, 0, 0, ctx.causal, ctx.sm_scale)
        return dq, dk, dv, None, None, None, None


def flash_attention_varlen(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens_q: torch.Tensor, cu_seqlens_k: torch.Tensor,
                           max_seqlen_q: int, max_seqlen_k: int, causal: bool = False, sm_scale: Optional[float] = None,
                           gqa_interleave: bool = False) -> torch.Tensor:
    """q [total_q, Hq, D]; k, v [total_k, Hkv, D]; returns [total_q, Hq, D].  causal: query i sees keys j <= i of its own
    sequence (both counted from the sequence start).  gqa_interleave: query head h uses kv head h % Hkv instead of
    h // (Hq / Hkv).  max_seqlen_q / max_seqlen_k are accepted for signature compatibility and not needed."""
    assert q.dtype == torch.bfloat16 or q.dtype == torch.float16
    assert k.dtype == q.dtype and v.dtype == q.dtype
    assert cu_seqlens_q.dtype == torch.int32 and cu_seqlens_k.dtype == torch.int32 and cu_seqlens_q.shape == cu_seqlens_k.shape
    Hq, Hkv = q.shape[1], k.shape[1]
    assert k.shape == v.shape and q.shape[2] == k.shape[2] and Hq % Hkv == 0
    d = q.shape[-1]
    if sm_scale is None:
        sm_scale = 1 / math.sqrt(d)
    if pad_head_dim(q)[0].shape[-1] != d:   # head size between the built ones: zero columns appended
        o = flash_attention_varlen(*pad_head_dim(q, k, v), cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, causal, sm_scale, gqa_interleave)
        return o[..., :d].contiguous()
    if gqa_interleave and Hq != Hkv:
        G = Hq // Hkv
        # the kernels group G consecutive query heads per kv head: reorder (g, kv) -> (kv, g) and back
        qg = q.view(q.shape[0], G, Hkv, q.shape[2]).transpose(1, 2).reshape(q.shape)
        o = FlashAttention.apply(qg, k, v, cu_seqlens_q, cu_seqlens_k, bool(causal), float(sm_scale))
        return o.view(o.shape[0], Hkv, G, o.shape[2]).transpose(1, 2).reshape(o.shape)
    return FlashAttention.apply(q, k, v, cu_seqlens_q, cu_seqlens_k, bool(causal), float(sm_scale))
