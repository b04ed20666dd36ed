"""Causal sliding-window varlen attention (forward only) for the window branch of the prefill path.

The reference calls the third-party flash_attn_varlen_func(..., causal=True, window_size=(W, -1))
here (native_sparse_attention/infer/inference_func.py:180-190); this is the in-repo counterpart."""
import math
from typing import Optional

import torch

from .. import _lib
from .utils import last_dim_contiguous


@torch.no_grad()
def sliding_window_attention_varlen(q, k, v, cu_seqlens, window_size: int, sm_scale: Optional[float] = None) -> torch.Tensor:
    """q [T,Hq,D], k/v [T,Hkv,D]; position i sees keys j of its own sequence with i - window_size <= j <= i."""
    assert q.dtype == torch.bfloat16 or q.dtype == torch.float16
    assert k.dtype == q.dtype and v.dtype == q.dtype and cu_seqlens.dtype == torch.int32
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    assert k.shape[0] == T and v.shape == k.shape and Hq % Hkv == 0
    if sm_scale is None:
        sm_scale = 1 / math.sqrt(D)
    q, k, v = map(last_dim_contiguous, (q, k, v))
    o = torch.zeros_like(q, memory_format=torch.contiguous_format)
    lse = torch.empty(Hq, T, dtype=torch.float32, device=q.device)
    strides = _lib.host_i64([q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1), o.stride(0), o.stride(1)])
    rc = _lib.load().nsa_window_attn_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(), cu_seqlens.data_ptr(),
                                         T, cu_seqlens.shape[0] - 1, Hq, Hkv, D, window_size, strides, sm_scale,
                                         _lib.dtype_code(q), _lib.stream_ptr(q))
    _lib.check(rc, "nsa_window_attn_fwd")
    return o
