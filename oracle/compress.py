"""Oracles for the three KV compression operators (sliding windows over each sequence).

Test infrastructure only (see package docstring).

Follows native_sparse_attention/ops/torch/compress_key_value.py:19-231 and
native_sparse_attention/ops/triton/utils.py:25-37 of the reference:
compressed token ``n`` of a sequence covers tokens ``[n*stride, n*stride+kernel)``
of that sequence; a sequence shorter than the kernel yields no token; windows
never cross sequences.  ``pe`` enters only as a per-head bias computed with the
same weights.  Unlike the reference these functions run on any device/dtype.
"""
from typing import Optional, Tuple

import torch


def compressed_seqlens(cu_seqlens: torch.Tensor, kernel_size: int, kernel_stride: int):
    """utils.py:25-37 - y_len = floor((L - ks) / st) + 1, or 0 when L < ks."""
    lens = (cu_seqlens[1:] - cu_seqlens[:-1]).to(torch.int64)
    y = torch.div(lens - kernel_size, kernel_stride, rounding_mode="floor") + 1
    y = torch.where(lens < kernel_size, torch.zeros_like(y), y)
    y_cu = torch.zeros(lens.numel() + 1, dtype=torch.int32, device=cu_seqlens.device)
    y_cu[1:] = torch.cumsum(y, 0).to(torch.int32)
    return y.to(torch.int32), y_cu


def _windows(x: torch.Tensor, cu_seqlens, ks: int, st: int):
    """Yield per-sequence window tensors [n, H, ks, d] (possibly n == 0)."""
    cu = [int(c) for c in cu_seqlens.tolist()]
    for b in range(len(cu) - 1):
        xs = x[cu[b] : cu[b + 1]]
        if xs.shape[0] < ks:
            yield xs.new_zeros((0, x.shape[1], ks, x.shape[2]))
        else:
            yield xs.unfold(0, ks, st).permute(0, 1, 3, 2)  # [n, H, ks, d]


def avgpool_compress(x, w, cu_seqlens, kernel_size, kernel_stride, pe: Optional[torch.Tensor] = None):
    """compress_key_value.py:19-81 - mean over the window, bias = mean_k pe."""
    assert w is None
    y = torch.cat([win.mean(dim=2) for win in _windows(x, cu_seqlens, kernel_size, kernel_stride)], 0)
    if pe is not None:
        y = y + pe.mean(dim=1)[None]
    return y, compressed_seqlens(cu_seqlens, kernel_size, kernel_stride)[1]


def weightedpool_compress(x, w, cu_seqlens, kernel_size, kernel_stride, pe: Optional[torch.Tensor] = None):
    """compress_key_value.py:84-153 - y[n,h,:] = sum_k w[h,k] x[n*st+k,h,:], bias = sum_k w[h,k] pe[h,k,:]."""
    assert w.shape == (x.shape[1], kernel_size)
    y = torch.cat(
        [torch.einsum("nhkd,hk->nhd", win, w) for win in _windows(x, cu_seqlens, kernel_size, kernel_stride)], 0
    )
    if pe is not None:
        y = y + torch.einsum("hkd,hk->hd", pe, w)[None]
    return y, compressed_seqlens(cu_seqlens, kernel_size, kernel_stride)[1]


def linear_compress(x, w, cu_seqlens, kernel_size, kernel_stride, pe: Optional[torch.Tensor] = None):
    """compress_key_value.py:156-231 - y[n,h,:] = concat_k(x[n*st+k,h,:]) @ w[h], bias = pe[h].flatten() @ w[h]."""
    H, d = x.shape[1], x.shape[2]
    assert w.shape == (H, kernel_size * d, d)
    w4 = w.reshape(H, kernel_size, d, d)
    y = torch.cat(
        [torch.einsum("nhkd,hkde->nhe", win, w4) for win in _windows(x, cu_seqlens, kernel_size, kernel_stride)], 0
    )
    if pe is not None:
        y = y + torch.einsum("hkd,hkde->he", pe, w4)[None]
    return y, compressed_seqlens(cu_seqlens, kernel_size, kernel_stride)[1]
