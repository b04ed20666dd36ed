"""weightedpool_compress / avgpool_compress: same signatures and checks as the reference operators
(native_sparse_attention/ops/triton/weighted_pool.py:182-363), running on the gfx950 pooling kernels."""
from typing import Optional

import torch

from .. import _lib
from .utils import compressed_seqlens_cached, last_dim_contiguous


class SlidingWindowWeightedPool(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w, cu_seqlens, kernel_size, kernel_stride, known_total=None, known_y_cu=None, bias=None):
        assert x.dtype == torch.float16 or x.dtype == torch.bfloat16
        if w is not None:
            assert x.dtype == w.dtype
        assert cu_seqlens.dtype == torch.int32
        total_len, num_heads, head_dim = x.shape
        batch = cu_seqlens.shape[0] - 1
        if w is not None:
            assert w.shape[0] == num_heads and w.shape[1] == kernel_size
            w = w.contiguous()
        assert kernel_size % kernel_stride == 0
        assert kernel_size in {16, 32, 64, 128}
        x = last_dim_contiguous(x)
        # compressed lengths and the output shape: a launch and the one host synchronisation the reference has too,
        # unless the caller passes them or this cu_seqlens tensor has been through here before
        if known_y_cu is not None and known_total is not None:
            y_cu_seqlens, total_y = known_y_cu, int(known_total)
        else:
            y_cu_seqlens, total_y = compressed_seqlens_cached(cu_seqlens, kernel_size, kernel_stride, known_total is None)
            y_cu_seqlens = known_y_cu if known_y_cu is not None else y_cu_seqlens
            total_y = int(known_total) if known_total is not None else total_y
        if bias is not None:
            assert bias.shape == (num_heads, head_dim) and bias.dtype == x.dtype
            bias = bias.contiguous()
        y = torch.empty(total_y, num_heads, head_dim, dtype=x.dtype, device=x.device)
        lib = _lib.load()
        rc = lib.nsa_pool_fwd_bias(
            x.data_ptr(), w.data_ptr() if w is not None else None, bias.data_ptr() if bias is not None else None, y.data_ptr(),
            cu_seqlens.data_ptr(), y_cu_seqlens.data_ptr(), total_len, total_y, batch, num_heads, head_dim, kernel_size, kernel_stride,
            x.stride(0), x.stride(1), y.stride(0), y.stride(1), w.stride(0) if w is not None else 0,
            bias.stride(0) if bias is not None else 0, _lib.dtype_code(x), _lib.stream_ptr(x))
        _lib.check(rc, "nsa_pool_fwd")
        ctx.save_for_backward(x, w, cu_seqlens, y_cu_seqlens)
        ctx.kernel_size, ctx.kernel_stride, ctx.total_y = kernel_size, kernel_stride, total_y
        ctx.has_bias = bias is not None
        ctx.mark_non_differentiable(y_cu_seqlens)
        return y, y_cu_seqlens

    @staticmethod
    def backward(ctx, dy, _):
        x, w, cu_seqlens, y_cu_seqlens = ctx.saved_tensors
        total_len, num_heads, head_dim = x.shape
        batch = cu_seqlens.shape[0] - 1
        dy = last_dim_contiguous(dy)
        dx = torch.empty_like(x, memory_format=torch.contiguous_format)
        dw = torch.empty_like(w) if w is not None else None
        lib = _lib.load()
        ws = _lib.workspace(lib.nsa_pool_bwd_workspace_bytes(ctx.total_y, num_heads, ctx.kernel_size), x.device)
        rc = lib.nsa_pool_bwd(
            x.data_ptr(), w.data_ptr() if w is not None else None, dy.data_ptr(), dx.data_ptr(),
            dw.data_ptr() if w is not None else None, cu_seqlens.data_ptr(), y_cu_seqlens.data_ptr(),
            total_len, ctx.total_y, batch, num_heads, head_dim, ctx.kernel_size, ctx.kernel_stride,
            x.stride(0), x.stride(1), dy.stride(0), dy.stride(1), dx.stride(0), dx.stride(1),
            w.stride(0) if w is not None else 0, dw.stride(0) if w is not None else 0,
            _lib.dtype_code(x), ws.data_ptr(), ws.numel(), _lib.stream_ptr(x))
        _lib.check(rc, "nsa_pool_bwd")
        # the bias row was added to every output row
        dbias = dy.sum(0) if ctx.has_bias else None
        return dx, dw, None, None, None, None, None, dbias


def weightedpool_compress(
    x: torch.Tensor,
    w: torch.Tensor,
    cu_seqlens: torch.Tensor,
    kernel_size: int,
    kernel_stride: int,
    pe: Optional[torch.Tensor] = None,
    known_total: Optional[int] = None,
    known_y_cu: Optional[torch.Tensor] = None,
):
    """Weighted sliding-window pooling of key/value states.

    x: [total_len, num_heads, head_dim]; w: [num_heads, kernel_size]; pe: optional
    [num_heads, kernel_size, head_dim] intra-block positional embedding, added as the bias
    sum_k w[h,k] pe[h,k,:].  Returns (y [total_y, num_heads, head_dim], y_cu_seqlens int32).
    known_total (not in the reference's signature): total number of output rows when the caller knows it on the
    host; the output is then allocated without reading y_cu_seqlens back.  known_y_cu (likewise): the output's
    cu_seqlens when the caller already holds them (a decode step compresses one full window per sequence).
    """
    bias = None
    if pe is not None:
        assert pe.dtype == x.dtype and pe.device == x.device
        bias = torch.einsum("hkd,hk->hd", pe, w)   # added to every output row by the kernel
    return SlidingWindowWeightedPool.apply(x, w, cu_seqlens, kernel_size, kernel_stride, known_total, known_y_cu, bias)


def avgpool_compress(
    x: torch.Tensor,
    w: torch.Tensor,
    cu_seqlens: torch.Tensor,
    kernel_size: int,
    kernel_stride: int,
    pe: Optional[torch.Tensor] = None,
    known_total: Optional[int] = None,
    known_y_cu: Optional[torch.Tensor] = None,
):
    """Average sliding-window pooling; ``w`` must be None.  Bias = mean_k pe[h,k,:].  known_total / known_y_cu as in
    weightedpool_compress."""
    assert w is None, "don't need additional weight for avgpool"
    bias = None
    if pe is not None:
        assert pe.dtype == x.dtype and pe.device == x.device
        bias = torch.mean(pe, dim=1)   # added to every output row by the kernel
    return SlidingWindowWeightedPool.apply(x, w, cu_seqlens, kernel_size, kernel_stride, known_total, known_y_cu, bias)
