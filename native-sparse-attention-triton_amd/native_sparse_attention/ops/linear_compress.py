"""linear_compress: same signature and checks as the reference operator
(native_sparse_attention/ops/triton/linear_compress.py:309-525), on the gfx950 strided-window GEMM kernels."""
from typing import Optional, Tuple

import torch

from .. import _lib
from .utils import compressed_seqlens_cached, last_dim_contiguous


class LinearCompress(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w, cu_seqlens, kernel_size, kernel_stride, known_total=None, known_y_cu=None, bias=None):
        assert x.dtype == torch.float16 or x.dtype == torch.bfloat16
        assert x.dtype == w.dtype
        assert cu_seqlens.dtype == torch.int32
        total_len, num_heads, head_dim = x.shape
        batch = cu_seqlens.shape[0] - 1
        assert w.shape[0] == num_heads
        assert w.shape[1] == kernel_size * head_dim
        assert w.shape[2] == head_dim
        assert kernel_size % kernel_stride == 0
        assert kernel_size in {16, 32, 64, 128}
        assert head_dim % 8 == 0
        x = last_dim_contiguous(x)
        w = w.contiguous()
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
        rc = lib.nsa_linear_compress_fwd_bias(
            x.data_ptr(), w.data_ptr(), bias.data_ptr() if bias is not None else None, y.data_ptr(), cu_seqlens.data_ptr(),
            y_cu_seqlens.data_ptr(), total_len, total_y, batch, num_heads, head_dim, kernel_size, kernel_stride, x.stride(0),
            x.stride(1), y.stride(0), y.stride(1), bias.stride(0) if bias is not None else 0, _lib.dtype_code(x), _lib.stream_ptr(x))
        _lib.check(rc, "nsa_linear_compress_fwd")
        ctx.save_for_backward(x, w, cu_seqlens, y_cu_seqlens)
        ctx.kernel_size, ctx.kernel_stride, ctx.total_y = kernel_size, kernel_stride, total_y
        ctx.has_bias = bias is not None
        ctx.mark_non_differentiable(y_cu_seqlens)
        return y, y_cu_seqlens

    @staticmethod
    def backward(ctx, dy, *args):
        x, w, cu_seqlens, y_cu_seqlens = ctx.saved_tensors
        total_len, num_heads, head_dim = x.shape
        batch = cu_seqlens.shape[0] - 1
        dy = last_dim_contiguous(dy)
        dx = torch.empty_like(x, memory_format=torch.contiguous_format)
        dw = torch.empty_like(w)
        lib = _lib.load()
        rc = lib.nsa_linear_compress_bwd(
            x.data_ptr(), w.data_ptr(), dy.data_ptr(), dx.data_ptr(), dw.data_ptr(), cu_seqlens.data_ptr(),
            y_cu_seqlens.data_ptr(), total_len, ctx.total_y, batch, num_heads, head_dim, ctx.kernel_size, ctx.kernel_stride,
            x.stride(0), x.stride(1), dy.stride(0), dy.stride(1), dx.stride(0), dx.stride(1),
            _lib.dtype_code(x), _lib.stream_ptr(x))
        _lib.check(rc, "nsa_linear_compress_bwd")
        # the bias row was added to every output row
        dbias = dy.sum(0) if ctx.has_bias else None
        return dx, dw, None, None, None, None, None, dbias


def linear_compress(
    x: torch.Tensor,
    w: torch.Tensor,
    cu_seqlens: torch.Tensor,
    kernel_size: int,
    kernel_stride: int,
    pe: Optional[torch.Tensor] = None,
    known_total: Optional[int] = None,
    known_y_cu: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Sliding-window linear projection of key/value states.

    x: [total_len, num_heads, head_dim]; w: [num_heads, kernel_size * head_dim, head_dim]; pe: optional
    [num_heads, kernel_size, head_dim], added as the bias pe[h].flatten() @ w[h].
    Returns (y [total_y, num_heads, head_dim], y_cu_seqlens int32).
    known_total (not in the reference's signature): total number of output rows when the caller knows it on the
    host; the output is then allocated without reading y_cu_seqlens back.  known_y_cu (likewise): the output's
    cu_seqlens when the caller already holds them.
    """
    bias = None
    if pe is not None:
        assert pe.dtype == x.dtype and pe.device == x.device
        bias = torch.einsum("hk,hkd->hd", pe.reshape(pe.shape[0], -1), w)   # added to every output row by the kernel
    return LinearCompress.apply(x, w, cu_seqlens, kernel_size, kernel_stride, known_total, known_y_cu, bias)
