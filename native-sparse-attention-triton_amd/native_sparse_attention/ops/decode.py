"""Decode-time operators: same signatures and checks as the reference's
flash_attention_decode (ops/triton/flash_attention_decode.py:142-217),
topk_sparse_attention_decode (ops/triton/topk_sparse_attention_decode.py:151-237) and
compressed_attention_decode (ops/torch/compressed_attention_decode.py:65-153), on the gfx950 kernels.
k / v may be strided views of a cache slab; nothing is copied."""
import math
from typing import Optional, Tuple

import torch

from .. import _lib
from .utils import built_head_dim, last_dim_contiguous, pad_head_dim


def _common_checks(q, k, v, seqlens):
    assert q.dtype == torch.bfloat16 or q.dtype == torch.float16
    assert k.dtype == q.dtype and v.dtype == q.dtype
    assert seqlens.dtype == torch.int32
    batch_size, num_q_heads, head_dim = q.shape
    _, k_len, num_k_heads, _ = k.shape
    _, v_len, num_v_heads, _ = v.shape
    assert k_len == v_len and batch_size == seqlens.shape[0]
    assert num_k_heads == num_v_heads
    assert num_q_heads % num_k_heads == 0
    return batch_size, num_q_heads, num_k_heads, head_dim, k_len


def _strides(q, k, v, o, idx=None):
    vals = [q.stride(0), q.stride(1), k.stride(0), k.stride(1), k.stride(2), v.stride(0), v.stride(1), v.stride(2),
            o.stride(0), o.stride(1)]
    if idx is not None:
        vals += [idx.stride(0), idx.stride(1), idx.stride(2)]
    return _lib.host_i64(vals)


def flash_attention_decode(q, k, v, seqlens, sm_scale: Optional[float] = None) -> torch.Tensor:
    """Dense attention of one query per sequence over the first seqlens[b] rows of k / v.

    q: [batch, num_q_heads, head_dim]; k, v: [batch, kv_len, num_kv_heads, head_dim]; seqlens: int32 [batch].
    """
    B, Hq, Hkv, D, L = _common_checks(q, k, v, seqlens)
    if sm_scale is None:
        sm_scale = 1 / math.sqrt(D)
    if L > 0 and built_head_dim(D) != D:   # head size between the built ones: zero columns appended (copies the slabs)
        return flash_attention_decode(*pad_head_dim(q, k, v), seqlens, sm_scale)[..., :D].contiguous()
    q, k, v = map(last_dim_contiguous, (q, k, v))
    o = torch.empty_like(q, memory_format=torch.contiguous_format)  # the merge kernel writes every element
    if L == 0:
        return o.zero_()
    lib = _lib.load()
    ws = _lib.workspace(lib.nsa_dense_decode_workspace_bytes(B, Hq, Hkv, D, L), q.device)
    rc = lib.nsa_dense_decode(q.data_ptr(), k.data_ptr(), v.data_ptr(), seqlens.data_ptr(), o.data_ptr(), B, Hq, Hkv, D, L,
                              _strides(q, k, v, o), sm_scale, _lib.dtype_code(q), ws.data_ptr(), ws.numel(), _lib.stream_ptr(q))
    _lib.check(rc, "nsa_dense_decode")
    return o


def topk_sparse_attention_decode(q, k, v, topk_idx, block_size: int, seqlens, sm_scale: Optional[float] = None) -> torch.Tensor:
    """Sparse attention of one query per sequence over the KV blocks named by topk_idx [num_kv_heads, batch, topk]."""
    B, Hq, Hkv, D, L = _common_checks(q, k, v, seqlens)
    assert Hkv == topk_idx.shape[0] and B == topk_idx.shape[1]
    assert topk_idx.dtype == torch.int32
    assert block_size in {32, 64, 128, 256}
    topk = topk_idx.shape[-1]
    if sm_scale is None:
        sm_scale = 1 / math.sqrt(D)
    if L > 0 and topk > 0 and built_head_dim(D) != D:
        return topk_sparse_attention_decode(*pad_head_dim(q, k, v), topk_idx, block_size, seqlens, sm_scale)[..., :D].contiguous()
    q, k, v = map(last_dim_contiguous, (q, k, v))
    o = torch.empty_like(q, memory_format=torch.contiguous_format)  # the merge kernel writes every element
    if L == 0 or topk == 0:
        return o.zero_()
    lib = _lib.load()
    ws = _lib.workspace(lib.nsa_topk_decode_workspace_bytes(B, Hq, Hkv, D, topk, block_size), q.device)
    rc = lib.nsa_topk_decode(q.data_ptr(), k.data_ptr(), v.data_ptr(), topk_idx.data_ptr(), seqlens.data_ptr(), o.data_ptr(),
                             B, Hq, Hkv, D, L, topk, block_size, _strides(q, k, v, o, topk_idx), sm_scale, _lib.dtype_code(q),
                             ws.data_ptr(), ws.numel(), _lib.stream_ptr(q))
    _lib.check(rc, "nsa_topk_decode")
    return o


def compressed_attention_decode(
    q, k, v, seqlens, compress_seqlens, kernel_size: int, kernel_stride: int, block_size: int, topk: int,
    init_blocks: int = 1, local_blocks: int = 2, sm_scale: Optional[float] = None, max_seqlen: Optional[int] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Attention over the compressed cache plus selection of the blocks for the sparse branch.

    q: [batch, num_q_heads, head_dim]; k, v: [batch, kv_len, num_kv_heads, head_dim] (compressed slab);
    seqlens: uncompressed length of each sequence including the token being decoded; compress_seqlens:
    compressed length.  Returns (out [batch, num_q_heads, head_dim],
    topk_idx int32 [num_kv_heads, batch, min(topk, ceil(max(seqlens) / block_size))]).
    max_seqlen (not in the reference's signature): max(seqlens) when the caller knows it on the host; the output
    shape then needs no device read.
    """
    assert block_size % kernel_size == 0 and kernel_size % kernel_stride == 0
    B, Hq, Hkv, D, L = _common_checks(q, k, v, seqlens)
    assert compress_seqlens.dtype == torch.int32 and compress_seqlens.shape[0] == B
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    if L == 0:  # input too short to have a compressed token
        return torch.zeros_like(q), torch.zeros(Hkv, B, 1, device=q.device, dtype=torch.int32)
    if built_head_dim(D) != D:
        o, idx = compressed_attention_decode(*pad_head_dim(q, k, v), seqlens, compress_seqlens, kernel_size, kernel_stride, block_size,
                                             topk, init_blocks, local_blocks, sm_scale, max_seqlen)
        return o[..., :D].contiguous(), idx
    q, k, v = map(last_dim_contiguous, (q, k, v))
    if max_seqlen is None:
        max_seqlen = int(seqlens.max())  # fixes the output shape; the reference synchronises here too (:30)
    k_out = min(topk, math.ceil(max_seqlen / block_size))
    o = torch.empty_like(q, memory_format=torch.contiguous_format)  # the merge kernel writes every element
    idx = torch.empty(Hkv, B, k_out, dtype=torch.int32, device=q.device)
    lib = _lib.load()
    ws = _lib.workspace(lib.nsa_cmp_decode_workspace_bytes(B, Hq, Hkv, D, L), q.device)
    rc = lib.nsa_cmp_decode(q.data_ptr(), k.data_ptr(), v.data_ptr(), seqlens.data_ptr(), compress_seqlens.data_ptr(),
                            o.data_ptr(), idx.data_ptr(), B, Hq, Hkv, D, L, kernel_size, kernel_stride, block_size, k_out,
                            max_seqlen, init_blocks, local_blocks, _strides(q, k, v, o, idx), sm_scale, _lib.dtype_code(q),
                            ws.data_ptr(), ws.numel(), _lib.stream_ptr(q))
    _lib.check(rc, "nsa_cmp_decode")
    return o, idx


def decode_branches_gate(q, sparse_k, sparse_v, sparse_len, topk_idx, block_size: int, window_k, window_v, window_len, cmp_out,
                         gate_value, sm_scale: Optional[float] = None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """topk_sparse_attention_decode + flash_attention_decode over the sliding-window ring + the gated sum
    gate[..., 0] * cmp_out + gate[..., 1] * selected + gate[..., 2] * window, as two kernel launches; the results are
    those of the separate calls bit for bit.  Returns (gated sum, selected-branch output, window-branch output).
    No counterpart of its own in the reference (it fuses infer/inference_func.py:140-202 and nsa_inference.py:146-150)."""
    B, Hq, Hkv, D, L = _common_checks(q, sparse_k, sparse_v, sparse_len)
    _, _, _, _, W = _common_checks(q, window_k, window_v, window_len)
    assert Hkv == topk_idx.shape[0] and B == topk_idx.shape[1] and topk_idx.dtype == torch.int32
    assert block_size in {32, 64, 128, 256} and L > 0 and W > 0 and topk_idx.shape[-1] > 0
    assert cmp_out.shape == q.shape and gate_value.shape == (B, Hq, 3) and cmp_out.dtype == gate_value.dtype == q.dtype
    topk = topk_idx.shape[-1]
    if sm_scale is None:
        sm_scale = 1 / math.sqrt(D)
    q, sparse_k, sparse_v, window_k, window_v, cmp_out = map(last_dim_contiguous, (q, sparse_k, sparse_v, window_k, window_v, cmp_out))
    out, o_sel, o_win = (torch.empty_like(q, memory_format=torch.contiguous_format) for _ in range(3))
    lib = _lib.load()
    ws = _lib.workspace(lib.nsa_decode_branches_gate_workspace_bytes(B, Hq, Hkv, D, W, topk, block_size), q.device)
    strides = _lib.host_i64([q.stride(0), q.stride(1), *sparse_k.stride()[:3], *sparse_v.stride()[:3], *topk_idx.stride(),
                             *window_k.stride()[:3], *window_v.stride()[:3], cmp_out.stride(0), cmp_out.stride(1), *gate_value.stride(),
                             out.stride(0), out.stride(1), o_sel.stride(0), o_sel.stride(1), o_win.stride(0), o_win.stride(1)])
    rc = lib.nsa_decode_branches_gate(q.data_ptr(), sparse_k.data_ptr(), sparse_v.data_ptr(), sparse_len.data_ptr(), topk_idx.data_ptr(),
                                      window_k.data_ptr(), window_v.data_ptr(), window_len.data_ptr(), cmp_out.data_ptr(),
                                      gate_value.data_ptr(), out.data_ptr(), o_sel.data_ptr(), o_win.data_ptr(), B, Hq, Hkv, D, L, W, topk,
                                      block_size, strides, sm_scale, _lib.dtype_code(q), ws.data_ptr(), ws.numel(), _lib.stream_ptr(q))
    _lib.check(rc, "nsa_decode_branches_gate")
    return out, o_sel, o_win
