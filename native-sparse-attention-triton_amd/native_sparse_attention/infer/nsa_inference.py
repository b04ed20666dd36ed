"""Prefill / decode orchestration of the three NSA branches over an NSACache.

Counterpart of the reference's nsa_infer (native_sparse_attention/infer/nsa_inference.py:24-151) and of
the per-branch helpers in infer/inference_func.py:27-202, with the same argument order and
conventions: step == 0 is the prefill over varlen tensors, step > 0 decodes one token per
sequence; ``cu_seqlens`` always describes the prompt, so the cache holds prompt_len + step tokens
after the update; ``rope(x, cu_seqlens, step, stride=1)`` is supplied by the caller.
"""
from typing import Callable, Optional, Tuple

import torch

from .. import _lib
from ..ops import (
    avgpool_compress,
    compressed_attention,
    compressed_attention_decode,
    flash_attention_decode,
    linear_compress,
    topk_sparse_attention,
    topk_sparse_attention_decode,
    weightedpool_compress,
)
from ..ops.decode import decode_branches_gate
from ..ops.gated_sum import gate_combine
from ..ops.sliding_window import sliding_window_attention_varlen
from ..ops.utils import get_compressed_seqlens, last_dim_contiguous


def compress_infer(cu_seqlens, step, key, value, cache, weight, compress_func, intra_block_pe, kernel_size, kernel_stride,
                   need_cu=True):
    if step == 0:
        key, compress_cu_seqlens = compress_func[0](key, weight[0], cu_seqlens, kernel_size, kernel_stride, intra_block_pe)
        value, _ = compress_func[1](value, weight[1], cu_seqlens, kernel_size, kernel_stride)
        return key, value, compress_cu_seqlens
    # decode: compress every sequence's staging window -> exactly one candidate token per sequence
    batch = cu_seqlens.shape[0] - 1
    aux_cu = cache.staging_cu_seqlens(batch)
    stage = cache.before_compress_kv_cache[:, :batch].reshape(2, batch * kernel_size, cache.num_kv_heads, cache.head_dim)
    out_cu = cache.staging_out_cu_seqlens(batch)
    key, _ = _compress_known_total(compress_func[0], batch, out_cu, stage[0], weight[0], aux_cu, kernel_size, kernel_stride, intra_block_pe)
    value, _ = _compress_known_total(compress_func[1], batch, out_cu, stage[1], weight[1], aux_cu, kernel_size, kernel_stride)
    if not need_cu:
        return key, value, None
    compress_cu_seqlens = torch.zeros(batch + 1, dtype=torch.int32, device=key.device)
    compress_cu_seqlens[1:] = torch.cumsum(cache.compress_kv_len[:batch], dim=0)  # lengths before this token
    return key, value, compress_cu_seqlens


def _compress_known_total(func, total, out_cu, *args):
    """Call a compression operator; this package's own operators are told the (host-known) number of output rows and
    their cu_seqlens so that they need neither read the one back from the device nor compute the other, any other
    callable gets the reference's arguments only."""
    if func in (weightedpool_compress, avgpool_compress, linear_compress):
        return func(*args, known_total=total, known_y_cu=out_cu)
    return func(*args)


def compressed_attention_infer(cu_seqlens, step, query, key, value, cache, kernel_size, kernel_stride, topk, block_size,
                               init_blocks, local_blocks):
    if step == 0:
        seqlens = cu_seqlens[1:] - cu_seqlens[:-1]
        comp_seqlens, comp_cu = get_compressed_seqlens(cu_seqlens, kernel_size, kernel_stride)
        return compressed_attention(query, key, value, kernel_size, kernel_stride, block_size, topk, cu_seqlens, comp_cu,
                                    int(seqlens.max()), int(comp_seqlens.max()), None, init_blocks, local_blocks)
    batch = cu_seqlens.shape[0] - 1
    seqlens = cache.sparse_kv_len[:batch]  # prompt length + step once the new token is in the cache
    # slab rows that can hold a compressed token at this step, from the host-side length bound (the reference
    # slices by compress_kv_len.max(), inference_func.py:127-135, which waits for the device)
    # (a cache marked static_shapes always passes its full extents, so that a captured step stays valid as sequences grow:
    # the kernels bound their work by the per-sequence lengths anyway; ids of blocks a sequence has not reached come out as -1)
    max_seqlen = cache.max_length if cache.static_shapes else cache.max_seqlen(step)
    rows = min(max((max_seqlen - kernel_size) // kernel_stride + 1, 0), cache.max_comp_length)
    return compressed_attention_decode(query, cache.compress_kv_cache[0, :batch, :rows], cache.compress_kv_cache[1, :batch, :rows],
                                       seqlens, cache.compress_kv_len[:batch], kernel_size, kernel_stride, block_size, topk,
                                       init_blocks, local_blocks, max_seqlen=max_seqlen)


def topk_sparse_attention_infer(cu_seqlens, step, query, key, value, cache, topk_idx, block_size):
    if step == 0:
        return topk_sparse_attention(query, key, value, topk_idx, block_size, cu_seqlens)
    batch = cu_seqlens.shape[0] - 1
    return topk_sparse_attention_decode(query, cache.sparse_kv_cache[0, :batch], cache.sparse_kv_cache[1, :batch], topk_idx,
                                        block_size, cache.sparse_kv_len[:batch])


def sliding_window_attention_infer(cu_seqlens, step, query, key, value, cache, window_size):
    if step == 0:
        return sliding_window_attention_varlen(query, key, value, cu_seqlens, window_size)
    batch = cu_seqlens.shape[0] - 1
    # the ring holds min(tokens seen, window_size) rows; the kernel clips the count to the slab by itself
    return flash_attention_decode(query, cache.sliding_kv_cache[0, :batch], cache.sliding_kv_cache[1, :batch],
                                  cache.sliding_kv_len[:batch])


def nsa_infer(
    cu_seqlens: torch.Tensor,
    step: int,
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    gate_value: torch.Tensor,
    rope,
    cache,
    compress_weight: Tuple[torch.Tensor, torch.Tensor],
    compress_func: Tuple[Callable, Callable],
    intra_block_pe: Optional[torch.Tensor],
    kernel_size: int,
    kernel_stride: int,
    block_size: int,
    topk: int,
    init_blocks: int,
    local_blocks: int,
    window_size: int,
    return_branches: bool = False,
) -> torch.Tensor:
    """Gated sum of the compressed, selected and sliding-window branches; same shape as ``query``."""
    if step == 0:
        cache.reset()
    if step > 0 and _single_launch_prepare_applies(rope, cache, compress_func):
        # pooling compression and this package's rotary module: everything up to the attention branches is one kernel
        assert cache.static_shapes or cache.max_seqlen(step) <= cache.max_length, "cache slab too short for this decode step"
        with torch.no_grad():
            wk, wv = (None if w is None else w.detach().contiguous() for w in compress_weight)
            query = cache.decode_prepare(query, key, value, rope._frequencies(), rope.attention_scaling, wk, wv,
                                         _pooled_position_bias(compress_func[0], wk, intra_block_pe))
        return _decode_branches(cu_seqlens, step, query, key, value, gate_value, cache, kernel_size, kernel_stride, block_size, topk,
                                init_blocks, local_blocks, window_size, return_branches)
    cache.prepare_compress(cu_seqlens, step, key, value)
    # In a decode step every position is a cache length that lives on the device: this package's rotary module can
    # take them from there, any other rope callable gets the reference's (cu_seqlens, step) arguments.
    on_device_positions = step > 0 and hasattr(rope, "rotate_at")
    compress_key, compress_value, compress_cu = compress_infer(
        cu_seqlens, step, key, value, cache, compress_weight, compress_func, intra_block_pe, kernel_size, kernel_stride,
        need_cu=not on_device_positions)
    if on_device_positions:
        batch = cu_seqlens.shape[0] - 1
        query = rope.rotate_at(query, cache.sparse_kv_len[:batch])
        key = rope.rotate_at(key, cache.sparse_kv_len[:batch])
        compress_key = rope.rotate_at(compress_key, cache.compress_kv_len[:batch], stride=cache.kernel_stride)
    else:
        query = rope(query, cu_seqlens, step)
        compress_key = rope(compress_key, compress_cu, step if step == 0 else 1, stride=cache.kernel_stride)
        key = rope(key, cu_seqlens, step)
    cache.update_kv(cu_seqlens, step, compress_key, compress_value, key, value, key, value)
    cmp_out, topk_idx = compressed_attention_infer(cu_seqlens, step, query, compress_key, compress_value, cache, kernel_size,
                                                   kernel_stride, topk, block_size, init_blocks, local_blocks)
    sparse_out = topk_sparse_attention_infer(cu_seqlens, step, query, key, value, cache, topk_idx, block_size)
    window_out = sliding_window_attention_infer(cu_seqlens, step, query, key, value, cache, window_size)
    out = gate_combine(gate_value, cmp_out, sparse_out, window_out)
    if return_branches:
        return out, (cmp_out, sparse_out, window_out, topk_idx)
    return out


def _single_launch_prepare_applies(rope, cache, compress_func) -> bool:
    return (hasattr(rope, "rotate_at") and hasattr(rope, "_frequencies") and hasattr(cache, "decode_prepare")
            and all(f in (weightedpool_compress, avgpool_compress) for f in compress_func) and compress_func[0] is compress_func[1])


def _pooled_position_bias(func, weight, intra_block_pe):
    """The term the pooling operators add to a compressed key for the intra-block position embedding
    (weighted_pool.py:318-321 and :360-362 of the reference), as they compute it."""
    if intra_block_pe is None:
        return None
    if func is weightedpool_compress:
        return torch.einsum("hkd,hk->hd", intra_block_pe, weight).contiguous()
    return torch.mean(intra_block_pe, dim=1).contiguous()


def _decode_branches(cu_seqlens, step, query, key, value, gate_value, cache, kernel_size, kernel_stride, block_size, topk, init_blocks,
                     local_blocks, window_size, return_branches):
    """The three attention branches of a decode step over the updated cache, and their gated sum."""
    cmp_out, topk_idx = compressed_attention_infer(cu_seqlens, step, query, None, None, cache, kernel_size, kernel_stride, topk,
                                                   block_size, init_blocks, local_blocks)
    batch = cu_seqlens.shape[0] - 1
    if topk_idx.shape[-1] > 0 and gate_value.dtype == query.dtype:
        # both remaining branches and the gate in two launches
        out, sparse_out, window_out = decode_branches_gate(
            query, cache.sparse_kv_cache[0, :batch], cache.sparse_kv_cache[1, :batch], cache.sparse_kv_len[:batch], topk_idx, block_size,
            cache.sliding_kv_cache[0, :batch], cache.sliding_kv_cache[1, :batch], cache.sliding_kv_len[:batch], cmp_out, gate_value)
    else:
        sparse_out = topk_sparse_attention_infer(cu_seqlens, step, query, key, value, cache, topk_idx, block_size)
        window_out = sliding_window_attention_infer(cu_seqlens, step, query, key, value, cache, window_size)
        out = gate_combine(gate_value, cmp_out, sparse_out, window_out)
    if return_branches:
        return out, (cmp_out, sparse_out, window_out, topk_idx)
    return out
