"""Oracles for the three single-query (decode) operators over KV-cache slabs.

Test infrastructure only (see package docstring).

* dense:      native_sparse_attention/ops/triton/flash_attention_decode.py:220-258
* top-k:      native_sparse_attention/ops/triton/topk_sparse_attention_decode.py:240-298
* compressed: native_sparse_attention/ops/torch/compressed_attention_decode.py:21-153

Slabs are [B, max_len, Hkv, d]; ``seqlens`` counts the tokens in the cache
including the one being decoded, so the query sits at position seqlens-1.
"""
import math
from typing import Optional

import torch

from .cmp_attn import overlap_weights


def _attend(q, k, v, visible, scale):
    """q [B,Hq,d], k/v [B,L,Hkv,d], visible [B,Hkv,L] -> (o [B,Hq,d], probs fp32 [B,Hkv,G,L])."""
    B, Hq, d = q.shape
    Hkv = k.shape[2]
    G = Hq // Hkv
    s = torch.einsum("bhgd,blhd->bhgl", q.reshape(B, Hkv, G, d), k) * scale
    s = s.masked_fill(~visible[:, :, None, :], float("-inf"))
    acc = torch.float64 if q.dtype == torch.float64 else torch.float32
    p = torch.softmax(s, dim=-1, dtype=acc).nan_to_num(0.0)
    o = torch.einsum("bhgl,blhd->bhgd", p.to(q.dtype), v).reshape(B, Hq, d)
    return o, p


def dense_attention_decode(q, k, v, seqlens, sm_scale: Optional[float] = None):
    """flash_attention_decode.py:220-258 - attend to the first seqlens[b] rows of the slab."""
    B, Hq, d = q.shape
    L, Hkv = k.shape[1], k.shape[2]
    scale = 1.0 / math.sqrt(d) if sm_scale is None else sm_scale
    vis = torch.arange(L, device=q.device)[None, :] < seqlens[:, None].to(torch.int64)
    return _attend(q, k, v, vis[:, None, :].expand(B, Hkv, L), scale)[0]


def topk_sparse_attention_decode(q, k, v, topk_idx, block_size, seqlens, sm_scale: Optional[float] = None):
    """topk_sparse_attention_decode.py:240-298 - union of the selected blocks, cut at seqlens-1."""
    B, Hq, d = q.shape
    L, Hkv = k.shape[1], k.shape[2]
    scale = 1.0 / math.sqrt(d) if sm_scale is None else sm_scale
    pos = torch.arange(L, device=q.device)
    blk = pos // block_size                                          # [L]
    ids = topk_idx.to(torch.int64).permute(1, 0, 2)                  # [B, Hkv, topk]
    picked = ((ids[..., None] == blk[None, None, None, :]) & (ids[..., None] >= 0)).any(2)  # [B,Hkv,L]
    vis = picked & (pos[None, None, :] <= (seqlens.to(torch.int64) - 1)[:, None, None])
    return _attend(q, k, v, vis, scale)[0]


def compressed_attention_decode(
    q, k, v, seqlens, compress_seqlens, kernel_size, kernel_stride, block_size, topk,
    init_blocks: int = 1, local_blocks: int = 2, sm_scale: Optional[float] = None, return_scores: bool = False,
):
    """compressed_attention_decode.py:65-153.

    Returns (out [B,Hq,d], topk_idx [Hkv,B,min(topk, ceil(max(seqlens)/block))] int32);
    an empty compressed slab gives zeros and a [Hkv,B,1] zero index (:105-108).  With ``return_scores`` the
    block scores [Hkv,B,max_blocks] the ids were taken from are returned as well (None for an empty slab).
    """
    assert block_size % kernel_size == 0 and kernel_size % kernel_stride == 0
    B, Hq, d = q.shape
    L, Hkv = k.shape[1], k.shape[2]
    scale = 1.0 / math.sqrt(d) if sm_scale is None else sm_scale
    if L == 0:
        empty = (torch.zeros_like(q), torch.zeros(Hkv, B, 1, dtype=torch.int32, device=q.device))
        return empty + (None,) if return_scores else empty
    vis = torch.arange(L, device=q.device)[None, :] < compress_seqlens[:, None].to(torch.int64)
    o, p = _attend(q, k, v, vis[:, None, :].expand(B, Hkv, L), scale)
    score = p.float().sum(2).permute(1, 0, 2)                        # [Hkv, B, L]
    # block scores (:21-62)
    w, pad = overlap_weights(kernel_size, kernel_stride, block_size)
    r = block_size // kernel_stride
    max_len = int(seqlens.max())
    max_blocks, full_blocks = math.ceil(max_len / block_size), max_len // block_size
    bscore = torch.zeros(Hkv, B, max_blocks, dtype=torch.float32, device=q.device)
    need = (full_blocks - 1) * r + len(w) - pad if full_blocks > 0 else 0
    sp = torch.nn.functional.pad(score, (pad, max(0, need - L) + pad))
    for o_, wo in enumerate(w):
        bscore[..., :full_blocks] += wo * sp[..., o_::r][..., :full_blocks]
    qb = (seqlens.to(torch.int64) - 1) // block_size
    bid = torch.arange(max_blocks, device=q.device)
    forced = (bid[None] < init_blocks) | ((qb[:, None] >= bid[None]) & (qb[:, None] < bid[None] + local_blocks))
    bscore = bscore.masked_fill(forced[None], float("inf")).nan_to_num(0.0, float("inf"), float("-inf"))
    kk = min(topk, max_blocks)
    idx = bscore.topk(kk, dim=-1).indices.sort(-1).values
    idx = torch.where(idx > qb[None, :, None], torch.full_like(idx, -1), idx)
    return (o, idx.to(torch.int32), bscore) if return_scores else (o, idx.to(torch.int32))
