"""Oracle for block-sparse GQA attention over the KV blocks named by ``topk_idx``.

Test infrastructure only (see package docstring).

Follows native_sparse_attention/ops/torch/topk_sparse_attention.py:19-83 of the
reference: key ``j`` of a sequence is visible to query ``i`` of the same
sequence iff ``j <= i`` and ``j // block_size`` is one of the ids in
``topk_idx[h_kv, t, :]``; negative ids are treated as block 0 (:66); q-head
``h`` reads kv-head ``h // G`` (:77); softmax in fp32, probabilities cast to the
input dtype before the value product (:81-82).

The reference materialises a dense [H, T, T] mask; this restatement walks
sequences and row chunks so that long sequences fit in memory, and can be asked
for a subset of rows only.
"""
import math
from typing import Optional, Sequence

import numpy as np
import torch


def _seq_of_rows(cu, rows):
    cu_t = torch.as_tensor(cu, dtype=torch.int64)
    return torch.bucketize(rows, cu_t[1:], right=True)


def topk_sparse_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    topk_idx: torch.Tensor,
    block_size: int,
    cu_seqlens: torch.Tensor,
    softmax_scale: Optional[float] = None,
    rows: Optional[Sequence[int]] = None,
    row_chunk: int = 512,
    return_lse: bool = False,
):
    """q [T,Hq,d], k/v [T,Hkv,d], topk_idx [Hkv,T,topk] -> o [T,Hq,d] (or [len(rows),Hq,d]).

    ``rows`` restricts the computation to the given global token indices (the
    result then has one output row per entry, in that order).  With
    ``return_lse`` the natural-log LSE [Hq, rows] is returned as well.
    """
    T, Hq, d = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    scale = 1.0 / math.sqrt(d) if softmax_scale is None else softmax_scale
    cu = [int(x) for x in cu_seqlens.tolist()]
    dev = q.device
    if rows is None:
        row_ids = torch.arange(T, device=dev)
    else:
        row_ids = torch.as_tensor(list(rows), dtype=torch.int64, device=dev)
    seq_of = _seq_of_rows(cu, row_ids.cpu()).to(dev)
    order_chunks = []
    for b in range(len(cu) - 1):
        sel = torch.nonzero(seq_of == b).flatten()
        for c0 in range(0, sel.numel(), row_chunk):
            order_chunks.append((b, sel[c0 : c0 + row_chunk]))
    result = q.new_zeros((row_ids.numel(), Hq, d))
    lse_res = torch.zeros((Hq, row_ids.numel()), dtype=torch.float32, device=dev)
    pieces = []
    for b, where in order_chunks:
        s0, s1 = cu[b], cu[b + 1]
        L = s1 - s0
        nblk = (L + block_size - 1) // block_size
        t = row_ids[where]                      # global token ids of this chunk
        pos = t - s0                            # position inside the sequence
        key_pos = torch.arange(L, device=dev)
        causal = key_pos[None, :] <= pos[:, None]            # [r, L]
        ks = k[s0:s1]
        vs = v[s0:s1]
        o_heads = []
        lse_heads = []
        for h in range(Hkv):
            ids = topk_idx[h, t].to(torch.int64).clamp(min=0)  # negative -> block 0
            assert int(ids.max()) < nblk, "block id beyond the sequence"
            picked = torch.zeros((t.numel(), nblk), dtype=torch.bool, device=dev)
            picked.scatter_(1, ids, True)
            vis = picked[:, key_pos // block_size] & causal  # [r, L]
            qh = q[t, h * G : (h + 1) * G]                   # [r, G, d]
            s = torch.einsum("rgd,ld->grl", qh, ks[:, h]) * scale
            s = s.masked_fill(~vis[None], float("-inf"))
            p32 = torch.softmax(s, dim=-1, dtype=torch.float32 if s.dtype != torch.float64 else torch.float64)
            p = p32.to(q.dtype)
            o_heads.append(torch.einsum("grl,ld->rgd", p, vs[:, h]))
            if return_lse:
                lse_heads.append(torch.logsumexp(s.float(), dim=-1))  # [G, r]
        pieces.append((where, torch.cat(o_heads, dim=1)))
        if return_lse:
            lse_res[:, where] = torch.cat(lse_heads, dim=0)
    if pieces:
        idx = torch.cat([w for w, _ in pieces])
        val = torch.cat([o for _, o in pieces], dim=0)
        result = result.index_copy(0, idx, val)
    if return_lse:
        return result, lse_res
    return result


def build_reverse_index(topk_idx: np.ndarray, cu_seqlens: np.ndarray, block_size: int):
    """CSR "KV block -> queries that selected it" index (integer work, numpy).

    Follows native_sparse_attention/ops/triton/topk_sparse_attention.py:960-981
    (count_query + reorder_topk_idx): a query at position ``p`` of its sequence
    contributes entry ``e`` iff ``0 <= e <= p // block_size`` (:89-93).  Blocks
    are numbered globally as ``cu_seqblocks[b] + e`` with
    ``cu_seqblocks = cumsum(ceil(len / block_size))``.

    Returns (cu_seqblocks [B+1], offsets [Hkv, total_blocks+1], queries [Hkv, max_total])
    where ``queries[h, offsets[h,g]:offsets[h,g+1]]`` are the global token ids,
    ascending, that selected global block ``g`` of head ``h``; unused tail = -1.
    """
    topk_idx = np.asarray(topk_idx)
    cu = np.asarray(cu_seqlens, dtype=np.int64)
    Hkv, T, K = topk_idx.shape
    lens = cu[1:] - cu[:-1]
    nblk = (lens + block_size - 1) // block_size
    cu_blk = np.concatenate([[0], np.cumsum(nblk)]).astype(np.int64)
    total_blocks = int(cu_blk[-1])
    seq_of = np.searchsorted(cu[1:], np.arange(T), side="right")
    pos = np.arange(T) - cu[seq_of]
    qblk = pos // block_size
    valid = (topk_idx >= 0) & (topk_idx <= qblk[None, :, None])
    gblk = topk_idx.astype(np.int64) + cu_blk[seq_of][None, :, None]
    offsets = np.zeros((Hkv, total_blocks + 1), dtype=np.int32)
    lists = []
    for h in range(Hkv):
        tt, kk = np.nonzero(valid[h])
        g = gblk[h, tt, kk]
        order = np.lexsort((tt, g))          # by block, then by token
        lists.append(tt[order].astype(np.int32))
        counts = np.bincount(g, minlength=total_blocks)
        offsets[h, 1:] = np.cumsum(counts)
    width = max((len(x) for x in lists), default=0)
    queries = np.full((Hkv, width), -1, dtype=np.int32)
    for h, x in enumerate(lists):
        queries[h, : len(x)] = x
    return cu_blk.astype(np.int32), offsets, queries
