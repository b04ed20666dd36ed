"""Oracle for attention over compressed keys plus the block-score / top-k selection.

Test infrastructure only (see package docstring).

Follows native_sparse_attention/ops/torch/compressed_attention.py:21-194 of the
reference:

* query at position ``i`` of its sequence sees compressed key ``c`` of the same
  sequence iff ``i >= c*stride + kernel - 1`` (:127-133); rows that see nothing
  give exactly 0 (:141-142);
* softmax in fp32, cast to the value dtype for the output product (:143-145);
* score[h_kv, t, c] = sum over the G query heads of the fp32 probabilities (:156);
* block score = overlap-weighted sum of the scores of the compressed tokens that
  touch the block (:34-53), computed for the first ``max_seqlen_q // block``
  blocks only, then +inf on the ``init_blocks`` first blocks and on the
  ``local_blocks`` blocks ending at the query's own block (:63-70);
* ``topk_idx`` = indices of the ``min(topk, ceil(max_seqlen_q/block))`` largest
  block scores, ascending, entries beyond the query's block replaced by -1
  (:190-193).
"""
import math
from typing import Optional, Tuple

import torch


def overlap_weights(kernel_size: int, kernel_stride: int, block_size: int):
    """Weights w[o] applied to score[b*(bs/st) + o - pad], pad = ks/st - 1 (:34,45-49)."""
    a, r = kernel_size // kernel_stride, block_size // kernel_stride
    w = [0] * (a + r - 1)
    for i in range(a):
        for j in range(r):
            w[i + j] += 1
    return w, a - 1


def block_scores_from_probs(
    score: torch.Tensor,      # [Hkv, rows, max_k] fp32, zero beyond each row's sequence
    q_pos: torch.Tensor,      # [rows] position of each row inside its own sequence
    kernel_size: int,
    kernel_stride: int,
    block_size: int,
    max_seqlen_q: int,
    init_blocks: int = 1,
    local_blocks: int = 2,
) -> torch.Tensor:
    """transform_score, compressed_attention.py:21-71."""
    Hkv, R, max_k = score.shape
    w, pad = overlap_weights(kernel_size, kernel_stride, block_size)
    r = block_size // kernel_stride
    max_blocks = math.ceil(max_seqlen_q / block_size)
    full_blocks = max_seqlen_q // block_size
    out = torch.zeros(Hkv, R, max_blocks, dtype=torch.float32, device=score.device)
    need = (full_blocks - 1) * r + len(w) - pad if full_blocks > 0 else 0
    sp = torch.nn.functional.pad(score.float(), (pad, max(0, need - max_k) + pad))
    for o, wo in enumerate(w):
        # padded index o + b*r  <->  compressed token b*r + o - pad
        out[..., :full_blocks] += wo * sp[..., o :: r][..., :full_blocks]
    qb = (q_pos // block_size).to(score.device)
    bid = torch.arange(max_blocks, device=score.device)
    forced = (bid[None, :] < init_blocks) | ((qb[:, None] >= bid[None, :]) & (qb[:, None] < bid[None, :] + local_blocks))
    out = out.masked_fill(forced[None], float("inf"))
    return out


def select_topk(block_score: torch.Tensor, q_pos: torch.Tensor, block_size: int, topk: int) -> torch.Tensor:
    """compressed_attention.py:190-193."""
    kk = min(topk, block_score.shape[-1])
    idx = block_score.topk(kk, dim=-1).indices.sort(-1).values
    qb = (q_pos // block_size).to(idx.device)
    idx = torch.where(idx > qb[None, :, None], torch.full_like(idx, -1), idx)
    return idx.to(torch.int32)


def compressed_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    kernel_size: int,
    kernel_stride: int,
    block_size: int,
    topk: int,
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_k: torch.Tensor,
    max_seqlen_q: Optional[int] = None,
    max_seqlen_k: Optional[int] = None,
    sm_scale: Optional[float] = None,
    init_blocks: int = 1,
    local_blocks: int = 2,
    row_chunk: int = 512,
    return_scores: bool = False,
):
    """Returns (out [T,Hq,d], topk_idx [Hkv,T,k'] int32 or None [, block_score])."""
    assert block_size % kernel_size == 0 and kernel_size % kernel_stride == 0
    T, Hq, d = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    scale = 1.0 / math.sqrt(d) if sm_scale is None else sm_scale
    cq = [int(x) for x in cu_seqlens_q.tolist()]
    ck = [int(x) for x in cu_seqlens_k.tolist()]
    if max_seqlen_q is None:
        max_seqlen_q = max(b - a for a, b in zip(cq[:-1], cq[1:]))
    if max_seqlen_k is None:
        max_seqlen_k = max(b - a for a, b in zip(ck[:-1], ck[1:]))
    dev = q.device
    outs, scores, poss = [], [], []
    acc_dtype = torch.float64 if q.dtype == torch.float64 else torch.float32
    for b in range(len(cq) - 1):
        Lq, Lk = cq[b + 1] - cq[b], ck[b + 1] - ck[b]
        kb, vb = k[ck[b] : ck[b + 1]], v[ck[b] : ck[b + 1]]
        last_tok = torch.arange(Lk, device=dev) * kernel_stride + kernel_size - 1
        for r0 in range(0, Lq, row_chunk):
            r1 = min(Lq, r0 + row_chunk)
            pos = torch.arange(r0, r1, device=dev)
            vis = pos[:, None] >= last_tok[None, :]                     # [r, Lk]
            qq = q[cq[b] + r0 : cq[b] + r1].reshape(r1 - r0, Hkv, G, d)
            s = torch.einsum("rhgd,lhd->hgrl", qq, kb) * scale
            s = s.masked_fill(~vis[None, None], float("-inf"))
            p = torch.softmax(s, dim=-1, dtype=acc_dtype).nan_to_num(0.0)
            o = torch.einsum("hgrl,lhd->rhgd", p.to(v.dtype), vb).reshape(r1 - r0, Hq, d)
            outs.append(o)
            if topk > 0:
                sc = torch.zeros(Hkv, r1 - r0, max_seqlen_k, dtype=torch.float32, device=dev)
                sc[..., :Lk] = p.detach().float().sum(1)
                scores.append(sc)
                poss.append(pos)
    out = torch.cat(outs, 0) if outs else q.new_zeros(q.shape)
    if topk <= 0:
        return (out, None, None) if return_scores else (out, None)
    assert topk >= init_blocks + local_blocks
    with torch.no_grad():
        q_pos = torch.cat(poss)
        bs_all = block_scores_from_probs(
            torch.cat(scores, 1), q_pos, kernel_size, kernel_stride, block_size, max_seqlen_q, init_blocks, local_blocks
        )
        idx = select_topk(bs_all, q_pos, block_size, topk)
    return (out, idx, bs_all) if return_scores else (out, idx)
