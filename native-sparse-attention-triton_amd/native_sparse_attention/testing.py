"""Synthetic workload generators shared by the tests and the benchmark."""
from typing import Optional

import torch


def make_topk_idx(
    cu_seqlens: torch.Tensor,
    block_size: int,
    topk: int,
    num_kv_heads: int,
    seed: int = 0,
    local_blocks: int = 2,
    device: Optional[torch.device] = None,
    row_chunk: int = 8192,
) -> torch.Tensor:
    """Causal block selection [num_kv_heads, T, topk] int32 in the layout the sparse kernels expect.

    For a token at position p of its sequence (own block qb = p // block_size) the row
    holds block 0, the ``local_blocks`` blocks ending at qb, and distinct uniformly
    drawn earlier blocks up to ``min(topk, qb + 1)`` entries; entries are ascending
    and the unused tail is -1.  Same convention as generate_topk_idx_example in the
    reference's test/test_topk_sparse_attention.py:34-86 (sorted, block 0 forced,
    causal, -1 right padding), with the local blocks forced as well.
    """
    device = torch.device(device) if device is not None else cu_seqlens.device
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    cu = [int(c) for c in cu_seqlens.tolist()]
    T = cu[-1]
    out = torch.full((num_kv_heads, T, topk), -1, dtype=torch.int32, device=device)
    for b in range(len(cu) - 1):
        L = cu[b + 1] - cu[b]
        nblk = (L + block_size - 1) // block_size
        kk = min(topk, nblk)
        if kk == 0:
            continue
        bid = torch.arange(nblk, device=device)
        for h in range(num_kv_heads):
            for r0 in range(0, L, row_chunk):
                pos = torch.arange(r0, min(L, r0 + row_chunk), device=device)
                qb = pos // block_size
                w = torch.rand((pos.numel(), nblk), generator=gen, device=device)
                forced = (bid[None] == 0) | ((bid[None] <= qb[:, None]) & (bid[None] > qb[:, None] - local_blocks))
                w = torch.where(forced, torch.full_like(w, 2.0), w)
                w = torch.where(bid[None] > qb[:, None], torch.full_like(w, -1.0), w)
                val, sel = w.topk(kk, dim=-1)
                sel = torch.where(val < 0, torch.full_like(sel, nblk + topk), sel).sort(-1).values
                sel = torch.where(sel >= nblk, torch.full_like(sel, -1), sel)
                out[h, cu[b] + r0 : cu[b] + r0 + pos.numel(), :kk] = sel.to(torch.int32)
    return out


def cu_from_lens(lens, device=None) -> torch.Tensor:
    t = torch.tensor([0] + list(lens), dtype=torch.int64).cumsum(0).to(torch.int32)
    return t.to(device) if device is not None else t
