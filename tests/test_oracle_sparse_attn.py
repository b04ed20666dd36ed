"""Pins oracle.sparse_attn against brute force, SDPA and structural invariants (CPU)."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from native_sparse_attention.testing import make_topk_idx


def _brute(q, k, v, idx, bs, cu, scale):
    """Scalar-loop statement of the visibility rule and the softmax."""
    T, Hq, d = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    o = torch.zeros_like(q)
    for b in range(len(cu) - 1):
        for t in range(cu[b], cu[b + 1]):
            i = t - cu[b]
            for h in range(Hq):
                hk = h // G
                blocks = {max(int(e), 0) for e in idx[hk, t].tolist()}
                keys = [j for j in range(i + 1) if (j // bs) in blocks]
                s = torch.tensor([float(q[t, h] @ k[cu[b] + j, hk]) * scale for j in keys], dtype=torch.float64)
                p = torch.exp(s - s.max())
                p = p / p.sum()
                for pj, j in zip(p.tolist(), keys):
                    o[t, h] += pj * v[cu[b] + j, hk]
    return o


def test_matches_brute_force_tiny():
    torch.manual_seed(1)
    cu = [0, 7, 30, 41]
    T, Hq, Hkv, d, bs, topk = 41, 4, 2, 8, 4, 3
    q, k, v = (torch.randn(T, h, d, dtype=torch.float64) for h in (Hq, Hkv, Hkv))
    cu_t = torch.tensor(cu, dtype=torch.int32)
    idx = make_topk_idx(cu_t, bs, topk, Hkv, seed=3, local_blocks=1)
    got = oracle.topk_sparse_attention(q, k, v, idx, bs, cu_t, row_chunk=5)
    want = _brute(q, k, v, idx, bs, cu, 1 / math.sqrt(d))
    assert torch.allclose(got, want, atol=1e-12)


def test_all_blocks_selected_is_causal_sdpa():
    torch.manual_seed(2)
    L, Hq, Hkv, d, bs = 96, 8, 2, 16, 16
    q, k, v = (torch.randn(L, h, d, dtype=torch.float64) for h in (Hq, Hkv, Hkv))
    nb = L // bs
    pos_blk = torch.arange(L) // bs
    idx = torch.arange(nb)[None, None, :].expand(Hkv, L, nb).clone()
    idx = torch.where(idx > pos_blk[None, :, None], torch.full_like(idx, -1), idx).int()
    cu = torch.tensor([0, L], dtype=torch.int32)
    got = oracle.topk_sparse_attention(q, k, v, idx, bs, cu)
    G = Hq // Hkv
    want = F.scaled_dot_product_attention(
        q.permute(1, 0, 2)[None], k.repeat_interleave(G, 1).permute(1, 0, 2)[None],
        v.repeat_interleave(G, 1).permute(1, 0, 2)[None], is_causal=True,
    )[0].permute(1, 0, 2)
    assert torch.allclose(got, want, atol=1e-10)


def test_varlen_equals_per_sequence_and_permutation_invariance():
    torch.manual_seed(3)
    lens = [50, 130, 64]
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
    T, Hq, Hkv, d, bs, topk = int(cu[-1]), 4, 2, 16, 16, 4
    q, k, v = (torch.randn(T, h, d) for h in (Hq, Hkv, Hkv))
    idx = make_topk_idx(cu, bs, topk, Hkv, seed=0)
    full = oracle.topk_sparse_attention(q, k, v, idx, bs, cu)
    for b in range(3):
        s0, s1 = int(cu[b]), int(cu[b + 1])
        one = oracle.topk_sparse_attention(
            q[s0:s1], k[s0:s1], v[s0:s1], idx[:, s0:s1], bs, torch.tensor([0, s1 - s0], dtype=torch.int32)
        )
        assert torch.allclose(full[s0:s1], one, atol=1e-6)
    perm = torch.randperm(topk)
    assert torch.allclose(full, oracle.topk_sparse_attention(q, k, v, idx[..., perm], bs, cu), atol=1e-6)
    rows = [3, 77, 200, 243]
    sub = oracle.topk_sparse_attention(q, k, v, idx, bs, cu, rows=rows)
    assert torch.allclose(sub, full[rows], atol=1e-6)


def test_lse_and_gradcheck():
    torch.manual_seed(4)
    cu = torch.tensor([0, 20, 37], dtype=torch.int32)
    T, Hq, Hkv, d, bs, topk = 37, 2, 1, 4, 4, 3
    q, k, v = (torch.randn(T, h, d, dtype=torch.float64, requires_grad=True) for h in (Hq, Hkv, Hkv))
    idx = make_topk_idx(cu, bs, topk, Hkv, seed=5, local_blocks=1)
    f = lambda a, b, c: oracle.topk_sparse_attention(a, b, c, idx, bs, cu)
    assert torch.autograd.gradcheck(f, (q, k, v), atol=1e-6)
    o, lse = oracle.topk_sparse_attention(q.detach(), k.detach(), v.detach(), idx, bs, cu, return_lse=True)
    # a query at position 0 sees exactly one key: lse = its score
    want = (q[0, 0] @ k[0, 0]).item() / math.sqrt(d)
    assert abs(lse[0, 0].item() - want) < 1e-5


def test_make_topk_idx_structure():
    cu = torch.tensor([0, 512, 1536, 2048], dtype=torch.int32)
    idx = make_topk_idx(cu, 64, 8, 1, seed=0, local_blocks=1)
    assert idx.shape == (1, 2048, 8) and idx.dtype == torch.int32
    for b in range(3):
        s0, s1 = int(cu[b]), int(cu[b + 1])
        for t in (s0, s0 + 63, s0 + 64, s0 + 300, s1 - 1):
            row = idx[0, t].tolist()
            qb = (t - s0) // 64
            valid = [e for e in row if e >= 0]
            assert valid == sorted(set(valid)) and row[len(valid):] == [-1] * (8 - len(valid))
            assert 0 in valid and qb in valid and max(valid) <= qb
            assert len(valid) == min(8, qb + 1)


def test_reverse_index_brute_force():
    cu = torch.tensor([0, 70, 200], dtype=torch.int32)
    bs, topk, Hkv = 16, 4, 2
    idx = make_topk_idx(cu, bs, topk, Hkv, seed=7).numpy()
    cu_blk, offs, qs = oracle.build_reverse_index(idx, cu.numpy(), bs)
    assert cu_blk.tolist() == [0, 5, 14]
    for h in range(Hkv):
        for b in range(2):
            for e in range(cu_blk[b + 1] - cu_blk[b]):
                want = [t for t in range(cu[b], cu[b + 1]) if e in idx[h, t].tolist() and e <= (t - cu[b]) // bs]
                g = cu_blk[b] + e
                assert qs[h, offs[h, g]:offs[h, g + 1]].tolist() == want
