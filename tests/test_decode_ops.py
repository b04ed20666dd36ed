"""GPU parity of the three decode operators (through the C ABI) against the oracle."""
import math

import pytest
import torch

import oracle
from helpers import assert_close, assert_ids_match
from native_sparse_attention.ops import compressed_attention_decode, flash_attention_decode, topk_sparse_attention_decode
from native_sparse_attention.testing import cu_from_lens, make_topk_idx

pytestmark = pytest.mark.gpu


def _slabs(B, L, Hq, Hkv, d, dtype, device, seed=0, extra=0):
    g = torch.Generator(device=device).manual_seed(seed)
    q = torch.empty(B, Hq, d, device=device).uniform_(-1, 1, generator=g).to(dtype)
    # slabs as views of one [2, B+extra, L, Hkv, d] cache, as the reference's callers pass them
    cache = torch.empty(2, B + extra, L, Hkv, d, device=device).uniform_(-1, 1, generator=g).to(dtype)
    return q, cache[0, :B], cache[1, :B]


def _ref_lens(B, max_len, device, seed=1):
    lens = torch.arange(B, dtype=torch.int32) * 128 + 1
    lens[lens > max_len] = max_len
    g = torch.Generator().manual_seed(seed)
    return lens[torch.randperm(B, generator=g)].to(device)


def _decode_idx(lens, bs, topk, Hkv, device):
    rows = []
    for b, L in enumerate(lens.tolist()):
        cu = cu_from_lens([L], device)
        rows.append(make_topk_idx(cu, bs, topk, Hkv, seed=b)[:, L - 1])
    return torch.stack(rows, 1).contiguous()          # [Hkv, B, topk]


@pytest.mark.parametrize("B,max_len,Hq,Hkv,d,dtype", [
    (76, 8192, 32, 4, 128, torch.float16),     # the reference's own check
    (4, 512, 32, 2, 128, torch.bfloat16),      # sliding-window ring of the decode benchmark
    (3, 200, 6, 2, 64, torch.bfloat16),        # G=3
    (2, 130, 40, 2, 96, torch.float16),        # G=20: two head tiles
])
def test_dense_decode(device, B, max_len, Hq, Hkv, d, dtype):
    q, k, v = _slabs(B, max_len, Hq, Hkv, d, dtype, device, extra=1)
    lens = _ref_lens(B, max_len, device)
    o = flash_attention_decode(q, k, v, lens)
    want = oracle.dense_attention_decode(q.float(), k.float(), v.float(), lens)
    assert_close(o, want, "o")


@pytest.mark.parametrize("B,max_len,Hq,Hkv,d,bs,topk,dtype", [
    (76, 8192, 32, 4, 128, 64, 16, torch.float16),   # the reference's own check
    (4, 8193, 32, 2, 128, 64, 8, torch.bfloat16),    # decode benchmark, sparse branch
    (5, 1000, 8, 2, 64, 32, 4, torch.bfloat16),
    (3, 1500, 16, 1, 128, 128, 3, torch.bfloat16),
    (3, 1500, 16, 1, 32, 256, 2, torch.float16),
])
def test_topk_decode(device, B, max_len, Hq, Hkv, d, bs, topk, dtype):
    q, k, v = _slabs(B, max_len, Hq, Hkv, d, dtype, device)
    lens = _ref_lens(B, max_len, device) if B > 5 else torch.tensor([max_len, 64, 65, 700, 1][:B], dtype=torch.int32, device=device)
    idx = _decode_idx(lens, bs, topk, Hkv, device)
    # garbage beyond each sequence's length must never leak into the result
    for b, L in enumerate(lens.tolist()):
        k[b, L:] = float("nan")
        v[b, L:] = float("nan")
    o = topk_sparse_attention_decode(q, k, v, idx, bs, lens)
    want = oracle.topk_sparse_attention_decode(q.float(), k.float().nan_to_num(0.0), v.float().nan_to_num(0.0), idx, bs, lens)
    assert_close(o, want, "o")


@pytest.mark.parametrize("lens,Hq,Hkv,d,topk,dtype", [
    ([2049, 4097, 6145, 8193], 32, 2, 128, 8, torch.bfloat16),   # decode benchmark, compressed branch
    ([40, 100, 31, 700], 8, 2, 64, 16, torch.float16),           # one sequence without compressed tokens
    ([64, 65], 4, 1, 128, 4, torch.bfloat16),
])
def test_compressed_decode(device, lens, Hq, Hkv, d, topk, dtype):
    ks, st, bs = 32, 16, 64
    B = len(lens)
    seqlens = torch.tensor(lens, dtype=torch.int32, device=device)
    clens = torch.tensor([0 if L < ks else (L - ks) // st + 1 for L in lens], dtype=torch.int32, device=device)
    slab = max(int(clens.max()), 1) + 3
    q, k, v = _slabs(B, slab, Hq, Hkv, d, dtype, device)
    o, idx = compressed_attention_decode(q, k, v, seqlens, clens, ks, st, bs, topk)
    want_o, want_idx, bscore = oracle.compressed_attention_decode(q.float(), k.float(), v.float(), seqlens, clens, ks, st, bs, topk,
                                                                  return_scores=True)
    assert_close(o, want_o, "o")
    # exact match wherever the oracle's k-th and (k+1)-th block scores differ by more than 1e-3, then structural invariants
    assert_ids_match(idx, want_idx, bscore, (seqlens.long() - 1) // bs, "decode topk_idx", min_overlap=0.9)
    for b, L in enumerate(lens):
        qb = (L - 1) // bs
        for h in range(Hkv):
            row = idx[h, b].tolist()
            valid = [e for e in row if e >= 0]
            assert row == valid + [-1] * (len(row) - len(valid)) and valid == sorted(set(valid))
            assert len(valid) == min(len(row), qb + 1) and {0, qb, max(qb - 1, 0)} <= set(valid)


def test_compressed_decode_empty_slab(device):
    q = torch.randn(2, 8, 64, device=device).bfloat16()
    k = torch.zeros(2, 0, 2, 64, device=device).bfloat16()
    lens = torch.tensor([5, 9], dtype=torch.int32, device=device)
    o, idx = compressed_attention_decode(q, k, k, lens, torch.zeros_like(lens), 32, 16, 64, 4)
    assert o.abs().max() == 0 and idx.shape == (2, 2, 1) and idx.dtype == torch.int32
