"""Head sizes between the compiled ones (48, 80, 112; 40 and 120 for the rotation): the reference serves any head_dim up to
128 by masking inside tiles of next_power_of_2(head_dim) (ops/triton/topk_sparse_attention.py:866, compressed_attention.py:579,
flash_attention_decode.py:185, topk_sparse_attention_decode.py:199).  Every operator is checked against the oracle at the true
head size."""
import math

import pytest
import torch

import oracle
from helpers import assert_close, assert_ids_match
from native_sparse_attention.module.rope import RopeConfig, RotaryEmbedding
from native_sparse_attention.ops import (compressed_attention, compressed_attention_decode, flash_attention_decode,
                                         topk_sparse_attention, topk_sparse_attention_decode)
from native_sparse_attention.ops.flash_attention import flash_attention_varlen
from native_sparse_attention.ops.sliding_window import sliding_window_attention_varlen
from native_sparse_attention.testing import cu_from_lens, make_topk_idx

pytestmark = pytest.mark.gpu

HEAD_DIMS = [48, 80, 112]


def _qkv(lens, Hq, Hkv, d, dtype, device, seed=0):
    g = torch.Generator(device=device).manual_seed(seed)
    cu = cu_from_lens(lens, device)
    T = int(cu[-1])
    q = torch.randn(T, Hq, d, generator=g, device=device).to(dtype)
    k = torch.randn(T, Hkv, d, generator=g, device=device).to(dtype)
    v = torch.randn(T, Hkv, d, generator=g, device=device).to(dtype)
    do = torch.randn(T, Hq, d, generator=g, device=device).to(dtype)
    return q, k, v, do, cu


@pytest.mark.parametrize("d", HEAD_DIMS)
def test_topk_sparse_attention(device, d):
    lens, Hq, Hkv, bs, topk = [700, 1300, 90], 16, 2, 64, 6
    q, k, v, do, cu = _qkv(lens, Hq, Hkv, d, torch.bfloat16, device)
    idx = make_topk_idx(cu, bs, topk, Hkv, seed=1)
    q1, k1, v1 = (x.clone().requires_grad_() for x in (q, k, v))
    o = topk_sparse_attention(q1, k1, v1, idx, bs, cu)
    assert o.shape == q.shape and o.is_contiguous()
    o.backward(do)
    qf, kf, vf = (x.float().requires_grad_() for x in (q, k, v))
    want = oracle.topk_sparse_attention(qf, kf, vf, idx, bs, cu)   # default scale: 1 / sqrt(d) of the TRUE head size
    want.backward(do.float())
    assert_close(o, want, "o")
    for name, a, b in (("dq", q1.grad, qf.grad), ("dk", k1.grad, kf.grad), ("dv", v1.grad, vf.grad)):
        assert a.shape == b.shape
        assert_close(a, b, name, rel_to=True)


@pytest.mark.parametrize("d", HEAD_DIMS)
def test_compressed_attention_and_selection(device, d):
    lens, Hq, Hkv, ks, st, bs, topk = [1024, 3000], 8, 2, 32, 16, 64, 8
    q, kx, vx, do, cu = _qkv(lens, Hq, Hkv, d, torch.bfloat16, device, seed=2)
    ck, cuk = oracle.avgpool_compress(kx.float(), None, cu, ks, st)
    cv, _ = oracle.avgpool_compress(vx.float(), None, cu, ks, st)
    ck, cv = (ck * 4).bfloat16(), (cv * 4).bfloat16()
    q1, k1, v1 = (x.clone().requires_grad_() for x in (q, ck, cv))
    o, idx = compressed_attention(q1, k1, v1, ks, st, bs, topk, cu, cuk)
    o.backward(do)
    qf, kf, vf = (x.float().requires_grad_() for x in (q, ck, cv))
    want, want_idx, bscore = oracle.compressed_attention(qf, kf, vf, ks, st, bs, topk, cu, cuk, return_scores=True)
    want.backward(do.float())
    assert_close(o, want, "o")
    for name, a, b in (("dq", q1.grad, qf.grad), ("dk", k1.grad, kf.grad), ("dv", v1.grad, vf.grad)):
        assert_close(a, b, name, rel_to=True)
    pos = torch.cat([torch.arange(L, device=device) for L in lens])
    assert_ids_match(idx, want_idx, bscore, pos // bs, "topk_idx d=%d" % d)


@pytest.mark.parametrize("d", HEAD_DIMS)
def test_dense_and_window_attention(device, d):
    lens, Hq, Hkv = [333, 800], 8, 2
    q, k, v, do, cu = _qkv(lens, Hq, Hkv, d, torch.float16, device, seed=3)
    pos = torch.cat([torch.arange(L, device=device) for L in lens])
    seq = torch.cat([torch.full((L,), i, device=device) for i, L in enumerate(lens)])
    same = seq[:, None] == seq[None, :]
    kr, vr = k.float().repeat_interleave(Hq // Hkv, 1), v.float().repeat_interleave(Hq // Hkv, 1)
    s = torch.einsum("ihd,jhd->hij", q.float(), kr) / math.sqrt(d)
    for name, mask, got in (
        ("causal", same & (pos[None, :] <= pos[:, None]), flash_attention_varlen(q, k, v, cu, cu, max(lens), max(lens), causal=True)),
        ("window 100", same & (pos[None, :] <= pos[:, None]) & (pos[None, :] >= pos[:, None] - 100), sliding_window_attention_varlen(q, k, v, cu, 100)),
    ):
        p = torch.softmax(s.masked_fill(~mask[None], float("-inf")), -1)
        want = torch.einsum("hij,jhd->ihd", p.to(torch.float16).float(), vr)
        assert got.shape == q.shape
        assert_close(got, want, name)


@pytest.mark.parametrize("d", HEAD_DIMS)
def test_decode_operators(device, d):
    B, L, Hq, Hkv, bs, topk, ks, st = 3, 700, 8, 2, 64, 4, 32, 16
    g = torch.Generator(device=device).manual_seed(4)
    q = torch.empty(B, Hq, d, device=device).uniform_(-1, 1, generator=g).bfloat16()
    cache = torch.empty(2, B + 1, L, Hkv, d, device=device).uniform_(-1, 1, generator=g).bfloat16()
    k, v = cache[0, :B], cache[1, :B]
    lens = torch.tensor([700, 130, 401], dtype=torch.int32, device=device)
    assert_close(flash_attention_decode(q, k, v, lens), oracle.dense_attention_decode(q.float(), k.float(), v.float(), lens), "dense decode")
    idx = torch.stack([make_topk_idx(cu_from_lens([n], device), bs, topk, Hkv, seed=b)[:, n - 1] for b, n in enumerate(lens.tolist())], 1).contiguous()
    assert_close(topk_sparse_attention_decode(q, k, v, idx, bs, lens),
                 oracle.topk_sparse_attention_decode(q.float(), k.float(), v.float(), idx, bs, lens), "topk decode")
    clens = torch.div(lens - ks, st, rounding_mode="floor").to(torch.int32) + 1
    Lc = int(clens.max())
    o, sel = compressed_attention_decode(q, k[:, :Lc], v[:, :Lc], lens, clens, ks, st, bs, topk)
    want, want_sel = oracle.compressed_attention_decode(q.float(), k[:, :Lc].float(), v[:, :Lc].float(), lens, clens, ks, st, bs, topk)
    assert_close(o, want, "compressed decode")
    assert sel.shape == want_sel.shape
    assert (sel == want_sel).float().mean().item() > 0.9


@pytest.mark.parametrize("d", [40, 48, 80, 112, 120])
def test_rotation(device, d):
    lens, H = [100, 257], 4
    g = torch.Generator(device=device).manual_seed(5)
    cu = cu_from_lens(lens, device)
    rope = RotaryEmbedding(RopeConfig(head_dim=d), device=device)
    x = torch.randn(int(cu[-1]), H, d, generator=g, device=device).bfloat16()
    pos = torch.cat([torch.arange(L, device=device) for L in lens])
    y = rope(x, cu)
    freqs = pos.float()[:, None] * rope.inv_freq.float()[None, :]
    cos = torch.cat([freqs.cos(), freqs.cos()], -1).to(x.dtype)[:, None, :]
    sin = torch.cat([freqs.sin(), freqs.sin()], -1).to(x.dtype)[:, None, :]
    want = x * cos + torch.cat((-x[..., d // 2:], x[..., :d // 2]), dim=-1) * sin
    assert ((y.float() - want.float()).abs() <= 2.0 ** -7 * want.float().abs().clamp(min=1.0)).all()
    assert (y == want).float().mean() > 0.98
