"""GPU parity of compressed_attention (output, gradients, selected block ids) against the oracle."""
import math

import pytest
import torch

import oracle
from helpers import assert_close, assert_ids_match
from native_sparse_attention.ops import avgpool_compress, compressed_attention
from native_sparse_attention.testing import cu_from_lens

pytestmark = pytest.mark.gpu

CASES = [
    # lens, Hq, Hkv, d, ks, st, bs, topk, dtype
    ([1000, 4000, 8192], 32, 8, 96, 32, 16, 64, 16, torch.float16),   # the reference's own test shape
    ([100, 257, 512], 4, 2, 32, 32, 16, 64, 4, torch.bfloat16),
    ([1024, 3000], 64, 4, 128, 32, 16, 64, 16, torch.bfloat16),        # benchmark head layout
    ([40, 700, 31, 65], 6, 2, 64, 32, 16, 64, 5, torch.bfloat16),      # G=3, a sequence with no compressed token
    ([900], 40, 2, 64, 64, 16, 128, 4, torch.float16),                 # G=20 (two head tiles), ks 64 / bs 128
    ([2100], 16, 1, 128, 32, 32, 64, 8, torch.bfloat16),               # non-overlapping windows (pad 0)
    ([17000], 4, 1, 32, 16, 16, 16, 6, torch.bfloat16),                # 1063 blocks: more than a lane keeps in registers
    ([20000, 9000], 2, 1, 32, 16, 16, 16, 6, torch.bfloat16),          # 1250 blocks: the selection runs as three launches
]


def _inputs(lens, Hq, Hkv, d, ks, st, dtype, device, seed=0):
    g = torch.Generator(device=device).manual_seed(seed)
    cu = cu_from_lens(lens, device)
    T = int(cu[-1])
    q = torch.randn(T, Hq, d, generator=g, device=device).to(dtype)
    kx = torch.randn(T, Hkv, d, generator=g, device=device).to(dtype)
    vx = torch.randn(T, Hkv, d, generator=g, device=device).to(dtype)
    ck, cuk = oracle.avgpool_compress(kx.float(), None, cu, ks, st)
    cv, _ = oracle.avgpool_compress(vx.float(), None, cu, ks, st)
    # spread the compressed keys so that attention is not nearly uniform
    return q, (ck * 4).to(dtype), (cv * 4).to(dtype), cu, cuk


@pytest.mark.parametrize("lens,Hq,Hkv,d,ks,st,bs,topk,dtype", CASES)
def test_forward_backward_and_selection(device, lens, Hq, Hkv, d, ks, st, bs, topk, dtype):
    print("case", lens, Hq, Hkv, d, ks, st, bs, topk, dtype, flush=True)
    q, ck, cv, cu, cuk = _inputs(lens, Hq, Hkv, d, ks, st, dtype, device)
    q1, k1, v1 = (x.clone().requires_grad_() for x in (q, ck, cv))
    o, idx = compressed_attention(q1, k1, v1, ks, st, bs, topk, cu, cuk)
    qf, kf, vf = (x.float().requires_grad_() for x in (q, ck, cv))
    want, want_idx, bscore = oracle.compressed_attention(qf, kf, vf, ks, st, bs, topk, cu, cuk, return_scores=True)
    assert_close(o, want, "o")
    g = torch.Generator(device=device).manual_seed(7)
    do = torch.randn(o.shape, generator=g, device=device).to(dtype)
    o.backward(do)
    want.backward(do.float())
    assert_close(q1.grad, qf.grad, "dq", rel_to=qf.grad.abs().max().item())
    assert_close(k1.grad, kf.grad, "dk", rel_to=kf.grad.abs().max().item())
    assert_close(v1.grad, vf.grad, "dv", rel_to=vf.grad.abs().max().item())

    # selection: shape/dtype, structure on every row, bit-exact wherever the oracle's decision margin is clear
    kk = min(topk, math.ceil(max(lens) / bs))
    assert idx.shape == (Hkv, int(cu[-1]), kk) and idx.dtype == torch.int32
    pos = torch.cat([torch.arange(L, device=device) for L in lens])
    qb = pos // bs
    valid = idx >= 0
    assert (valid.sum(-1) == torch.minimum(qb + 1, torch.tensor(kk, device=device))[None]).all()
    assert ((idx <= qb[None, :, None]) | ~valid).all()
    srt = torch.where(valid, idx, torch.full_like(idx, 1 << 30))
    assert (srt[..., 1:] > srt[..., :-1]).logical_or(~valid[..., 1:]).all()          # ascending, -1 right-padded
    assert (idx[..., 0] == 0).all()                                                    # init block
    own = (idx == qb[None, :, None]).any(-1)
    assert own.all()                                                                   # local block
    assert_ids_match(idx, want_idx, bscore, qb, "topk_idx")


def test_topk_disabled_and_given_max_seqlens(device):
    q, ck, cv, cu, cuk = _inputs([300, 200], 8, 2, 64, 32, 16, torch.bfloat16, device)
    with pytest.warns(UserWarning):
        o, idx = compressed_attention(q, ck, cv, 32, 16, 64, -1, cu, cuk, 300, 17)
    assert idx is None
    want, _ = oracle.compressed_attention(q.float(), ck.float(), cv.float(), 32, 16, 64, -1, cu, cuk)
    assert_close(o, want, "o")
    with pytest.raises(AssertionError):
        compressed_attention(q, ck, cv, 32, 16, 64, 2, cu, cuk)          # topk < init_blocks + local_blocks


def test_selection_is_reproducible_on_near_ties(device):
    """Thousands of rows whose block scores nearly tie (tiny queries: every key gets almost the same probability): repeated
    calls must return identical ids, whatever else the GPU is doing in between."""
    lens, Hq, Hkv, d, ks, st, bs, topk = [3000, 5000], 40, 2, 64, 32, 16, 64, 8      # G = 20: two head tiles add into one score
    q, ck, cv, cu, cuk = _inputs(lens, Hq, Hkv, d, ks, st, torch.bfloat16, device, seed=3)
    q = (q.float() * 1e-3).bfloat16()
    _, first = compressed_attention(q, ck, cv, ks, st, bs, topk, cu, cuk)
    _, _, bscore = oracle.compressed_attention(q.float(), ck.float(), cv.float(), ks, st, bs, topk, cu, cuk, return_scores=True)
    top2 = torch.where(torch.isfinite(bscore), bscore, torch.zeros_like(bscore)).topk(topk, -1).values
    assert ((top2[..., :-1] - top2[..., 1:]).abs() < 1e-3).any(-1).float().mean() > 0.5   # most rows do hold near-ties
    noise = torch.randn(4096, 4096, device=device)
    for _ in range(5):
        noise = noise @ noise.T / 4096          # unrelated work between the calls
        _, again = compressed_attention(q, ck, cv, ks, st, bs, topk, cu, cuk)
        assert torch.equal(first, again)


def test_negative_softmax_scale(device):
    q, ck, cv, cu, cuk = _inputs([300, 200], 8, 2, 64, 32, 16, torch.bfloat16, device)
    q = (q.float() * 0.3).bfloat16()
    o, idx = compressed_attention(q, ck, cv, 32, 16, 64, 4, cu, cuk, 300, 17, -0.125)
    want, want_idx, bscore = oracle.compressed_attention(q.float(), ck.float(), cv.float(), 32, 16, 64, 4, cu, cuk, 300, 17, -0.125,
                                                         return_scores=True)
    assert_close(o, want, "o")
    qb = torch.cat([torch.arange(L, device=device) for L in (300, 200)]) // 64
    assert_ids_match(idx, want_idx, bscore, qb, "topk_idx", min_overlap=0.9)


@pytest.mark.parametrize("scale", [-0.2, 0.0])
def test_any_finite_scale_forward_and_backward(device, scale):
    """Every entry point of the compressed-attention family takes any finite softmax scale: forward, selection and both
    backward kernels at a negative and at a zero scale (all probabilities equal among the visible keys)."""
    lens, Hq, Hkv, d, ks, st, bs, topk = [300, 700], 8, 2, 64, 32, 16, 64, 4
    q, ck, cv, cu, cuk = _inputs(lens, Hq, Hkv, d, ks, st, torch.bfloat16, device, seed=5)
    q = (q.float() * 0.3).bfloat16()
    q1, k1, v1 = (x.clone().requires_grad_() for x in (q, ck, cv))
    o, idx = compressed_attention(q1, k1, v1, ks, st, bs, topk, cu, cuk, max(lens), None, scale)
    qf, kf, vf = (x.float().requires_grad_() for x in (q, ck, cv))
    want, want_idx, bscore = oracle.compressed_attention(qf, kf, vf, ks, st, bs, topk, cu, cuk, max(lens), None, scale, return_scores=True)
    assert_close(o, want, "o")
    g = torch.Generator(device=device).manual_seed(8)
    do = torch.randn(o.shape, generator=g, device=device).to(o.dtype)
    o.backward(do)
    want.backward(do.float())
    for name, a, b in (("dq", q1.grad, qf.grad), ("dk", k1.grad, kf.grad), ("dv", v1.grad, vf.grad)):
        assert_close(a, b, name, rel_to=True)
    qb = torch.cat([torch.arange(L, device=device) for L in lens]) // bs
    # at scale 0 every block score ties with its neighbours: only the shape and the forced blocks are fixed
    if scale != 0.0:
        assert_ids_match(idx, want_idx, bscore, qb, "topk_idx", min_overlap=0.9)
    else:
        assert idx.shape == want_idx.shape and (idx[..., 0] == 0).all() and (idx == qb[None, :, None]).any(-1).all()
