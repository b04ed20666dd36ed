"""GPU parity of topk_sparse_attention (through the C ABI) against the oracle."""
import pytest
import torch

import oracle
from helpers import assert_close
from native_sparse_attention.ops import topk_sparse_attention
from native_sparse_attention.testing import cu_from_lens, make_topk_idx

pytestmark = pytest.mark.gpu

CASES = [
    # lens, Hq, Hkv, d, block, topk, dtype, local_blocks
    ([512, 1024, 512], 16, 1, 64, 64, 8, torch.bfloat16, 1),          # shape of the reference's CPU-runnable test
    ([1000, 2000, 4096], 64, 8, 96, 64, 5, torch.float16, 1),         # the reference's own test shape
    ([2048], 64, 4, 128, 64, 16, torch.bfloat16, 2),                  # sweep shape, small N
    ([4096], 64, 4, 128, 64, 8, torch.bfloat16, 2),
    ([12, 576, 130, 1], 8, 2, 128, 32, 4, torch.bfloat16, 2),         # ragged, sequences shorter than a block
    ([700, 300], 6, 2, 64, 128, 3, torch.bfloat16, 1),                # G=3, big blocks
    ([300, 900], 32, 1, 32, 256, 2, torch.float16, 1),                # G=32: two head tiles per token
]


def _make(lens, Hq, Hkv, d, dtype, device, seed=0):
    g = torch.Generator(device=device).manual_seed(seed)
    cu = cu_from_lens(lens, device)
    T = int(cu[-1])
    q = torch.randn(T, Hq, d, generator=g, device=device).to(dtype)
    k = torch.randn(T, Hkv, d, generator=g, device=device).to(dtype)
    v = torch.randn(T, Hkv, d, generator=g, device=device).to(dtype)
    return q, k, v, cu


@pytest.mark.parametrize("lens,Hq,Hkv,d,bs,topk,dtype,local", CASES)
def test_forward_matches_oracle(device, lens, Hq, Hkv, d, bs, topk, dtype, local):
    print("case", lens, Hq, Hkv, d, bs, topk, dtype, flush=True)
    q, k, v, cu = _make(lens, Hq, Hkv, d, dtype, device)
    idx = make_topk_idx(cu, bs, topk, Hkv, seed=1, local_blocks=local)
    o = topk_sparse_attention(q, k, v, idx, bs, cu)
    torch.cuda.synchronize()
    want = oracle.topk_sparse_attention(q.float(), k.float(), v.float(), idx, bs, cu)
    assert o.dtype == dtype and o.shape == q.shape
    assert_close(o, want, "o")


def test_forward_strided_views_and_scale(device):
    lens, Hq, Hkv, d, bs, topk = [333, 800], 16, 2, 128, 64, 6
    cu = cu_from_lens(lens, device)
    T = int(cu[-1])
    g = torch.Generator(device=device).manual_seed(5)
    qkv = torch.randn(T, Hq + 2 * Hkv, d, generator=g, device=device).to(torch.bfloat16)
    q, k, v = qkv[:, :Hq], qkv[:, Hq:Hq + Hkv], qkv[:, Hq + Hkv:]
    idx_full = make_topk_idx(cu, bs, topk + 2, Hkv, seed=2)
    idx = idx_full.permute(1, 0, 2).contiguous().permute(1, 0, 2)      # non-standard strides
    o = topk_sparse_attention(q, k, v, idx, bs, cu, softmax_scale=0.05)
    want = oracle.topk_sparse_attention(q.float(), k.float(), v.float(), idx, bs, cu, softmax_scale=0.05)
    assert_close(o, want, "o")


def test_rejects_bad_dtypes(device):
    q = torch.randn(64, 4, 64, device=device)
    cu = cu_from_lens([64], device)
    idx = make_topk_idx(cu, 64, 1, 1)
    with pytest.raises(AssertionError):
        topk_sparse_attention(q, q[:, :1], q[:, :1], idx, 64, cu)             # fp32 not accepted
    qb = q.bfloat16()
    with pytest.raises(AssertionError):
        topk_sparse_attention(qb, qb[:, :1], qb[:, :1], idx.long(), 64, cu)   # idx must be int32
    with pytest.raises(AssertionError):
        topk_sparse_attention(qb, qb[:, :1], qb[:, :1], idx, 48, cu)          # block size set


def _grad_check(device, lens, Hq, Hkv, d, bs, topk, dtype, local, seed=0):
    q, k, v, cu = _make(lens, Hq, Hkv, d, dtype, device, seed)
    idx = make_topk_idx(cu, bs, topk, Hkv, seed=1, local_blocks=local)
    g = torch.Generator(device=device).manual_seed(9)
    do = torch.randn(q.shape, generator=g, device=device).to(dtype)
    q1, k1, v1 = (x.clone().requires_grad_() for x in (q, k, v))
    o = topk_sparse_attention(q1, k1, v1, idx, bs, cu)
    o.backward(do)
    qf, kf, vf = (x.float().requires_grad_() for x in (q, k, v))
    want = oracle.topk_sparse_attention(qf, kf, vf, idx, bs, cu)
    want.backward(do.float())
    # gradients of early keys sum over thousands of queries: bound errors relative to the
    # largest reference magnitude when that exceeds 1 (bf16 output rounding alone is 2^-9 relative)
    for name, got, ref in (("dq", q1.grad, qf.grad), ("dk", k1.grad, kf.grad), ("dv", v1.grad, vf.grad)):
        assert_close(got, ref, name, rel_to=ref.abs().max().item())


@pytest.mark.parametrize("lens,Hq,Hkv,d,bs,topk,dtype,local", CASES)
def test_backward_matches_oracle(device, lens, Hq, Hkv, d, bs, topk, dtype, local):
    print("case", lens, Hq, Hkv, d, bs, topk, dtype, flush=True)
    _grad_check(device, lens, Hq, Hkv, d, bs, topk, dtype, local)


def test_reverse_index_bit_exact_and_deterministic(device):
    from native_sparse_attention.ops.topk_sparse_attention import _topk_sparse_attention_bwd, _topk_sparse_attention_fwd
    lens, Hq, Hkv, d, bs, topk = [700, 64, 1500], 16, 2, 64, 64, 6
    q, k, v, cu = _make(lens, Hq, Hkv, d, torch.bfloat16, device)
    idx = make_topk_idx(cu, bs, topk, Hkv, seed=4)
    o, lse = _topk_sparse_attention_fwd(q, k, v, idx, bs, cu, cu, None, None, d ** -0.5)
    do = torch.randn_like(o)
    dq, dk, dv, seg_off, queries = _topk_sparse_attention_bwd(
        o, do, lse, q, k, v, idx, bs, cu, cu, None, None, d ** -0.5, return_reverse_index=True)
    cu_blk, offs, qs = oracle.build_reverse_index(idx.cpu().numpy(), cu.cpu().numpy(), bs)
    T, B = int(cu[-1]), len(lens)
    max_blocks = T // bs + B
    seg_off, queries = seg_off.cpu().numpy(), queries.cpu().numpy()
    total_blocks = int(cu_blk[-1])
    for h in range(Hkv):
        for g in range(total_blocks):
            s = h * max_blocks + g
            got = queries[seg_off[s]:seg_off[s + 1]].tolist()
            assert got == qs[h, offs[h, g]:offs[h, g + 1]].tolist(), (h, g)
        for g in range(total_blocks, max_blocks):                      # unused segments are empty
            s = h * max_blocks + g
            assert seg_off[s] == seg_off[s + 1]
    dq2, dk2, dv2 = _topk_sparse_attention_bwd(o, do, lse, q, k, v, idx, bs, cu, cu, None, None, d ** -0.5)
    assert torch.equal(dq, dq2) and torch.equal(dk, dk2) and torch.equal(dv, dv2)
