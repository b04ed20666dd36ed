"""GPU parity on batches that contain zero-length sequences (cu_seqlens with repeated entries): every training-side
operator, through the C ABI, against the oracle.  The reference's scripts never pass such a batch; a varlen
batch assembled from a data loader can."""
import pytest
import torch

import oracle
from helpers import assert_close
from native_sparse_attention.ops import (compressed_attention, flash_attention_varlen, linear_compress,
                                         topk_sparse_attention, weightedpool_compress)
from native_sparse_attention.ops.sliding_window import sliding_window_attention_varlen
from native_sparse_attention.testing import cu_from_lens, make_topk_idx

pytestmark = pytest.mark.gpu

LENS = [[0, 100, 0, 300, 0], [70, 0, 0, 129], [0, 0, 64]]
HQ, HKV, D, KS, ST, BS, TOPK = 8, 2, 64, 32, 16, 64, 4


def _tensors(lens, device):
    g = torch.Generator(device=device).manual_seed(0)
    cu = cu_from_lens(lens, device)
    T = int(cu[-1])
    q, do = (torch.randn(T, HQ, D, generator=g, device=device).bfloat16() for _ in range(2))
    k, v = (torch.randn(T, HKV, D, generator=g, device=device).bfloat16() for _ in range(2))
    return cu, q, k, v, do, g


def _grads_close(pairs):
    for name, got, want in pairs:
        assert_close(got, want, name, rel_to=max(1.0, want.abs().max().item()))


@pytest.mark.parametrize("lens", LENS)
def test_compression_operators(device, lens):
    print("case", lens, flush=True)
    cu, _, k, _, _, g = _tensors(lens, device)
    wp = torch.softmax(torch.randn(HKV, KS, generator=g, device=device), -1).bfloat16()
    wl = (torch.randn(HKV, KS * D, D, generator=g, device=device) / (KS * D) ** 0.5).bfloat16()
    for fn, ofn, w in ((weightedpool_compress, oracle.weightedpool_compress, wp), (linear_compress, oracle.linear_compress, wl)):
        x1, w1 = k.clone().requires_grad_(), w.clone().requires_grad_()
        xf, wf = k.float().requires_grad_(), w.float().requires_grad_()
        y, ycu = fn(x1, w1, cu, KS, ST)
        want, want_cu = ofn(xf, wf, cu, KS, ST)
        assert ycu.tolist() == want_cu.tolist() == cu_from_lens([max(0, (L - KS) // ST + 1) if L >= KS else 0 for L in lens], device).tolist()
        assert_close(y, want, "y")
        dy = torch.randn(y.shape, generator=g, device=device).bfloat16()
        y.backward(dy)
        want.backward(dy.float())
        _grads_close((("dx", x1.grad, xf.grad), ("dw", w1.grad, wf.grad)))


@pytest.mark.parametrize("lens", LENS)
def test_topk_sparse_attention(device, lens):
    print("case", lens, flush=True)
    cu, q, k, v, do, _ = _tensors(lens, device)
    idx = make_topk_idx(cu, BS, TOPK, HKV, seed=1, local_blocks=2)
    q1, k1, v1 = (x.clone().requires_grad_() for x in (q, k, v))
    qf, kf, vf = (x.float().requires_grad_() for x in (q, k, v))
    o = topk_sparse_attention(q1, k1, v1, idx, BS, cu)
    want = oracle.topk_sparse_attention(qf, kf, vf, idx, BS, cu)
    assert_close(o, want, "o")
    o.backward(do)
    want.backward(do.float())
    _grads_close((("dq", q1.grad, qf.grad), ("dk", k1.grad, kf.grad), ("dv", v1.grad, vf.grad)))


@pytest.mark.parametrize("lens", LENS)
def test_compressed_attention_and_selection(device, lens):
    print("case", lens, flush=True)
    cu, q, k, v, do, g = _tensors(lens, device)
    wp = torch.softmax(torch.randn(HKV, KS, generator=g, device=device), -1).bfloat16()
    ck, ccu = weightedpool_compress(k, wp, cu, KS, ST)
    cv, _ = weightedpool_compress(v, wp, cu, KS, ST)
    max_c = int((ccu[1:] - ccu[:-1]).max())
    q1, k1, v1 = (x.clone().requires_grad_() for x in (q, ck, cv))
    qf, kf, vf = (x.float().requires_grad_() for x in (q, ck, cv))
    o, idx = compressed_attention(q1, k1, v1, KS, ST, BS, TOPK, cu, ccu, max(lens), max_c, None, 1, 2)
    want, want_idx = oracle.compressed_attention(qf, kf, vf, KS, ST, BS, TOPK, cu, ccu, max(lens), max_c, None, 1, 2)
    assert_close(o, want, "o")
    assert torch.equal(idx, want_idx)
    o.backward(do)
    want.backward(do.float())
    _grads_close((("dq", q1.grad, qf.grad), ("dk", k1.grad, kf.grad), ("dv", v1.grad, vf.grad)))


@pytest.mark.parametrize("lens", LENS)
def test_window_and_dense_attention(device, lens):
    print("case", lens, flush=True)
    cu, q, k, v, do, _ = _tensors(lens, device)
    G = HQ // HKV

    def masked(qf, kf, vf, window):
        outs = []
        for b in range(len(lens)):
            s0, s1 = int(cu[b]), int(cu[b + 1])
            if s1 == s0:
                continue
            i = torch.arange(s1 - s0, device=device)
            mask = (i[None, :] <= i[:, None]) & (i[None, :] >= i[:, None] - window)
            s = torch.einsum("qhd,khd->hqk", qf[s0:s1], kf[s0:s1].repeat_interleave(G, 1)) / D ** 0.5
            p = torch.softmax(s.masked_fill(~mask, float("-inf")), -1)
            outs.append(torch.einsum("hqk,khd->qhd", p, vf[s0:s1].repeat_interleave(G, 1)))
        return torch.cat(outs)

    for window in (64, None):
        q1, k1, v1 = (x.clone().requires_grad_() for x in (q, k, v))
        qf, kf, vf = (x.float().requires_grad_() for x in (q, k, v))
        if window is None:
            o = flash_attention_varlen(q1, k1, v1, cu, cu, max(lens), max(lens), causal=True)
        else:
            o = sliding_window_attention_varlen(q1, k1, v1, cu, window)
        want = masked(qf, kf, vf, window if window is not None else 1 << 30)
        assert_close(o, want, "o")
        o.backward(do)
        want.backward(do.float())
        _grads_close((("dq", q1.grad, qf.grad), ("dk", k1.grad, kf.grad), ("dv", v1.grad, vf.grad)))


def test_many_short_sequences(device):
    """300 sequences (more than one per thread of the 256-thread prefix sums over the batch), some of them empty:
    block-sparse and compressed attention, forward and backward."""
    import random
    rng = random.Random(5)
    lens = [rng.choice([0, 1, 17, 33, 64, 65, 100, 130]) for _ in range(300)]
    print("case", len(lens), sum(lens), flush=True)
    cu, q, k, v, do, g = _tensors(lens, device)
    idx = make_topk_idx(cu, BS, TOPK, HKV, seed=2, local_blocks=2)
    q1, k1, v1 = (x.clone().requires_grad_() for x in (q, k, v))
    qf, kf, vf = (x.float().requires_grad_() for x in (q, k, v))
    o = topk_sparse_attention(q1, k1, v1, idx, BS, cu)
    want = oracle.topk_sparse_attention(qf, kf, vf, idx, BS, cu)
    assert_close(o, want, "o")
    o.backward(do)
    want.backward(do.float())
    _grads_close((("dq", q1.grad, qf.grad), ("dk", k1.grad, kf.grad), ("dv", v1.grad, vf.grad)))
    wp = torch.softmax(torch.randn(HKV, KS, generator=g, device=device), -1).bfloat16()
    ck, ccu = weightedpool_compress(k, wp, cu, KS, ST)
    cv, _ = weightedpool_compress(v, wp, cu, KS, ST)
    max_c = int((ccu[1:] - ccu[:-1]).max())
    q1, k1, v1 = (x.clone().requires_grad_() for x in (q, ck, cv))
    qf, kf, vf = (x.float().requires_grad_() for x in (q, ck, cv))
    o, sel = compressed_attention(q1, k1, v1, KS, ST, BS, TOPK, cu, ccu, max(lens), max_c, None, 1, 2)
    want, want_sel = oracle.compressed_attention(qf, kf, vf, KS, ST, BS, TOPK, cu, ccu, max(lens), max_c, None, 1, 2)
    assert_close(o, want, "o")
    assert torch.equal(sel, want_sel)
    o.backward(do)
    want.backward(do.float())
    _grads_close((("dq", q1.grad, qf.grad), ("dk", k1.grad, kf.grad), ("dv", v1.grad, vf.grad)))
