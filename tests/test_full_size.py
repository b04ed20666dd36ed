"""The headline configurations at full size (the top-k sweep's N=32768 and N=65536 points and the N=65536
compressed-attention benchmark) on the GPU, checked through properties that do not need a dense oracle: sampled-row
parity of the forward and of dQ (a row of either depends on that row's attention only), element-wise parity of dK / dV
on the last 1024 keys (which only the last 1024 queries see), and exact identities of the backward:
  * every row of P sums to 1, so  sum_j dV[j, hkv, :] = sum_t sum_{h in group} dO[t, h, :]  (over rows that see a key);
  * dS = P (dP - delta) pairs every (query, key) once on each side, so  sum <q, dq> = sum <k, dk>;
  * the backward is linear in dO."""
import pytest
import torch

import oracle
from helpers import assert_close, assert_ids_match
from native_sparse_attention.ops import compressed_attention, topk_sparse_attention, weightedpool_compress
from native_sparse_attention.testing import cu_from_lens, make_topk_idx

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("N,topk", [(32768, 16), (65536, 8), (65536, 16)])
def test_topk_sparse_attention_full_size(device, N, topk):
    Hq, Hkv, d, bs = 64, 4, 128, 64
    g = torch.Generator(device=device).manual_seed(0)
    cu = cu_from_lens([N], device)
    q, k, v = (torch.randn(N, h, d, generator=g, device=device).bfloat16().requires_grad_() for h in (Hq, Hkv, Hkv))
    do1, do2 = (torch.randn(N, Hq, d, generator=g, device=device).bfloat16() for _ in range(2))
    idx = make_topk_idx(cu, bs, topk, Hkv, seed=0, local_blocks=2)
    o = topk_sparse_attention(q, k, v, idx, bs, cu)
    rows = [0, 1, 63, 64, 65, 1000, 4095, 4096, 9999, 16384, 20000, 31000, N - 65, N - 2, N - 1]
    rows += torch.randint(0, N, (49,), generator=torch.Generator().manual_seed(1)).tolist()
    qf, kf, vf = (x.detach().float() for x in (q, k, v))
    qf.requires_grad_()
    want = oracle.topk_sparse_attention(qf, kf, vf, idx, bs, cu, rows=rows)
    assert_close(o[rows], want, "o rows")
    dq1, dk1, dv1 = torch.autograd.grad(o, (q, k, v), do1, retain_graph=True)
    want.backward(do1[rows].float())
    assert_close(dq1[rows], qf.grad[rows], "dq rows", rel_to=qf.grad[rows].abs().max().item())
    # element-wise dK / dV of the last 1024 keys: only the last 1024 queries see them, so the oracle restricted to
    # those rows yields their gradients completely (and o, dq of the same rows on the way)
    tail = list(range(N - 1024, N))
    qt, kt, vt = (x.detach().float().requires_grad_() for x in (q, k, v))
    want_t = oracle.topk_sparse_attention(qt, kt, vt, idx, bs, cu, rows=tail, row_chunk=256)
    want_t.backward(do1[tail].float())
    assert_close(o[tail], want_t, "o tail rows")
    assert_close(dq1[tail], qt.grad[tail], "dq tail rows", rel_to=qt.grad[tail].abs().max().item())
    assert_close(dk1[tail], kt.grad[tail], "dk of the last 1024 keys", rel_to=kt.grad[tail].abs().max().item())
    assert_close(dv1[tail], vt.grad[tail], "dv of the last 1024 keys", rel_to=vt.grad[tail].abs().max().item())
    del qt, kt, vt, want_t
    # column sums of dV against row sums of dO (fp32 sums of bf16 values: tolerance of the bf16 rounding of dV entries)
    G = Hq // Hkv
    want_sum = do1.float().view(N, Hkv, G, d).sum((0, 2))
    got_sum = dv1.float().sum(0)
    assert (got_sum - want_sum).abs().max() < 2e-2 * want_sum.abs().max()
    # sum <q, dq> == sum <k, dk>
    a = (q.detach().float() * dq1.float()).sum().item()
    b = (k.detach().float() * dk1.float()).sum().item()
    scale = (q.detach().float() * dq1.float()).abs().sum().item()
    assert abs(a - b) < 2e-3 * scale, (a, b, scale)
    # linearity in dO
    dq2, dk2, dv2 = torch.autograd.grad(o, (q, k, v), do2, retain_graph=True)
    dq12, dk12, dv12 = torch.autograd.grad(o, (q, k, v), (do1.float() + do2.float()).bfloat16())
    for name, x12, x1, x2 in (("dq", dq12, dq1, dq2), ("dk", dk12, dk1, dk2), ("dv", dv12, dv1, dv2)):
        ref = x1.float() + x2.float()
        assert_close(x12, ref, "linearity " + name, rel_to=ref.abs().max().item())


def test_compressed_attention_n65536(device):
    N, Hq, Hkv, d, ks, st, bs, topk = 65536, 32, 2, 128, 32, 16, 64, 16
    g = torch.Generator(device=device).manual_seed(0)
    cu = cu_from_lens([N], device)
    q = torch.randn(N, Hq, d, generator=g, device=device).bfloat16().requires_grad_()
    k, v = (torch.randn(N, Hkv, d, generator=g, device=device).bfloat16() for _ in range(2))
    w = torch.softmax(torch.randn(Hkv, ks, generator=g, device=device), -1).bfloat16()
    ck, cuk = weightedpool_compress(k, w, cu, ks, st)
    cv, _ = weightedpool_compress(v, w, cu, ks, st)
    ck = (ck * 4).detach().requires_grad_()
    cv = cv.detach().requires_grad_()
    o, idx = compressed_attention(q, ck, cv, ks, st, bs, topk, cu, cuk)
    assert idx.shape == (Hkv, N, topk)
    pos = torch.arange(N, device=device)
    qb = pos // bs
    valid = idx >= 0
    assert (valid.sum(-1) == torch.clamp(qb + 1, max=topk)[None]).all()           # min(topk, own block + 1) ids per row
    assert ((idx <= qb[None, :, None]) | ~valid).all() and (idx[..., 0] == 0).all()
    assert (idx == qb[None, :, None]).any(-1).all()                                  # the query's own block is always there
    srt = torch.where(valid, idx, torch.full_like(idx, 1 << 30))
    assert (srt[..., 1:] > srt[..., :-1]).logical_or(~valid[..., 1:]).all()
    assert (o[: ks - 1] == 0).all()                                                  # nothing visible before the first window ends
    # sampled rows against the oracle restricted to a short prefix and to the rows' own keys: row i only needs keys
    # c with c*st + ks - 1 <= i, so a prefix of the sequence reproduces its rows exactly
    P = 4096
    cuP = cu_from_lens([P], device)
    nP = (P - ks) // st + 1
    cukP = torch.tensor([0, nP], dtype=torch.int32, device=device)
    want, want_idx, bscore = oracle.compressed_attention(q[:P].detach().float(), ck[:nP].detach().float(), cv[:nP].detach().float(), ks, st,
                                                         bs, topk, cuP, cukP, return_scores=True)
    assert_close(o[:P], want, "o prefix")
    # the full-length selection equals the prefix selection on the prefix rows (same id width): bit-exact wherever
    # the oracle's decision margin is clear
    assert_ids_match(idx[:, :P].contiguous(), want_idx, bscore, qb[:P], "topk_idx of the prefix rows")
    do = torch.randn(N, Hq, d, generator=g, device=device).bfloat16()
    dq, dck, dcv = torch.autograd.grad(o, (q, ck, cv), do)
    G = Hq // Hkv
    want_sum = do[ks - 1:].float().view(N - ks + 1, Hkv, G, d).sum((0, 2))          # rows that see at least one key
    got_sum = dcv.float().sum(0)
    assert (got_sum - want_sum).abs().max() < 2e-2 * want_sum.abs().max()
    a = (q.detach().float() * dq.float()).sum().item()
    b = (ck.detach().float() * dck.float()).sum().item()
    scale = (q.detach().float() * dq.float()).abs().sum().item()
    assert abs(a - b) < 2e-3 * scale, (a, b, scale)
