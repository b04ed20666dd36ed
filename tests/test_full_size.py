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


@pytest.mark.parametrize("N,topk", [(2048, 8), (4096, 16), (8192, 8), (8192, 16)])
def test_topk_sparse_attention_sweep_points_in_full(device, N, topk):
    """The short points of the benchmark sweep against the oracle on every row (forward and all three gradients); with the
    points below, every tier of the dK/dV work-item size (128, 192, 384, 768 queries) is exercised."""
    Hq, Hkv, d, bs = 64, 4, 128, 64
    g = torch.Generator(device=device).manual_seed(2)
    cu = cu_from_lens([N], device)
    q, k, v = (torch.randn(N, h, d, generator=g, device=device).bfloat16().requires_grad_() for h in (Hq, Hkv, Hkv))
    do = torch.randn(N, Hq, d, generator=g, device=device).bfloat16()
    idx = make_topk_idx(cu, bs, topk, Hkv, seed=3, local_blocks=2)
    o = topk_sparse_attention(q, k, v, idx, bs, cu)
    o.backward(do)
    qf, kf, vf = (x.detach().float().requires_grad_() for x in (q, k, v))
    want = oracle.topk_sparse_attention(qf, kf, vf, idx, bs, cu, row_chunk=256)
    want.backward(do.float())
    assert_close(o, want, "o")
    for name, a, b in (("dq", q.grad, qf.grad), ("dk", k.grad, kf.grad), ("dv", v.grad, vf.grad)):
        assert_close(a, b, name, rel_to=True)


@pytest.mark.parametrize("N,topk", [(16384, 8), (16384, 16), (32768, 8), (32768, 16), (65536, 8), (65536, 16), (131072, 8), (131072, 16)])
def test_topk_sparse_attention_full_size(device, N, topk):
    Hq, Hkv, d, bs = 64, 4, 128, 64
    g = torch.Generator(device=device).manual_seed(0)
    cu = cu_from_lens([N], device)
    q, k, v = (torch.randn(N, h, d, generator=g, device=device).bfloat16().requires_grad_() for h in (Hq, Hkv, Hkv))
    do1, do2 = (torch.randn(N, Hq, d, generator=g, device=device).bfloat16() for _ in range(2))
    idx = make_topk_idx(cu, bs, topk, Hkv, seed=0, local_blocks=2)
    o = topk_sparse_attention(q, k, v, idx, bs, cu)
    rows = [r for r in (0, 1, 63, 64, 65, 1000, 4095, 4096, 9999, 16384, 20000, 31000, 70000, 100000) if r < N] + [N - 65, N - 2, N - 1]
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
    k, v = (torch.randn(N, Hkv, d, generator=g, device=device).bfloat16().requires_grad_() for _ in range(2))
    wk, wv = (torch.softmax(torch.randn(Hkv, ks, generator=g, device=device), -1).bfloat16().requires_grad_() for _ in range(2))
    # the whole of the benchmark's chain with gradients flowing back through the pooling into k, v and the weights
    ck, cuk = weightedpool_compress(k, wk, cu, ks, st)
    cv, _ = weightedpool_compress(v, wv, cu, ks, st)
    ck4 = ck * 4                       # spreads the compressed keys so that attention is not nearly uniform (exact in bf16)
    for t in (ck, ck4, cv):
        t.retain_grad()
    o, idx = compressed_attention(q, ck4, cv, ks, st, bs, topk, cu, cuk)
    Tc = ck.shape[0]
    assert Tc == (N - ks) // st + 1 and idx.shape == (Hkv, N, topk)
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
    want, want_idx, bscore = oracle.compressed_attention(q[:P].detach().float(), ck4[:nP].detach().float(), cv[:nP].detach().float(), ks, st,
                                                         bs, topk, cuP, cukP, return_scores=True)
    assert_close(o[:P], want, "o prefix")
    # the full-length selection equals the prefix selection on the prefix rows (same id width): bit-exact wherever
    # the oracle's decision margin is clear
    assert_ids_match(idx[:, :P].contiguous(), want_idx, bscore, qb[:P], "topk_idx of the prefix rows")
    do = torch.randn(N, Hq, d, generator=g, device=device).bfloat16()
    o.backward(do)
    dq, dck, dcv = q.grad, ck4.grad, cv.grad
    G = Hq // Hkv
    want_sum = do[ks - 1:].float().view(N - ks + 1, Hkv, G, d).sum((0, 2))          # rows that see at least one key
    got_sum = dcv.float().sum(0)
    assert (got_sum - want_sum).abs().max() < 2e-2 * want_sum.abs().max()
    a = (q.detach().float() * dq.float()).sum().item()
    b = (ck4.detach().float() * dck.float()).sum().item()
    scale = (q.detach().float() * dq.float()).abs().sum().item()
    assert abs(a - b) < 2e-3 * scale, (a, b, scale)

    # Element-wise: the last 64 compressed keys are seen by the last queries only (key c by queries i >= c*st + ks - 1),
    # so attention of those queries over ALL compressed keys, stated directly as a masked softmax in fp32 (the rule of
    # oracle/cmp_attn.py: visibility i >= c*st + ks - 1, probabilities rounded to the value type), yields o and dq of
    # those rows and dK / dV of those keys completely.  The last 64 keys are pooled from the last 64*st + ks - st tokens
    # alone, so pooling that tail as a sequence of its own carries the gradient on into k, v of those tokens.
    C = 64
    c0 = Tc - C
    i0 = c0 * st + ks - 1                      # first query that sees key c0
    t0 = c0 * st                               # first token under key c0
    kt, vt = (x.detach()[t0:].float().requires_grad_() for x in (k, v))
    wkf, wvf = wk.detach().float(), wv.detach().float()
    cu_t = cu_from_lens([N - t0], device)
    ck_t, _ = oracle.weightedpool_compress(kt, wkf, cu_t, ks, st)
    cv_t, _ = oracle.weightedpool_compress(vt, wvf, cu_t, ks, st)
    assert ck_t.shape[0] == C
    ck_t.retain_grad(); cv_t.retain_grad()
    ck_all = torch.cat([ck4.detach()[:c0].float(), 4 * (ck_t.detach().to(torch.bfloat16).float() + (ck_t - ck_t.detach()))], 0)   # bf16 values, fp32 gradient path
    cv_all = torch.cat([cv.detach()[:c0].float(), cv_t.detach().to(torch.bfloat16).float() + (cv_t - cv_t.detach())], 0)
    qt = q.detach()[i0:].float().requires_grad_()
    vis = pos[i0:, None] >= (torch.arange(Tc, device=device) * st + ks - 1)[None, :]
    s_ = torch.einsum("rhgd,lhd->hgrl", qt.view(N - i0, Hkv, G, d), ck_all) / d ** 0.5
    p_ = torch.softmax(s_.masked_fill(~vis[None, None], float("-inf")), -1)
    want_t = torch.einsum("hgrl,lhd->rhgd", p_.to(torch.bfloat16).float(), cv_all).reshape(N - i0, Hq, d)
    want_t.backward(do[i0:].float())
    assert_close(o[i0:], want_t, "o of the last queries")
    assert_close(dq[i0:], qt.grad, "dq of the last queries", rel_to=True)
    # gradients of compressed keys >= c0 come from queries >= i0 only; ck_t's gradient is the oracle's dK for them
    assert_close(ck.grad[c0:], ck_t.grad, "dK of the last 64 compressed keys", rel_to=True)
    assert_close(cv.grad[c0:], cv_t.grad, "dV of the last 64 compressed keys", rel_to=True)
    assert_close(k.grad[t0 + ks - st:], kt.grad[ks - st:], "dk of the last tokens (through the pooling)", rel_to=True)
    assert_close(v.grad[t0 + ks - st:], vt.grad[ks - st:], "dv of the last tokens (through the pooling)", rel_to=True)
    # the weights' gradients sum over every window: dw[h, j] = sum_n sum_d dck[n, h, d] * k[n*st + j, h, d] (oracle/compress.py)
    for name, wg, dc, x in (("dwk", wk.grad, ck.grad, k), ("dwv", wv.grad, dcv, v)):
        win = x.detach().float().unfold(0, ks, st)[:Tc]                                # [Tc, Hkv, d, ks]
        want_w = torch.einsum("nhd,nhdj->hj", dc.float(), win)
        assert_close(wg, want_w, name, rel_to=True)
