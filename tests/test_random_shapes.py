"""Seeded sweep over ragged shapes, head layouts, head sizes, block sizes and dtypes: forward and backward of the
block-sparse attention, the compressed attention with its block selection, and the sliding-window / dense causal
attention against the oracle (or a masked softmax where the oracle has no such function); the same for the decode
operators."""
import random

import pytest
import torch

import oracle
from helpers import assert_close, assert_ids_match
from native_sparse_attention.ops import compressed_attention, flash_attention_varlen, topk_sparse_attention, weightedpool_compress
from native_sparse_attention.ops.sliding_window import sliding_window_attention_varlen
from native_sparse_attention.testing import cu_from_lens, make_topk_idx

pytestmark = pytest.mark.gpu

LENS = [1, 2, 31, 32, 33, 63, 64, 65, 127, 128, 129, 200, 333, 700, 1025]


def _window_ref(q, k, v, cu, window):
    G = q.shape[1] // k.shape[1]
    outs = []
    for b in range(cu.shape[0] - 1):
        s0, s1 = int(cu[b]), int(cu[b + 1])
        i = torch.arange(s1 - s0, device=q.device)
        mask = (i[None, :] <= i[:, None]) & (i[None, :] >= i[:, None] - window)
        outs.append(torch.nn.functional.scaled_dot_product_attention(
            q[s0:s1].permute(1, 0, 2)[None], k[s0:s1].repeat_interleave(G, 1).permute(1, 0, 2)[None],
            v[s0:s1].repeat_interleave(G, 1).permute(1, 0, 2)[None], attn_mask=mask)[0].permute(1, 0, 2))
    return torch.cat(outs)


@pytest.mark.parametrize("seed", range(4))
def test_random_shapes(device, seed):
    rng = random.Random(1000 + seed)
    for case in range(12):
        kind = rng.choice(["topk", "topk", "cmp", "window"])
        dtype = rng.choice([torch.bfloat16, torch.float16])
        d, Hkv, G = rng.choice([32, 64, 96, 128]), rng.choice([1, 2, 3]), rng.choice([1, 2, 3, 4, 8, 16, 20, 32])
        Hq = Hkv * G
        lens = [rng.choice(LENS) for _ in range(rng.randint(1, 4))]
        cu = cu_from_lens(lens, device)
        T = int(cu[-1])
        g = torch.Generator(device=device).manual_seed(100 * seed + case)
        q, k, v, do = (torch.randn(T, h, d, generator=g, device=device).to(dtype) for h in (Hq, Hkv, Hkv, Hq))
        if kind == "topk":
            bs, topk = rng.choice([32, 64, 128, 256]), rng.randint(1, 9)
            print("case", seed, case, kind, lens, Hq, Hkv, d, bs, topk, dtype, flush=True)
            idx = make_topk_idx(cu, bs, topk, Hkv, seed=case, local_blocks=rng.choice([1, 2]))
            q1, k1, v1 = (x.clone().requires_grad_() for x in (q, k, v))
            o = topk_sparse_attention(q1, k1, v1, idx, bs, cu)
            qf, kf, vf = (x.float().requires_grad_() for x in (q, k, v))
            want = oracle.topk_sparse_attention(qf, kf, vf, idx, bs, cu)
        elif kind == "window":
            window, dense = rng.choice([16, 64, 100, 512]), rng.random() < 0.3
            print("case", seed, case, kind, lens, Hq, Hkv, d, window, dense, dtype, flush=True)
            q1, k1, v1 = (x.clone().requires_grad_() for x in (q, k, v))
            qf, kf, vf = (x.float().requires_grad_() for x in (q, k, v))
            if dense:
                o = flash_attention_varlen(q1, k1, v1, cu, cu, max(lens), max(lens), causal=True)
                want = _window_ref(qf, kf, vf, cu, 1 << 30)
            else:
                o = sliding_window_attention_varlen(q1, k1, v1, cu, window)
                want = _window_ref(qf, kf, vf, cu, window)
        else:
            ks, st = rng.choice([(32, 16), (32, 32), (16, 16), (64, 16), (64, 32)])
            bs, topk = rng.choice([b for b in (64, 128) if b % ks == 0]), rng.randint(3, 8)
            print("case", seed, case, kind, lens, Hq, Hkv, d, ks, st, bs, topk, dtype, flush=True)
            w = torch.softmax(torch.randn(Hkv, ks, generator=g, device=device), -1).to(dtype)
            ck, ccu = weightedpool_compress(k, w, cu, ks, st)
            cv, _ = weightedpool_compress(v, w, cu, ks, st)
            if ck.shape[0] == 0:
                continue
            max_c = int((ccu[1:] - ccu[:-1]).max())
            q1, k1, v1 = q.clone().requires_grad_(), ck.detach().clone().requires_grad_(), cv.detach().clone().requires_grad_()
            o, idx = compressed_attention(q1, k1, v1, ks, st, bs, topk, cu, ccu, max(lens), max_c, None, 1, 2)
            qf, kf, vf = q.float().requires_grad_(), ck.detach().float().requires_grad_(), cv.detach().float().requires_grad_()
            want, want_idx, bscore = oracle.compressed_attention(qf, kf, vf, ks, st, bs, topk, cu, ccu, max(lens), max_c, None, 1, 2,
                                                                 return_scores=True)
            qb = torch.cat([torch.arange(L, device=device) for L in lens]) // bs
            assert_ids_match(idx, want_idx, bscore, qb, "topk_idx", min_overlap=0.9)
        o.backward(do)
        want.backward(do.float())
        assert_close(o, want, "o")
        for name, a, b in (("dq", q1.grad, qf.grad), ("dk", k1.grad, kf.grad), ("dv", v1.grad, vf.grad)):
            assert_close(a, b, name, rel_to=max(1.0, b.abs().max().item()))


@pytest.mark.parametrize("seed", range(3))
def test_random_decode_shapes(device, seed):
    """The three decode operators against the oracle, and the fused selected + window branches + gated sum against
    the separate calls (bit for bit), on random batches, slab sizes, head layouts and block sizes."""
    from native_sparse_attention.ops import compressed_attention_decode, flash_attention_decode, topk_sparse_attention_decode
    from native_sparse_attention.ops.decode import decode_branches_gate
    from native_sparse_attention.ops.gated_sum import gate_combine

    rng = random.Random(2000 + seed)
    for case in range(10):
        dtype = rng.choice([torch.bfloat16, torch.float16])
        d, Hkv, G = rng.choice([32, 64, 96, 128]), rng.choice([1, 2, 3]), rng.choice([1, 2, 4, 8, 16, 20])
        Hq = Hkv * G
        B, bs, topk = rng.randint(1, 6), rng.choice([32, 64, 128]), rng.randint(1, 8)
        lens = [rng.choice([1, 2, 31, 33, 64, 65, 127, 129, 500, 1000, 2049]) for _ in range(B)]
        slab = max(lens) + rng.randint(0, 70)
        print("case", seed, case, lens, Hq, Hkv, d, bs, topk, dtype, flush=True)
        g = torch.Generator(device=device).manual_seed(100 * seed + case)
        q = torch.randn(B, Hq, d, generator=g, device=device).to(dtype)
        cache = torch.randn(2, B + 1, slab, Hkv, d, generator=g, device=device).to(dtype)   # slabs are views, as in a cache
        k, v = cache[0, :B], cache[1, :B]
        seqlens = torch.tensor(lens, dtype=torch.int32, device=device)
        o_dense = flash_attention_decode(q, k, v, seqlens)
        assert_close(o_dense, oracle.dense_attention_decode(q.float(), k.float(), v.float(), seqlens), "dense o")
        idx = torch.stack([make_topk_idx(cu_from_lens([L], device), bs, topk, Hkv, seed=7 * case + b)[:, L - 1]
                           for b, L in enumerate(lens)], 1).contiguous()
        o_sel = topk_sparse_attention_decode(q, k, v, idx, bs, seqlens)
        assert_close(o_sel, oracle.topk_sparse_attention_decode(q.float(), k.float(), v.float(), idx, bs, seqlens), "topk o")
        ks, st = rng.choice([(32, 16), (16, 16), (64, 16)])
        cbs = rng.choice([x for x in (64, 128) if x % ks == 0])
        clens = torch.tensor([0 if L < ks else (L - ks) // st + 1 for L in lens], dtype=torch.int32, device=device)
        cslab = max(int(clens.max()), 1) + rng.randint(0, 5)
        ck, cv = cache[0, :B, :cslab], cache[1, :B, :cslab]
        k_sel = rng.randint(1, 8)
        o_cmp, sel = compressed_attention_decode(q, ck, cv, seqlens, clens, ks, st, cbs, k_sel)
        want_cmp, want_sel, bscore = oracle.compressed_attention_decode(q.float(), ck.float(), cv.float(), seqlens, clens, ks, st, cbs,
                                                                        k_sel, return_scores=True)
        assert_close(o_cmp, want_cmp, "cmp o")
        assert_ids_match(sel, want_sel, bscore, (seqlens.long() - 1) // cbs, "decode ids", min_overlap=0.8)
        W = min(slab, rng.choice([16, 64, 512]))
        wk, wv = cache[0, 1:B + 1, :W], cache[1, 1:B + 1, :W]
        wlen = torch.tensor([min(L, W) for L in lens], dtype=torch.int32, device=device)
        gate = torch.sigmoid(torch.randn(B, Hq, 3, generator=g, device=device)).to(dtype)
        out, f_sel, f_win = decode_branches_gate(q, k, v, seqlens, idx, bs, wk, wv, wlen, o_cmp, gate)
        o_win = flash_attention_decode(q, wk, wv, wlen)
        assert torch.equal(f_sel, o_sel) and torch.equal(f_win, o_win)
        assert torch.equal(out, gate_combine(gate, o_cmp, o_sel, o_win))
