"""Pins oracle.cmp_attn / oracle.decode (CPU): masked SDPA, overlap derivation, invariants, decode==prefill row."""
import math

import torch
import torch.nn.functional as F

import oracle
from oracle.cmp_attn import overlap_weights

KS, ST, BS = 32, 16, 64


def _inputs(lens=(100, 257, 512), Hq=4, Hkv=2, d=32, dtype=torch.float64, seed=0):
    torch.manual_seed(seed)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    T = int(cu[-1])
    q = torch.randn(T, Hq, d, dtype=dtype)
    kx = torch.randn(T, Hkv, d, dtype=dtype)
    vx = torch.randn(T, Hkv, d, dtype=dtype)
    ck, cuk = oracle.avgpool_compress(kx, None, cu, KS, ST)
    cv, _ = oracle.avgpool_compress(vx, None, cu, KS, ST)
    return q, ck, cv, cu, cuk


def test_output_is_masked_sdpa():
    q, ck, cv, cu, cuk = _inputs()
    out, idx = oracle.compressed_attention(q, ck, cv, KS, ST, BS, 4, cu, cuk)
    G = q.shape[1] // ck.shape[1]
    for b in range(3):
        qs = q[cu[b]:cu[b + 1]]
        ks, vs = ck[cuk[b]:cuk[b + 1]], cv[cuk[b]:cuk[b + 1]]
        Lq, Lk = qs.shape[0], ks.shape[0]
        mask = torch.arange(Lq)[:, None] >= (torch.arange(Lk)[None, :] * ST + KS - 1)
        want = F.scaled_dot_product_attention(
            qs.permute(1, 0, 2)[None], ks.repeat_interleave(G, 1).permute(1, 0, 2)[None],
            vs.repeat_interleave(G, 1).permute(1, 0, 2)[None], attn_mask=mask,
        )[0].permute(1, 0, 2).nan_to_num(0.0)
        assert torch.allclose(out[cu[b]:cu[b + 1]][KS - 1:], want[KS - 1:], atol=1e-10)
        assert out[cu[b]:cu[b + 1]][:KS - 1].abs().max() == 0          # nothing visible -> exact zeros


def test_overlap_weights_by_set_intersection():
    for ks, st, bs in [(32, 16, 64), (32, 8, 64), (64, 16, 128), (16, 16, 64), (32, 16, 32)]:
        w, pad = overlap_weights(ks, st, bs)
        r = bs // st
        for b in (0, 3):
            blk_chunks = set(range(b * r, b * r + r))                   # stride-sized chunks forming block b
            for c in range(-2, 40):
                tok_chunks = set(range(c, c + ks // st))                # chunks covered by compressed token c
                o = c - b * r + pad
                want = len(blk_chunks & tok_chunks)
                got = w[o] if 0 <= o < len(w) else 0
                assert got == want, (ks, st, bs, b, c)


def test_block_scores_brute_force_and_forced_blocks():
    torch.manual_seed(1)
    Hkv, R, max_k, max_q = 2, 6, 15, 257
    score = torch.rand(Hkv, R, max_k)
    q_pos = torch.tensor([0, 63, 64, 130, 200, 256])
    bsx = oracle.block_scores_from_probs(score, q_pos, KS, ST, BS, max_q, 1, 2)
    assert bsx.shape == (Hkv, R, 5)
    for r_i, p in enumerate(q_pos.tolist()):
        qb = p // BS
        for b in range(5):
            forced = b < 1 or (qb - 2 < b <= qb)
            if forced:
                assert torch.isinf(bsx[:, r_i, b]).all()
            elif b < max_q // BS:
                want = sum(
                    len(set(range(4 * b, 4 * b + 4)) & {c, c + 1}) * score[:, r_i, c] for c in range(max_k)
                )
                assert torch.allclose(bsx[:, r_i, b], want, atol=1e-6)
            else:
                assert (bsx[:, r_i, b] == 0).all()                     # ragged last block is never scored


def test_topk_idx_invariants():
    q, ck, cv, cu, cuk = _inputs(dtype=torch.float32)
    for topk in (4, 16):
        out, idx, bsc = oracle.compressed_attention(q, ck, cv, KS, ST, BS, topk, cu, cuk, return_scores=True)
        kk = min(topk, math.ceil(512 / BS))
        assert idx.shape == (2, int(cu[-1]), kk) and idx.dtype == torch.int32
        for b in range(3):
            for t in range(int(cu[b]), int(cu[b + 1]), 17):
                qb = (t - int(cu[b])) // BS
                for h in range(2):
                    row = idx[h, t].tolist()
                    valid = [e for e in row if e >= 0]
                    assert row == valid + [-1] * (kk - len(valid)) and valid == sorted(set(valid))
                    assert len(valid) == min(kk, qb + 1) and max(valid) <= qb
                    assert {0, qb, max(qb - 1, 0)} <= set(valid)
                    # the unforced picks are the best-scoring causal blocks
                    free = [e for e in valid if e not in (0, qb, qb - 1)]
                    rest = [e for e in range(qb + 1) if e not in valid]
                    if free and rest:
                        assert bsc[h, t, free].min() >= bsc[h, t, rest].max()


def test_decode_oracles_equal_last_prefill_row():
    torch.manual_seed(5)
    Hq, Hkv, d, topk = 4, 2, 32, 4
    lens = [130, 300, 64]
    B, maxlen = len(lens), 320
    kc = torch.randn(B, maxlen, Hkv, d, dtype=torch.float64)
    vc = torch.randn(B, maxlen, Hkv, d, dtype=torch.float64)
    qd = torch.randn(B, Hq, d, dtype=torch.float64)
    seqlens = torch.tensor(lens, dtype=torch.int32)
    # dense: equals sparse prefill with every block selected, last row
    o_dense = oracle.dense_attention_decode(qd, kc, vc, seqlens)
    from native_sparse_attention.testing import make_topk_idx
    for b, L in enumerate(lens):
        cu = torch.tensor([0, L], dtype=torch.int32)
        qfull = torch.randn(L, Hq, d, dtype=torch.float64)
        qfull[-1] = qd[b]
        nb = math.ceil(L / BS)
        all_idx = torch.arange(nb, dtype=torch.int32)[None, None].expand(Hkv, L, nb).contiguous()
        want = oracle.topk_sparse_attention(qfull, kc[b, :L], vc[b, :L], all_idx, BS, cu, rows=[L - 1])
        assert torch.allclose(o_dense[b], want[0], atol=1e-10)
        # top-k decode equals the sparse prefill row with the same ids
        idx = make_topk_idx(cu, BS, topk, Hkv, seed=b)
        got = oracle.topk_sparse_attention_decode(
            qd[b:b + 1], kc[b:b + 1], vc[b:b + 1], idx[:, L - 1:L], BS, seqlens[b:b + 1])
        want = oracle.topk_sparse_attention(qfull, kc[b, :L], vc[b, :L], idx, BS, cu, rows=[L - 1])
        assert torch.allclose(got[0], want[0], atol=1e-10)
        # compressed decode equals the compressed prefill row
        ck, cuk = oracle.avgpool_compress(kc[b, :L], None, cu, KS, ST)
        cv, _ = oracle.avgpool_compress(vc[b, :L], None, cu, KS, ST)
        o_p, idx_p = oracle.compressed_attention(qfull, ck, cv, KS, ST, BS, topk, cu, cuk)
        nck = ck.shape[0]
        slab_k = torch.zeros(1, nck + 3, Hkv, d, dtype=torch.float64)
        slab_v = torch.zeros_like(slab_k)
        slab_k[0, :nck], slab_v[0, :nck] = ck, cv
        o_d, idx_d = oracle.compressed_attention_decode(
            qd[b:b + 1], slab_k, slab_v, seqlens[b:b + 1], torch.tensor([nck], dtype=torch.int32), KS, ST, BS, topk)
        assert torch.allclose(o_d[0], o_p[L - 1], atol=1e-10)
        assert idx_d[:, 0].tolist() == idx_p[:, L - 1].tolist()


def test_compressed_decode_empty_slab():
    q = torch.randn(2, 4, 8)
    k = torch.zeros(2, 0, 2, 8)
    o, idx = oracle.compressed_attention_decode(q, k, k, torch.tensor([5, 9], dtype=torch.int32),
                                                torch.zeros(2, dtype=torch.int32), KS, ST, BS, 4)
    assert o.abs().max() == 0 and idx.shape == (2, 2, 1) and idx.dtype == torch.int32
