"""Writes the known-answer fixtures in this folder (run once; the .npz files are committed).

    python tests/golden/make_golden.py

The reference stores no golden vectors of its own, so these come from scalar-loop statements of the
definitions, written here with Python floats and `math.exp` only: no tensor library, nothing imported
from the oracle or the product.  Each routine cites the reference lines whose rule it spells out.
Inputs are rounded to bf16-representable values so that the CPU oracle (fp32/fp64) and the bf16 GPU
kernels read exactly the same numbers; shapes use head_dim 32 and block sizes the kernels accept.
"""
import math
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def bf16_round(a):
    """Round float32 values to the nearest bf16 (ties to even), returned as float32."""
    u = np.asarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def randn(rs, *shape, scale=1.0):
    return bf16_round(rs.standard_normal(shape).astype(np.float32) * scale)


def softmax_rows(scores):
    """scores: list of floats (may be empty) -> probabilities and natural-log LSE."""
    if not scores:
        return [], -math.inf
    m = max(scores)
    e = [math.exp(s - m) for s in scores]
    z = sum(e)
    return [x / z for x in e], m + math.log(z)


def dot(a, b):
    return sum(float(x) * float(y) for x, y in zip(a, b))


# ----------------------------------------------------------------------------------------------
def topk_sparse_attention(q, k, v, idx, bs, cu, scale):
    """ops/torch/topk_sparse_attention.py:58-83: key j of the same sequence is visible to position i
    iff j <= i and block j // bs is listed in topk_idx[h_kv, token] (-1 counts as block 0, :66)."""
    T, Hq, d = q.shape
    G = Hq // k.shape[1]
    o = np.zeros((T, Hq, d))
    lse = np.full((Hq, T), -math.inf)
    for b in range(len(cu) - 1):
        for t in range(cu[b], cu[b + 1]):
            i = t - cu[b]
            for h in range(Hq):
                hk = h // G
                blocks = {max(int(e), 0) for e in idx[hk, t]}
                keys = [j for j in range(i + 1) if j // bs in blocks]
                p, l = softmax_rows([dot(q[t, h], k[cu[b] + j, hk]) * scale for j in keys])
                lse[h, t] = l
                for pj, j in zip(p, keys):
                    o[t, h] += pj * v[cu[b] + j, hk].astype(np.float64)
    return o, lse


def compressed_lens(lens, ks, st):
    """ops/triton/utils.py:25-37."""
    return [0 if L < ks else (L - ks) // st + 1 for L in lens]


def pool(x, w, lens, ks, st):
    """ops/torch/compress_key_value.py:95-160: y[n, h] = sum_k w[h, k] x[n*st + k, h] inside each sequence
    (w = 1/ks everywhere for the average pool, :30-92)."""
    H, d = x.shape[1], x.shape[2]
    out, s0 = [], 0
    for L, n in zip(lens, compressed_lens(lens, ks, st)):
        for c in range(n):
            row = np.zeros((H, d))
            for h in range(H):
                for kk in range(ks):
                    row[h] += float(w[h, kk]) * x[s0 + c * st + kk, h].astype(np.float64)
            out.append(row)
        s0 += L
    return np.array(out).reshape(-1, H, d)


def linear(x, w, lens, ks, st):
    """ops/torch/compress_key_value.py:163-231: y[n, h, :] = concat_k(x[n*st + k, h, :]) @ w[h]."""
    H, d = x.shape[1], x.shape[2]
    dout = w.shape[2]
    out, s0 = [], 0
    w64 = w.astype(np.float64)
    for L, n in zip(lens, compressed_lens(lens, ks, st)):
        for c in range(n):
            row = np.zeros((H, dout))
            for h in range(H):
                for kk in range(ks):
                    row[h] += x[s0 + c * st + kk, h].astype(np.float64) @ w64[h, kk * d:(kk + 1) * d]
            out.append(row)
        s0 += L
    return np.array(out).reshape(-1, H, dout)


def compressed_attention(q, ck, cv, lens, ks, st, bs, topk, init_blocks, local_blocks, scale):
    """ops/torch/compressed_attention.py:74-194.  Compressed key c is visible to position i iff
    i >= c*st + ks - 1 (:127-133); rows that see nothing give 0 (:141-142).  Block score (:21-71): the
    probabilities summed over the query heads of a kv head, then
    block[b] = sum over the ks/st x bs/st pairs (i, j) of score[b*(bs/st) + i + j - (ks/st - 1)],
    only for blocks that lie wholly inside the longest sequence; forced blocks get +inf; the k best
    (ties: lower index) are listed ascending, entries beyond the query's own block become -1."""
    T, Hq, d = q.shape
    Hkv = ck.shape[1]
    G = Hq // Hkv
    clens = compressed_lens(lens, ks, st)
    a, r = ks // st, bs // st
    max_len = max(lens)
    nb, full = -(-max_len // bs), max_len // bs
    kk = min(topk, nb)
    out = np.zeros((T, Hq, d))
    bscore = np.zeros((Hkv, T, nb))
    idx = np.full((Hkv, T, kk), -1, dtype=np.int32)
    s0 = c0 = 0
    for L, C in zip(lens, clens):
        for i in range(L):
            t = s0 + i
            vis = [c for c in range(C) if i >= c * st + ks - 1]
            for hk in range(Hkv):
                score = [0.0] * C
                for g in range(G):
                    h = hk * G + g
                    p, _ = softmax_rows([dot(q[t, h], ck[c0 + c, hk]) * scale for c in vis])
                    for pc, c in zip(p, vis):
                        out[t, h] += pc * cv[c0 + c, hk].astype(np.float64)
                        score[c] += pc
                for b in range(full):
                    tot = 0.0
                    for ii in range(a):
                        for jj in range(r):
                            c = b * r + ii + jj - (a - 1)
                            if 0 <= c < C:
                                tot += score[c]
                    bscore[hk, t, b] = tot
                qb = i // bs
                for b in range(nb):
                    if b < init_blocks or (qb - local_blocks < b <= qb):
                        bscore[hk, t, b] = math.inf
                order = sorted(range(nb), key=lambda b: (-bscore[hk, t, b], b))[:kk]
                chosen = sorted(order)
                idx[hk, t] = [b if b <= qb else -1 for b in chosen]  # ascending, so the -1 entries end up on the right
        s0 += L
        c0 += C
    return out, bscore, idx


def decode_dense(q, k, v, seqlens, scale):
    """ops/triton/flash_attention_decode.py:220-258: one query per sequence over the first seqlens[b] rows."""
    B, Hq, d = q.shape
    G = Hq // k.shape[2]
    o = np.zeros((B, Hq, d))
    for b in range(B):
        for h in range(Hq):
            hk = h // G
            p, _ = softmax_rows([dot(q[b, h], k[b, j, hk]) * scale for j in range(seqlens[b])])
            for j, pj in enumerate(p):
                o[b, h] += pj * v[b, j, hk].astype(np.float64)
    return o


def decode_topk(q, k, v, idx, bs, seqlens, scale):
    """ops/triton/topk_sparse_attention_decode.py:240-298: the query sits at position seqlens[b] - 1 and
    sees the listed blocks (entries < 0 skipped), clipped to the sequence length."""
    B, Hq, d = q.shape
    G = Hq // k.shape[2]
    o = np.zeros((B, Hq, d))
    for b in range(B):
        for h in range(Hq):
            hk = h // G
            blocks = {int(e) for e in idx[hk, b] if e >= 0}
            keys = [j for j in range(seqlens[b]) if j // bs in blocks]
            p, _ = softmax_rows([dot(q[b, h], k[b, j, hk]) * scale for j in keys])
            for pj, j in zip(p, keys):
                o[b, h] += pj * v[b, j, hk].astype(np.float64)
    return o


# ----------------------------------------------------------------------------------------------
def main():
    rs = np.random.RandomState(20250101)

    # topk sparse attention
    lens, Hq, Hkv, d, bs, topk = [70, 33], 4, 2, 32, 32, 2
    cu = [0, 70, 103]
    T = cu[-1]
    q, k, v = randn(rs, T, Hq, d), randn(rs, T, Hkv, d), randn(rs, T, Hkv, d)
    idx = np.full((Hkv, T, topk), -1, dtype=np.int32)
    for b in range(2):
        for t in range(cu[b], cu[b + 1]):
            qb = (t - cu[b]) // bs
            for h in range(Hkv):
                other = 0 if qb < 2 else int(rs.randint(0, qb))  # an earlier block (block 0 for short prefixes)
                row = sorted({other, qb})
                idx[h, t, :len(row)] = row
    o, lse = topk_sparse_attention(q, k, v, idx, bs, cu, 1 / math.sqrt(d))
    np.savez(os.path.join(HERE, "topk_sparse_attention.npz"), q=q, k=k, v=v, topk_idx=idx, cu_seqlens=np.array(cu, dtype=np.int32),
             block_size=bs, o=o, lse=lse)

    # compression
    H, ks, st = 2, 32, 16
    x = randn(rs, T, H, d)
    w_pool = bf16_round(rs.dirichlet(np.ones(ks), size=H).astype(np.float32))
    w_lin = randn(rs, H, ks * d, d, scale=1 / math.sqrt(ks * d))
    np.savez(os.path.join(HERE, "compress.npz"), x=x, w_pool=w_pool, w_lin=w_lin, cu_seqlens=np.array(cu, dtype=np.int32), kernel_size=ks,
             kernel_stride=st, y_cu_seqlens=np.cumsum([0] + compressed_lens(lens, ks, st)).astype(np.int32),
             y_avg=pool(x, np.full((H, ks), 1.0 / ks), lens, ks, st), y_pool=pool(x, w_pool, lens, ks, st), y_lin=linear(x, w_lin, lens, ks, st))

    # compressed attention and block selection
    lens2, bs2, topk2 = [200, 90], 64, 3
    cu2 = [0, 200, 290]
    T2 = cu2[-1]
    clens = compressed_lens(lens2, ks, st)
    q2 = randn(rs, T2, Hq, d)
    ck, cv = randn(rs, sum(clens), Hkv, d, scale=2.0), randn(rs, sum(clens), Hkv, d)
    out, bscore, idx2 = compressed_attention(q2, ck, cv, lens2, ks, st, bs2, topk2, 1, 2, 1 / math.sqrt(d))
    np.savez(os.path.join(HERE, "compressed_attention.npz"), q=q2, k=ck, v=cv, cu_seqlens_q=np.array(cu2, dtype=np.int32),
             cu_seqlens_k=np.cumsum([0] + clens).astype(np.int32), kernel_size=ks, kernel_stride=st, block_size=bs2, topk=topk2,
             out=out, block_score=bscore, topk_idx=idx2)

    # decode
    B, slab = 2, 72
    seqlens = [72, 37]
    qd = randn(rs, B, Hq, d)
    kd, vd = randn(rs, B, slab, Hkv, d), randn(rs, B, slab, Hkv, d)
    idxd = np.array([[[0, 2], [0, 1]], [[1, 2], [1, -1]]], dtype=np.int32)  # [Hkv, B, topk]
    np.savez(os.path.join(HERE, "decode.npz"), q=qd, k=kd, v=vd, seqlens=np.array(seqlens, dtype=np.int32), topk_idx=idxd, block_size=32,
             o_dense=decode_dense(qd, kd, vd, seqlens, 1 / math.sqrt(d)), o_topk=decode_topk(qd, kd, vd, idxd, 32, seqlens, 1 / math.sqrt(d)))
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
