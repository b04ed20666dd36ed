"""Decode path over the cache slabs: every decode step must reproduce the last row of the prefill
operators run on the concatenated sequence, branch by branch (and the cache must follow the
shift / append / ring rules that make that true)."""
import pytest
import torch

import oracle
from helpers import assert_close, assert_ids_match
from native_sparse_attention.infer import nsa_infer
from native_sparse_attention.module import NSACache
from native_sparse_attention.ops import weightedpool_compress
from native_sparse_attention.ops.sliding_window import sliding_window_attention_varlen
from native_sparse_attention.testing import cu_from_lens

pytestmark = pytest.mark.gpu


def _rope(x, cu_seqlens, step, stride=1):
    return x  # positional encoding is outside the operator path


def test_sliding_window_prefill_matches_masked_softmax(device):
    g = torch.Generator(device=device).manual_seed(0)
    lens, Hq, Hkv, d, W = [700, 90, 1300], 16, 2, 128, 256
    cu = cu_from_lens(lens, device)
    T = int(cu[-1])
    q = torch.randn(T, Hq, d, generator=g, device=device).bfloat16()
    k = torch.randn(T, Hkv, d, generator=g, device=device).bfloat16()
    v = torch.randn(T, Hkv, d, generator=g, device=device).bfloat16()
    o = sliding_window_attention_varlen(q, k, v, cu, W)
    G = Hq // Hkv
    for b in range(len(lens)):
        s0, s1 = int(cu[b]), int(cu[b + 1])
        L = s1 - s0
        i = torch.arange(L, device=device)
        mask = (i[None, :] <= i[:, None]) & (i[None, :] >= i[:, None] - W)
        want = torch.nn.functional.scaled_dot_product_attention(
            q[s0:s1].float().permute(1, 0, 2)[None], k[s0:s1].float().repeat_interleave(G, 1).permute(1, 0, 2)[None],
            v[s0:s1].float().repeat_interleave(G, 1).permute(1, 0, 2)[None], attn_mask=mask)[0].permute(1, 0, 2)
        assert_close(o[s0:s1], want, "window o seq %d" % b)


# the last case is the decode benchmark as one composed step: batch 4, cached lengths 2048 / 4096 / 6144 / 8192, window 512
@pytest.mark.parametrize("prompt_lens,steps,W", [([130, 47, 300], 40, 128), ([2048, 515], 3, 128), ([2048, 4096, 6144, 8192], 2, 512)])
def test_decode_steps_equal_prefill_last_row(device, prompt_lens, steps, W):
    Hq, Hkv, d = 32, 2, 128
    ks, st, bs, topk = 32, 16, 64, 8
    B = len(prompt_lens)
    g = torch.Generator(device=device).manual_seed(1)
    total = [L + steps for L in prompt_lens]
    full_cu = cu_from_lens(total, device)
    Tfull = int(full_cu[-1])
    q_all = torch.randn(Tfull, Hq, d, generator=g, device=device).bfloat16()
    k_all = torch.randn(Tfull, Hkv, d, generator=g, device=device).bfloat16()
    v_all = torch.randn(Tfull, Hkv, d, generator=g, device=device).bfloat16()
    gate_all = torch.sigmoid(torch.randn(Tfull, Hq, 3, generator=g, device=device)).bfloat16()
    wk = torch.softmax(torch.randn(Hkv, ks, generator=g, device=device), -1).bfloat16()
    wv = torch.softmax(torch.randn(Hkv, ks, generator=g, device=device), -1).bfloat16()
    cache = NSACache(B + 1, max(total) + 8, Hkv, d, ks, st, W, torch.bfloat16, device)
    args = (_rope, cache, (wk, wv), (weightedpool_compress, weightedpool_compress), None, ks, st, bs, topk, 1, 2, W)

    def rows(step):  # global rows of every sequence's token number prompt_len + step - 1
        return torch.tensor([int(full_cu[b]) + prompt_lens[b] + step - 1 for b in range(B)], device=device)

    prompt_cu = cu_from_lens(prompt_lens, device)
    sel = torch.cat([torch.arange(int(full_cu[b]), int(full_cu[b]) + prompt_lens[b], device=device) for b in range(B)])
    out0 = nsa_infer(prompt_cu, 0, q_all[sel], k_all[sel], v_all[sel], gate_all[sel], *args)
    assert out0.shape == (sum(prompt_lens), Hq, d)
    for step in range(1, steps + 1):
        r = rows(step)
        out, (cmp_o, sp_o, win_o, idx) = nsa_infer(prompt_cu, step, q_all[r], k_all[r], v_all[r], gate_all[r], *args,
                                                   return_branches=True)
        # reference: the prefill operators (oracle) on the sequences cut after this token
        for b in range(B):
            L = prompt_lens[b] + step
            s0 = int(full_cu[b])
            cu1 = cu_from_lens([L], device)
            qs, kk, vv = (x[s0:s0 + L].float() for x in (q_all, k_all, v_all))
            ck, cuk = oracle.weightedpool_compress(kk, wk.float(), cu1, ks, st)
            cv, _ = oracle.weightedpool_compress(vv, wv.float(), cu1, ks, st)
            # the kernels see compressed tokens rounded to bf16 in the cache
            ck, cv = ck.bfloat16().float(), cv.bfloat16().float()
            if ck.shape[0] > 0:
                want_cmp, want_idx, bscore = oracle.compressed_attention(qs, ck, cv, ks, st, bs, topk, cu1, cuk, return_scores=True)
                assert_close(cmp_o[b], want_cmp[L - 1], "compressed branch b=%d step=%d" % (b, step))
                use_idx = idx[:, b:b + 1]
                # ids: the sequence on its own may have fewer blocks than the batch's id width (then every causal block
                # is selected and the extra slots hold -1); bit-exact wherever the oracle's margin is clear
                kk_ref = want_idx.shape[-1]
                assert (use_idx[:, 0, kk_ref:] == -1).all()
                last = torch.tensor([(L - 1) // bs], device=device)
                assert_ids_match(use_idx[:, :, :kk_ref].contiguous(), want_idx[:, L - 1:L].contiguous(), bscore[:, L - 1:L], last,
                                 "decode ids b=%d step=%d" % (b, step), min_overlap=0.8)
            else:
                assert cmp_o[b].abs().max() == 0
                use_idx = idx[:, b:b + 1]
            # the sparse branch is checked with the ids the decode path actually selected
            row_idx = use_idx[:, 0, :].clone()
            full_idx = torch.full((Hkv, L, row_idx.shape[-1]), -1, dtype=torch.int32, device=device)
            full_idx[:, :, 0] = 0
            full_idx[:, L - 1] = row_idx
            want_sp = oracle.topk_sparse_attention(qs, kk, vv, full_idx, bs, cu1, rows=[L - 1])
            assert_close(sp_o[b], want_sp[0], "sparse branch b=%d step=%d" % (b, step))
            # window branch: the ring holds the last W tokens (decode uses W keys, see module docstring)
            lo = max(0, L - W)
            att = torch.softmax(torch.einsum("hgd,lhd->hgl", qs[L - 1].view(Hkv, Hq // Hkv, d), kk[lo:L]) / d ** 0.5, -1)
            want_win = torch.einsum("hgl,lhd->hgd", att, vv[lo:L]).reshape(Hq, d)
            assert_close(win_o[b], want_win, "window branch b=%d step=%d" % (b, step))
            gv = gate_all[r[b]].float()
            want = gv[:, 0, None] * cmp_o[b].float() + gv[:, 1, None] * sp_o[b].float() + gv[:, 2, None] * win_o[b].float()
            assert_close(out[b], want, "gated sum b=%d step=%d" % (b, step))
        # cache bookkeeping
        for b in range(B):
            L = prompt_lens[b] + step
            assert int(cache.sparse_kv_len[b]) == L and int(cache.sliding_kv_len[b]) == min(prompt_lens[b], W) + step
            assert int(cache.compress_kv_len[b]) == (0 if L < ks else (L - ks) // st + 1)


@pytest.mark.parametrize("n,H,d,dtype", [(1000, 32, 128, torch.bfloat16), (3, 6, 64, torch.float16), (257, 16, 96, torch.bfloat16)])
def test_gate_combine_is_bit_identical_to_the_tensor_expression(device, n, H, d, dtype):
    from native_sparse_attention.infer.nsa_inference import gate_combine
    g = torch.Generator(device=device).manual_seed(2)
    gate = torch.sigmoid(torch.randn(n, H * 3, generator=g, device=device)).to(dtype).view(n, H, 3)
    a, b = (torch.randn(n, H, d, generator=g, device=device).to(dtype) for _ in range(2))
    c = torch.randn(n, H, 2 * d, generator=g, device=device).to(dtype)[..., :d]   # strided rows
    want = gate[..., 0, None] * a + gate[..., 1, None] * b + gate[..., 2, None] * c
    assert torch.equal(gate_combine(gate, a, b, c), want)


def test_graphed_decode_step_equals_eager_steps(device):
    """The decode step recorded in a HIP graph, replayed for many tokens with eager work in between, against the eager
    decode steps on an identically prefilled second cache."""
    from native_sparse_attention.infer import NSADecodeGraph
    from native_sparse_attention.module import RopeConfig, RotaryEmbedding
    Hq, Hkv, d, ks, st, bs, topk, W = 32, 2, 128, 32, 16, 64, 8, 128
    lens, steps = [300, 47, 1100], 40
    B = len(lens)
    g = torch.Generator(device=device).manual_seed(5)
    cu = cu_from_lens(lens, device)
    T = int(cu[-1])
    rope = RotaryEmbedding(RopeConfig(head_dim=d), device=device)
    wk = torch.softmax(torch.randn(Hkv, ks, generator=g, device=device), -1).bfloat16()
    wv = torch.softmax(torch.randn(Hkv, ks, generator=g, device=device), -1).bfloat16()
    pe = (torch.randn(Hkv, ks, d, generator=g, device=device) * 0.02).bfloat16()

    def rnd(*shape):
        return torch.randn(*shape, generator=g, device=device).bfloat16()

    q0, k0, v0, g0 = rnd(T, Hq, d), rnd(T, Hkv, d), rnd(T, Hkv, d), torch.sigmoid(rnd(T, Hq, 3).float()).bfloat16()
    caches = [NSACache(B, max(lens) + steps + 8, Hkv, d, ks, st, W, torch.bfloat16, device) for _ in range(2)]
    tail = ((wk, wv), (weightedpool_compress, weightedpool_compress), pe, ks, st, bs, topk, 1, 2, W)
    outs = [nsa_infer(cu, 0, q0, k0, v0, g0, rope, c, *tail) for c in caches]
    assert torch.equal(outs[0], outs[1])
    graph = NSADecodeGraph(cu, Hq, rope, caches[0], *tail)
    for step in range(1, steps + 1):
        q, k, v, gt = rnd(B, Hq, d), rnd(B, Hkv, d), rnd(B, Hkv, d), torch.sigmoid(rnd(B, Hq, 3).float()).bfloat16()
        want = nsa_infer(cu, step, q, k, v, gt, rope, caches[1], *tail)
        got = graph.step(q, k, v, gt)
        assert_close(got, want.float(), "graph replay %d" % step)
        for name in ("sparse_kv_len", "compress_kv_len", "before_compress_kv_len", "sliding_kv_len"):
            assert torch.equal(getattr(caches[0], name), getattr(caches[1], name)), (name, step)
    n = int(caches[1].sparse_kv_len[2])
    assert torch.equal(caches[0].sparse_kv_cache[:, 2, :n], caches[1].sparse_kv_cache[:, 2, :n])


@pytest.mark.parametrize("weighted,with_pe,dtype", [(True, True, torch.bfloat16), (True, False, torch.float16), (False, True, torch.bfloat16)])
def test_single_launch_prepare_equals_separate_operators(device, weighted, with_pe, dtype):
    """The decode step whose cache work is one kernel (pooling compression + this package's rotary module) against the
    same step built from the separate operators (forced by handing the compression in as plain callables), on two
    identically prefilled caches: outputs, lengths and every valid cache row must be identical, window completions,
    staging shifts and ring wrap-around included."""
    from native_sparse_attention.module import RopeConfig, RotaryEmbedding
    from native_sparse_attention.ops import avgpool_compress
    Hq, Hkv, d, ks, st, bs, topk, W = 16, 2, 128, 32, 16, 64, 4, 64
    lens, steps = [300, 47, 20, 1100], 70
    B = len(lens)
    g = torch.Generator(device=device).manual_seed(11)
    cu = cu_from_lens(lens, device)
    T = int(cu[-1])
    rope = RotaryEmbedding(RopeConfig(head_dim=d), device=device)

    def rnd(*shape):
        return torch.randn(*shape, generator=g, device=device).to(dtype)

    if weighted:
        weights = (torch.softmax(torch.randn(Hkv, ks, generator=g, device=device), -1).to(dtype),
                   torch.softmax(torch.randn(Hkv, ks, generator=g, device=device), -1).to(dtype))
        fn = weightedpool_compress
    else:
        weights, fn = (None, None), avgpool_compress
    pe = (rnd(Hkv, ks, d).float() * 0.02).to(dtype) if with_pe else None
    plain = lambda *a, **kw: fn(*a, **kw)   # not recognised as a pooling operator: the separate-operator path runs
    q0, k0, v0, g0 = rnd(T, Hq, d), rnd(T, Hkv, d), rnd(T, Hkv, d), torch.sigmoid(rnd(T, Hq, 3).float()).to(dtype)
    caches = [NSACache(B, max(lens) + steps + 8, Hkv, d, ks, st, W, dtype, device) for _ in range(2)]
    tails = [(weights, (fn, fn), pe, ks, st, bs, topk, 1, 2, W), (weights, (plain, plain), pe, ks, st, bs, topk, 1, 2, W)]
    for c, tail in zip(caches, tails):
        nsa_infer(cu, 0, q0, k0, v0, g0, rope, c, *tail)
    for step in range(1, steps + 1):
        kv = rnd(B, Hkv + 1, 2 * d)
        q, k, v, gt = rnd(B, Hq, d), kv[:, :Hkv, :d], kv[:, 1:, d:], torch.sigmoid(rnd(B, Hq, 3).float()).to(dtype)   # strided k, v
        got = nsa_infer(cu, step, q, k, v, gt, rope, caches[0], *tails[0])
        want = nsa_infer(cu, step, q, k, v, gt, rope, caches[1], *tails[1])
        assert torch.equal(got, want), step
        for name in ("sparse_kv_len", "compress_kv_len", "before_compress_kv_len", "sliding_kv_len"):
            assert torch.equal(getattr(caches[0], name), getattr(caches[1], name)), (name, step)
    for b in range(B):
        for slab, ln in (("sparse_kv_cache", "sparse_kv_len"), ("compress_kv_cache", "compress_kv_len"),
                         ("before_compress_kv_cache", "before_compress_kv_len")):
            n = int(getattr(caches[1], ln)[b])
            assert torch.equal(getattr(caches[0], slab)[:, b, :n], getattr(caches[1], slab)[:, b, :n]), (slab, b)
        n = min(int(caches[1].sliding_kv_len[b]), W)
        assert torch.equal(caches[0].sliding_kv_cache[:, b, :n], caches[1].sliding_kv_cache[:, b, :n]), ("ring", b)


def test_graphed_decode_refuses_to_outgrow_the_cache(device):
    """A recorded step cannot check lengths on the host: the cache counts the decode steps run on it (replays and eager
    steps alike) and raises before the longest sequence would need a row it does not have; a new prefill restarts the count."""
    from native_sparse_attention.infer import NSADecodeGraph
    from native_sparse_attention.module import RopeConfig, RotaryEmbedding
    Hq, Hkv, d, ks, st, bs, topk, W = 16, 2, 128, 32, 16, 64, 4, 64
    lens = [70, 33]
    g = torch.Generator(device=device).manual_seed(3)
    cu = cu_from_lens(lens, device)
    T = int(cu[-1])
    rope = RotaryEmbedding(RopeConfig(head_dim=d), device=device)
    wk = torch.softmax(torch.randn(Hkv, ks, generator=g, device=device), -1).bfloat16()

    def rnd(*shape):
        return torch.randn(*shape, generator=g, device=device).bfloat16()

    cache = NSACache(2, max(lens) + 3, Hkv, d, ks, st, W, torch.bfloat16, device)
    tail = ((wk, wk), (weightedpool_compress, weightedpool_compress), None, ks, st, bs, topk, 1, 2, W)
    prefill = lambda: nsa_infer(cu, 0, rnd(T, Hq, d), rnd(T, Hkv, d), rnd(T, Hkv, d), torch.sigmoid(rnd(T, Hq, 3).float()).bfloat16(), rope, cache, *tail)
    prefill()
    graph = NSADecodeGraph(cu, Hq, rope, cache, *tail)
    tok = lambda: (rnd(2, Hq, d), rnd(2, Hkv, d), rnd(2, Hkv, d), torch.sigmoid(rnd(2, Hq, 3).float()).bfloat16())
    for _ in range(3):
        graph.step(*tok())
    with pytest.raises(RuntimeError):
        graph.step(*tok())
    assert int(cache.sparse_kv_len[0]) == 73          # the refused step touched nothing
    prefill()
    graph.step(*tok())                                 # the count restarted with the new prompt
    assert int(cache.sparse_kv_len[0]) == 71
    # eager steps and replays on one cache are counted together: one replay above, two eager steps here, then neither fits
    for step in (2, 3):
        nsa_infer(cu, step, *tok(), rope, cache, *tail)
    assert int(cache.sparse_kv_len[0]) == 73 and cache.decode_steps == 3
    with pytest.raises(RuntimeError):
        graph.step(*tok())
    with pytest.raises((RuntimeError, AssertionError)):
        nsa_infer(cu, 4, *tok(), rope, cache, *tail)
    assert int(cache.sparse_kv_len[0]) == 73
