"""The forward operator pipeline of the reference's README.md:46-93 at the size of the pipeline benchmark: a varlen batch
cu_seqlens = [0, 1024, 8192, 16384], 64 query / 4 KV heads, head_dim 128; linear_compress (kernel 32, stride 16, a weight
per tensor, the intra-block position term on the keys only) -> compressed_attention (block 64, top-16, one initial and
two local blocks) -> topk_sparse_attention on the block ids the compressed stage selected.  Every stage is checked
against the oracle on the inputs the HIP stage before it produced (so an error cannot hide behind the next stage's
tolerance); the ids are bit-exact wherever the oracle's decision margin exceeds 1e-3."""
import pytest
import torch

import oracle
from helpers import assert_close, assert_ids_match
from native_sparse_attention.ops import compressed_attention, linear_compress, topk_sparse_attention
from native_sparse_attention.testing import cu_from_lens

pytestmark = pytest.mark.gpu


def test_linear_compress_compressed_attention_topk_attention_chain(device):
    lens, Hq, Hkv, d, ks, st, bs, topk = [1024, 7168, 8192], 64, 4, 128, 32, 16, 64, 16
    g = torch.Generator(device=device).manual_seed(0)
    cu = cu_from_lens(lens, device)
    T = int(cu[-1])
    q = torch.randn(T, Hq, d, generator=g, device=device).bfloat16()
    k = torch.randn(T, Hkv, d, generator=g, device=device).bfloat16()
    v = torch.randn(T, Hkv, d, generator=g, device=device).bfloat16()
    wk = (torch.randn(Hkv, ks * d, d, generator=g, device=device) / (ks * d) ** 0.5).bfloat16()
    wv = (torch.randn(Hkv, ks * d, d, generator=g, device=device) / (ks * d) ** 0.5).bfloat16()
    pe = (0.02 * torch.randn(Hkv, ks, d, generator=g, device=device)).bfloat16()

    # stage 1: compression
    ck, cuk = linear_compress(k, wk, cu, ks, st, pe)
    cv, cuv = linear_compress(v, wv, cu, ks, st, None)
    want_ck, want_cuk = oracle.linear_compress(k.float(), wk.float(), cu, ks, st, pe.float())
    want_cv, _ = oracle.linear_compress(v.float(), wv.float(), cu, ks, st, None)
    assert cuk.dtype == torch.int32 and cuk.tolist() == want_cuk.tolist() == [0, 63, 510, 1021] and torch.equal(cuk, cuv)
    assert_close(ck, want_ck, "compressed k", rel_to=want_ck.abs().max().item())
    assert_close(cv, want_cv, "compressed v", rel_to=want_cv.abs().max().item())

    # stage 2: attention over the compressed keys + block selection, on the compressed tokens the kernels produced
    o_cmp, idx = compressed_attention(q, ck, cv, ks, st, bs, topk, cu, cuk, max(lens), 511, None, 1, 2)
    want_cmp, want_idx, bscore = oracle.compressed_attention(q.float(), ck.float(), cv.float(), ks, st, bs, topk, cu, cuk, max(lens), 511,
                                                             None, 1, 2, return_scores=True)
    assert_close(o_cmp, want_cmp, "compressed attention output")
    assert idx.shape == (Hkv, T, topk)
    qb = torch.cat([torch.arange(L, device=device) for L in lens]) // bs
    assert_ids_match(idx, want_idx, bscore, qb, "topk_idx")

    # stage 3: block-sparse attention on the selected ids
    o = topk_sparse_attention(q, k, v, idx, bs, cu)
    want = oracle.topk_sparse_attention(q.float(), k.float(), v.float(), idx, bs, cu)
    assert_close(o, want, "sparse attention output")
