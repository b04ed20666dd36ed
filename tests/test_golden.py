"""The oracle against the committed known-answer fixtures (tests/golden/*.npz, made by scalar-loop
statements of the definitions in tests/golden/make_golden.py)."""
import os

import numpy as np
import torch

import oracle

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    z = np.load(os.path.join(GOLDEN, name + ".npz"))
    return {k: (torch.from_numpy(z[k]) if z[k].ndim else int(z[k])) for k in z.files}


def f64(x):
    return x.to(torch.float64)


def test_topk_sparse_attention_fixture():
    g = load("topk_sparse_attention")
    o, lse = oracle.topk_sparse_attention(f64(g["q"]), f64(g["k"]), f64(g["v"]), g["topk_idx"], g["block_size"], g["cu_seqlens"], return_lse=True)
    assert torch.allclose(o, g["o"], atol=1e-12)
    assert torch.allclose(lse.double(), g["lse"], atol=1e-5)         # the oracle keeps the LSE in fp32


def test_compress_fixture():
    g = load("compress")
    ks, st, cu = g["kernel_size"], g["kernel_stride"], g["cu_seqlens"]
    y, ycu = oracle.avgpool_compress(f64(g["x"]), None, cu, ks, st)
    assert torch.equal(ycu.cpu().int(), g["y_cu_seqlens"]) and torch.allclose(y, g["y_avg"], atol=1e-12)
    y, _ = oracle.weightedpool_compress(f64(g["x"]), f64(g["w_pool"]), cu, ks, st)
    assert torch.allclose(y, g["y_pool"], atol=1e-12)
    y, _ = oracle.linear_compress(f64(g["x"]), f64(g["w_lin"]), cu, ks, st)
    assert torch.allclose(y, g["y_lin"], atol=1e-12)


def test_compressed_attention_fixture():
    g = load("compressed_attention")
    out, idx, bscore = oracle.compressed_attention(
        f64(g["q"]), f64(g["k"]), f64(g["v"]), g["kernel_size"], g["kernel_stride"], g["block_size"], g["topk"],
        g["cu_seqlens_q"], g["cu_seqlens_k"], return_scores=True)
    assert torch.allclose(out, g["out"], atol=1e-12)
    assert torch.allclose(bscore.double(), g["block_score"], atol=1e-6)   # fp32 scores; +inf entries compare equal
    assert torch.equal(idx, g["topk_idx"])


def test_decode_fixture():
    g = load("decode")
    o = oracle.dense_attention_decode(f64(g["q"]), f64(g["k"]), f64(g["v"]), g["seqlens"])
    assert torch.allclose(o, g["o_dense"], atol=1e-12)
    o = oracle.topk_sparse_attention_decode(f64(g["q"]), f64(g["k"]), f64(g["v"]), g["topk_idx"], g["block_size"], g["seqlens"])
    assert torch.allclose(o, g["o_topk"], atol=1e-12)
