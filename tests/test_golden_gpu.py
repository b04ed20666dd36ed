"""The HIP operators (through the C ABI) against the committed known-answer fixtures."""
import pytest
import torch

from helpers import assert_close
from native_sparse_attention.ops import (avgpool_compress, compressed_attention, flash_attention_decode, linear_compress,
                                         topk_sparse_attention, topk_sparse_attention_decode, weightedpool_compress)
from test_golden import load

pytestmark = pytest.mark.gpu


def dev(g, device, dtype=torch.bfloat16):
    return {k: (v.to(device).to(dtype) if torch.is_tensor(v) and v.is_floating_point() and v.dtype == torch.float32 else
                (v.to(device) if torch.is_tensor(v) else v)) for k, v in g.items()}


def test_topk_sparse_attention_fixture(device):
    g = dev(load("topk_sparse_attention"), device)
    o = topk_sparse_attention(g["q"], g["k"], g["v"], g["topk_idx"], g["block_size"], g["cu_seqlens"])
    assert_close(o, g["o"].float(), "o")


def test_compress_fixture(device):
    g = dev(load("compress"), device)
    ks, st, cu = g["kernel_size"], g["kernel_stride"], g["cu_seqlens"]
    y, ycu = avgpool_compress(g["x"], None, cu, ks, st)
    assert torch.equal(ycu, g["y_cu_seqlens"])
    assert_close(y, g["y_avg"].float(), "avgpool")
    y, _ = weightedpool_compress(g["x"], g["w_pool"], cu, ks, st)
    assert_close(y, g["y_pool"].float(), "weightedpool")
    y, _ = linear_compress(g["x"], g["w_lin"], cu, ks, st)
    assert_close(y, g["y_lin"].float(), "linear", rel_to=g["y_lin"].abs().max().item())


def test_compressed_attention_fixture(device):
    g = dev(load("compressed_attention"), device)
    out, idx = compressed_attention(g["q"], g["k"], g["v"], g["kernel_size"], g["kernel_stride"], g["block_size"], g["topk"],
                                    g["cu_seqlens_q"], g["cu_seqlens_k"])
    assert_close(out, g["out"].float(), "out")
    # bit-exact rows wherever the fixture's own scores separate the last selected from the best rejected block
    sc = g["block_score"]                                           # [Hkv, T, nb], +inf on forced blocks
    want = g["topk_idx"]
    sel = torch.zeros_like(sc, dtype=torch.bool).scatter_(2, want.clamp(min=0).long(), want >= 0)
    worst_in = torch.where(sel, sc, torch.full_like(sc, float("inf"))).amin(-1)
    best_out = torch.where(sel, torch.full_like(sc, float("-inf")), sc).amax(-1)
    clear = (worst_in - best_out) > 1e-3
    exact = (idx == want).all(-1)
    assert exact[clear].all()
    assert exact.float().mean() > 0.99


def test_decode_fixture(device):
    g = dev(load("decode"), device)
    o = flash_attention_decode(g["q"], g["k"], g["v"], g["seqlens"])
    assert_close(o, g["o_dense"].float(), "dense decode")
    o = topk_sparse_attention_decode(g["q"], g["k"], g["v"], g["topk_idx"], g["block_size"], g["seqlens"])
    assert_close(o, g["o_topk"].float(), "topk decode")
