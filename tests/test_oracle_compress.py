"""Pins oracle.compress against library pooling / convolution routines (CPU)."""
import torch
import torch.nn.functional as F

import oracle

LENS = [12, 100, 257, 64]   # one sequence shorter than the kernel, one exactly two windows short of ragged
KS, ST = 32, 16


def _setup(H=3, d=8, dtype=torch.float64):
    torch.manual_seed(0)
    cu = torch.tensor([0, 12, 112, 369, 433], dtype=torch.int32)
    x = torch.randn(int(cu[-1]), H, d, dtype=dtype)
    return x, cu


def test_seqlens_closed_form():
    _, cu = _setup()
    y, ycu = oracle.compressed_seqlens(cu, KS, ST)
    assert y.tolist() == [0, 5, 15, 3] and ycu.tolist() == [0, 0, 5, 20, 23] and ycu.dtype == torch.int32


def test_avgpool_is_avg_pool1d():
    x, cu = _setup()
    pe = torch.randn(3, KS, 8, dtype=torch.float64)
    y, ycu = oracle.avgpool_compress(x, None, cu, KS, ST, pe)
    parts = []
    for b in range(4):
        xs = x[cu[b]:cu[b + 1]]
        if xs.shape[0] >= KS:
            parts.append(F.avg_pool1d(xs.permute(1, 2, 0), KS, ST).permute(2, 0, 1))
    want = torch.cat(parts) + pe.mean(1)[None]
    assert torch.allclose(y, want, atol=1e-12) and y.shape[0] == int(ycu[-1])


def test_weightedpool_is_grouped_conv1d():
    x, cu = _setup()
    H, d = 3, 8
    w = torch.randn(H, KS, dtype=torch.float64)
    pe = torch.randn(H, KS, d, dtype=torch.float64)
    y, _ = oracle.weightedpool_compress(x, w, cu, KS, ST, pe)
    parts = []
    for b in range(4):
        xs = x[cu[b]:cu[b + 1]]
        if xs.shape[0] >= KS:
            inp = xs.reshape(-1, H * d).t()[None]                         # [1, H*d, L]
            ker = w.repeat_interleave(d, 0)[:, None, :]                   # one filter per (h, d) channel
            parts.append(F.conv1d(inp, ker, stride=ST, groups=H * d)[0].t().reshape(-1, H, d))
    bias = torch.stack([(pe[h] * w[h][:, None]).sum(0) for h in range(H)])
    assert torch.allclose(y, torch.cat(parts) + bias[None], atol=1e-10)


def test_linear_is_conv1d_per_head():
    x, cu = _setup()
    H, d = 3, 8
    w = torch.randn(H, KS * d, d, dtype=torch.float64)
    pe = torch.randn(H, KS, d, dtype=torch.float64)
    y, _ = oracle.linear_compress(x, w, cu, KS, ST, pe)
    parts = []
    for b in range(4):
        xs = x[cu[b]:cu[b + 1]]
        if xs.shape[0] < KS:
            continue
        per_head = []
        for h in range(H):
            ker = w[h].reshape(KS, d, d).permute(2, 1, 0)                  # [out, in, k]
            per_head.append(F.conv1d(xs[:, h].t()[None], ker, stride=ST)[0].t())
        parts.append(torch.stack(per_head, 1))
    bias = torch.stack([pe[h].reshape(-1) @ w[h] for h in range(H)])
    assert torch.allclose(y, torch.cat(parts) + bias[None], atol=1e-9)
