"""NativeSparseAttention layer on the GPU: the training forward/backward against a restatement that keeps
the layer's own front part (projections, compression, rotary embedding, block selection, all deterministic
calls) and replaces the three attention branches, the gate and the output projection by fp32 oracle code;
and cached inference against the training forward."""
import pytest
import torch

import oracle
from helpers import assert_close
from native_sparse_attention.module import NativeSparseAttention, NSACache, RopeConfig
from native_sparse_attention.ops import compressed_attention
from native_sparse_attention.testing import cu_from_lens

pytestmark = pytest.mark.gpu

CFG = dict(hidden_size=256, num_q_heads=8, num_kv_heads=2, head_dim=64, kernel_size=32, kernel_stride=16, block_size=64, topk=4,
           init_blocks=1, local_blocks=2, window_size=512)


def _layer(compress_type, device, seed=0):
    torch.manual_seed(seed)
    layer = NativeSparseAttention(compress_type=compress_type, rope_config=RopeConfig(head_dim=64), rope_device=device, **CFG)
    layer = layer.to(device).to(torch.bfloat16)
    with torch.no_grad():                       # parameters that start at zero would hide wiring mistakes
        layer.intra_block_pe.normal_(0, 0.02)
    return layer


def _window_reference(q, k, v, lens, W):
    G = q.shape[1] // k.shape[1]
    outs, s0 = [], 0
    for L in lens:
        i = torch.arange(L, device=q.device)
        mask = (i[None, :] <= i[:, None]) & (i[None, :] >= i[:, None] - W)
        s = torch.einsum("qhd,khd->hqk", q[s0:s0 + L], k[s0:s0 + L].repeat_interleave(G, 1)) / q.shape[-1] ** 0.5
        p = torch.softmax(s.masked_fill(~mask[None], float("-inf")), -1)
        outs.append(torch.einsum("hqk,khd->qhd", p, v[s0:s0 + L].repeat_interleave(G, 1)))
        s0 += L
    return torch.cat(outs)


@pytest.mark.parametrize("compress_type", ["avgpool", "weightedpool", "linear"])
def test_training_forward_backward(device, compress_type):
    lens = [300, 130, 20]                       # the last sequence is shorter than one compression window
    layer = _layer(compress_type, device)
    cu = cu_from_lens(lens, device)
    g = torch.Generator(device=device).manual_seed(5)
    x = torch.empty(int(cu[-1]), CFG["hidden_size"], device=device).uniform_(-1, 1, generator=g).bfloat16().requires_grad_()
    y = layer(x, cu)
    assert y.shape == x.shape and y.dtype == x.dtype

    H, Hkv, d = CFG["num_q_heads"], CFG["num_kv_heads"], CFG["head_dim"]
    ks, st, bs = CFG["kernel_size"], CFG["kernel_stride"], CFG["block_size"]
    with torch.no_grad():
        xd = x.detach()
        q = layer.proj_q(xd).view(-1, H, d)
        k = layer.proj_k(xd).view(-1, Hkv, d)
        v = layer.proj_v(xd).view(-1, Hkv, d)
        ck, ccu = layer.compress_func(k, layer.compress_key, cu, ks, st, layer.intra_block_pe)
        cv, _ = layer.compress_func(v, layer.compress_value, cu, ks, st, None)
        q = layer.rope(q, cu)
        ck = layer.rope(ck, ccu, stride=st)
        k = layer.rope(k, cu)
        _, idx = compressed_attention(q, ck, cv, ks, st, bs, CFG["topk"], cu, ccu, None, None, None, 1, 2)
        qf, kf, vf, ckf, cvf = (t.float() for t in (q, k, v, ck, cv))
        cmp_out, _ = oracle.compressed_attention(qf, ckf, cvf, ks, st, bs, -1, cu, ccu)
        sel_out = oracle.topk_sparse_attention(qf, kf, vf, idx, bs, cu)
        win_out = _window_reference(qf, kf, vf, lens, CFG["window_size"])
        gate = layer.gate(xd).float().view(-1, H, 3)
        mix = gate[..., 0:1] * cmp_out + gate[..., 1:2] * sel_out + gate[..., 2:3] * win_out
        want = mix.reshape(-1, H * d) @ layer.proj_o.weight.float().t()
    assert_close(y, want, "layer output", rel_to=max(1.0, want.abs().max().item()))

    (y.float() * torch.randn(y.shape, generator=g, device=device)).sum(-1).mean().backward()
    assert torch.isfinite(x.grad).all() and x.grad.abs().max() > 0
    for name, p in layer.named_parameters():
        assert p.grad is not None and torch.isfinite(p.grad).all(), name
        assert p.grad.abs().max() > 0, name


def test_cached_inference_matches_training_forward(device):
    lens, steps = [200, 90, 333], 6             # all sequences stay shorter than the window
    layer = _layer("weightedpool", device, seed=1).eval()
    B = len(lens)
    g = torch.Generator(device=device).manual_seed(9)
    total = [L + steps for L in lens]
    full_cu = cu_from_lens(total, device)
    x_full = torch.empty(int(full_cu[-1]), CFG["hidden_size"], device=device).uniform_(-1, 1, generator=g).bfloat16()
    with torch.no_grad():
        y_full = layer(x_full, full_cu)
    starts = [int(full_cu[b]) for b in range(B)]
    cu = cu_from_lens(lens, device)
    prompt = torch.cat([x_full[s:s + L] for s, L in zip(starts, lens)])
    cache = NSACache(B, max(total) + 8, CFG["num_kv_heads"], CFG["head_dim"], CFG["kernel_size"], CFG["kernel_stride"],
                     CFG["window_size"], torch.bfloat16, device)
    y0 = layer.inference(prompt, cu, 0, cache)
    want0 = torch.cat([y_full[s:s + L] for s, L in zip(starts, lens)])
    assert_close(y0, want0.float(), "prefill", rel_to=max(1.0, want0.abs().max().item()))
    for step in range(1, steps + 1):
        rows = torch.tensor([s + L + step - 1 for s, L in zip(starts, lens)], device=device)
        y = layer.inference(x_full[rows], cu, step, cache)
        assert_close(y, y_full[rows].float(), "decode step %d" % step, rel_to=max(1.0, y_full[rows].abs().max().item()))
