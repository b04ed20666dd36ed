"""GPU parity of the sliding-window varlen attention (forward and backward, through the C ABI) against a
plain fp32 masked-softmax reference.  The reference repository delegates this operator to flash-attn
(absent here): the visibility rule i - W <= j <= i is flash-attn's documented window_size=(W, -1) with
causal=True; nothing in the reference's own tests pins the windowed call."""
import pytest
import torch

from helpers import assert_close
from native_sparse_attention.ops.sliding_window import sliding_window_attention_varlen
from native_sparse_attention.testing import cu_from_lens

pytestmark = pytest.mark.gpu


def _reference(q, k, v, lens, W, scale=None):
    G = q.shape[1] // k.shape[1]
    scale = q.shape[-1] ** -0.5 if scale is None else scale
    outs, s0 = [], 0
    for L in lens:
        i = torch.arange(L, device=q.device)
        mask = (i[None, :] <= i[:, None]) & (i[None, :] >= i[:, None] - W)
        qs, ks, vs = q[s0:s0 + L], k[s0:s0 + L].repeat_interleave(G, 1), v[s0:s0 + L].repeat_interleave(G, 1)
        s = torch.einsum("qhd,khd->hqk", qs, ks) * scale
        p = torch.softmax(s.masked_fill(~mask[None], float("-inf")), -1)
        outs.append(torch.einsum("hqk,khd->qhd", p, vs))
        s0 += L
    return torch.cat(outs)


@pytest.mark.parametrize("lens,Hq,Hkv,d,W,dtype", [
    ([100, 300, 77], 8, 2, 64, 32, torch.bfloat16),
    ([700, 90, 1300], 16, 1, 128, 256, torch.bfloat16),      # G = 16
    ([65, 130], 4, 4, 32, 0, torch.float16),                  # each position sees only itself
    ([513, 40], 40, 2, 96, 1 << 20, torch.float16),           # window beyond every sequence: plain causal; G = 20
    ([2049], 64, 4, 128, 512, torch.bfloat16),                # benchmark head layout
])
def test_forward_backward(device, lens, Hq, Hkv, d, W, dtype):
    print("case", lens, Hq, Hkv, d, W, dtype, flush=True)
    g = torch.Generator(device=device).manual_seed(3)
    cu = cu_from_lens(lens, device)
    T = int(cu[-1])
    q, k, v = (torch.randn(T, h, d, generator=g, device=device).to(dtype) for h in (Hq, Hkv, Hkv))
    do = torch.randn(T, Hq, d, generator=g, device=device).to(dtype)
    q1, k1, v1 = (x.clone().requires_grad_() for x in (q, k, v))
    o = sliding_window_attention_varlen(q1, k1, v1, cu, W)
    o.backward(do)
    qf, kf, vf = (x.float().requires_grad_() for x in (q, k, v))
    want = _reference(qf, kf, vf, lens, W)
    want.backward(do.float())
    assert_close(o, want, "o")
    assert_close(q1.grad, qf.grad, "dq", rel_to=qf.grad.abs().max().item())
    assert_close(k1.grad, kf.grad, "dk", rel_to=kf.grad.abs().max().item())
    assert_close(v1.grad, vf.grad, "dv", rel_to=vf.grad.abs().max().item())


@pytest.mark.parametrize("scale", [-0.2, 0.0])
def test_any_finite_scale(device, scale):
    """Forward and backward at a negative and at a zero softmax scale (the window kernels share their scale handling with
    the compressed-attention kernels; the dense varlen operator runs the same kernels in its causal mode)."""
    from native_sparse_attention.ops.flash_attention import flash_attention_varlen

    lens, Hq, Hkv, d, W = [200, 333], 8, 2, 64, 48
    g = torch.Generator(device=device).manual_seed(6)
    cu = cu_from_lens(lens, device)
    T = int(cu[-1])
    q, k, v = (torch.randn(T, h, d, generator=g, device=device).bfloat16() for h in (Hq, Hkv, Hkv))
    q = (q.float() * 0.5).bfloat16()
    do = torch.randn(T, Hq, d, generator=g, device=device).bfloat16()
    for name, fn, win in (("window", lambda a, b, c: sliding_window_attention_varlen(a, b, c, cu, W, scale), W),
                          ("causal", lambda a, b, c: flash_attention_varlen(a, b, c, cu, cu, max(lens), max(lens), True, scale), 1 << 20)):
        q1, k1, v1 = (x.clone().requires_grad_() for x in (q, k, v))
        o = fn(q1, k1, v1)
        o.backward(do)
        qf, kf, vf = (x.float().requires_grad_() for x in (q, k, v))
        want = _reference(qf, kf, vf, lens, win, scale)
        want.backward(do.float())
        assert_close(o, want, name + " o")
        for gname, a, b in (("dq", q1.grad, qf.grad), ("dk", k1.grad, kf.grad), ("dv", v1.grad, vf.grad)):
            assert_close(a, b, name + " " + gname, rel_to=True)
