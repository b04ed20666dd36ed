"""GPU parity of flash_attention_varlen (dense varlen attention, forward and backward, through the C ABI) against
a plain fp32 masked softmax, with the reference's conventions (ops/triton/flash_attention.py:117-131): causal masks
are aligned at the start of the query and key sequences; GQA groups consecutive query heads unless gqa_interleave."""
import pytest
import torch

from helpers import assert_close
from native_sparse_attention.ops import flash_attention_varlen
from native_sparse_attention.testing import cu_from_lens

pytestmark = pytest.mark.gpu


def _reference(q, k, v, lens_q, lens_k, causal, interleave):
    Hq, Hkv = q.shape[1], k.shape[1]
    G = Hq // Hkv
    kv_of = [h % Hkv if interleave else h // G for h in range(Hq)]
    outs, sq, sk = [], 0, 0
    for Lq, Lk in zip(lens_q, lens_k):
        qs, ks, vs = q[sq:sq + Lq], k[sk:sk + Lk][:, kv_of], v[sk:sk + Lk][:, kv_of]
        s = torch.einsum("qhd,khd->hqk", qs, ks) / q.shape[-1] ** 0.5
        if causal:
            mask = torch.arange(Lk, device=q.device)[None, :] <= torch.arange(Lq, device=q.device)[:, None]
            s = s.masked_fill(~mask[None], float("-inf"))
        p = torch.softmax(s, -1).nan_to_num(0.0)
        outs.append(torch.einsum("hqk,khd->qhd", p, vs))
        sq += Lq
        sk += Lk
    return torch.cat(outs)


@pytest.mark.parametrize("lens_q,lens_k,Hq,Hkv,d,causal,interleave,dtype", [
    ([1000, 4000, 8192], [1000, 4000, 8192], 32, 2, 128, True, False, torch.bfloat16),   # the reference's own test sizes
    ([100, 300, 77], [100, 300, 77], 8, 2, 64, False, False, torch.bfloat16),
    ([128, 40], [300, 17], 4, 4, 32, False, False, torch.float16),                        # cross lengths
    ([200, 64], [90, 500], 6, 2, 96, True, False, torch.float16),                         # causal with different lengths, G = 3
    ([257], [257], 8, 2, 64, True, True, torch.bfloat16),                                 # interleaved GQA
])
def test_forward_backward(device, lens_q, lens_k, Hq, Hkv, d, causal, interleave, dtype):
    print("case", lens_q, lens_k, Hq, Hkv, d, causal, interleave, dtype, flush=True)
    g = torch.Generator(device=device).manual_seed(11)
    cu_q, cu_k = cu_from_lens(lens_q, device), cu_from_lens(lens_k, device)
    q = torch.randn(int(cu_q[-1]), Hq, d, generator=g, device=device).to(dtype)
    k, v = (torch.randn(int(cu_k[-1]), Hkv, d, generator=g, device=device).to(dtype) for _ in range(2))
    do = torch.randn(q.shape, generator=g, device=device).to(dtype)
    q1, k1, v1 = (x.clone().requires_grad_() for x in (q, k, v))
    o = flash_attention_varlen(q1, k1, v1, cu_q, cu_k, max(lens_q), max(lens_k), causal, None, interleave)
    o.backward(do)
    qf, kf, vf = (x.float().requires_grad_() for x in (q, k, v))
    want = _reference(qf, kf, vf, lens_q, lens_k, causal, interleave)
    want.backward(do.float())
    assert_close(o, want, "o")
    assert_close(q1.grad, qf.grad, "dq", rel_to=qf.grad.abs().max().item())
    assert_close(k1.grad, kf.grad, "dk", rel_to=kf.grad.abs().max().item())
    assert_close(v1.grad, vf.grad, "dv", rel_to=vf.grad.abs().max().item())
