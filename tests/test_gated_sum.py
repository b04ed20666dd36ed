"""GPU parity of the gated sum of the three branches (forward and backward through the C ABI) against the
element-wise tensor expression of the reference's layer (module/native_sparse_attention.py:228-232)."""
import pytest
import torch

from native_sparse_attention.ops.gated_sum import gate_combine, gated_sum

pytestmark = pytest.mark.gpu


def _expression(gate, a, b, c):
    return gate[..., 0:1] * a + gate[..., 1:2] * b + gate[..., 2:3] * c


@pytest.mark.parametrize("n,H,d,dtype", [
    (1000, 64, 128, torch.bfloat16),
    (333, 6, 96, torch.float16),        # rows of 12 threads: workgroups with idle threads
    (17, 3, 64, torch.bfloat16),
    (5, 40, 32, torch.float16),
])
def test_forward_bit_exact_and_backward(device, n, H, d, dtype):
    print("case", n, H, d, dtype, flush=True)
    g = torch.Generator(device=device).manual_seed(0)
    gate = torch.sigmoid(torch.randn(n, H, 3, generator=g, device=device)).to(dtype)
    # branches as slices of wider tensors: token and head strides differ from the dense ones
    wide = torch.randn(3, n, H, d + 8, generator=g, device=device).to(dtype)
    a, b, c = (wide[i, :, :, :d] for i in range(3))
    dout = torch.randn(n, H, d, generator=g, device=device).to(dtype)
    leaves = [t.clone().requires_grad_() for t in (gate, a, b, c)]
    out = gated_sum(*leaves)
    ref_leaves = [t.clone().requires_grad_() for t in (gate, a, b, c)]
    want = _expression(*ref_leaves)
    assert torch.equal(out, want) and torch.equal(gate_combine(gate, a, b, c), want)
    out.backward(dout)
    want.backward(dout)
    for name, x, y in zip(("da", "db", "dc"), leaves[1:], ref_leaves[1:]):
        assert torch.equal(x.grad, y.grad), name                     # one product, one rounding
    # dgate: the same rounded products, summed in fp32 in a different order, rounded once
    err = (leaves[0].grad.float() - ref_leaves[0].grad.float()).abs()
    tol = 2.0 ** (-7 if dtype == torch.bfloat16 else -10) * ref_leaves[0].grad.float().abs().clamp(min=1.0)
    assert (err <= tol).all(), err.max().item()
    # and against an fp32 evaluation of the same sums
    exact = torch.stack([(dout.float() * t.float()).sum(-1) for t in (a, b, c)], -1)
    assert (leaves[0].grad.float() - exact).abs().max() <= 0.05 * exact.abs().max().clamp(min=1.0)


def test_empty(device):
    gate = torch.zeros(0, 4, 3, device=device, dtype=torch.bfloat16)
    x = torch.zeros(0, 4, 64, device=device, dtype=torch.bfloat16, requires_grad=True)
    out = gated_sum(gate, x, x, x)
    assert out.shape == (0, 4, 64)
    out.sum().backward()
    assert x.grad.shape == x.shape
