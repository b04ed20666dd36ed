"""GPU parity of the compression operators (through the C ABI) against the oracle."""
import pytest
import torch

import oracle
from helpers import assert_close
from native_sparse_attention.ops import avgpool_compress, weightedpool_compress
from native_sparse_attention.testing import cu_from_lens

pytestmark = pytest.mark.gpu

POOL_CASES = [
    # lens, H, d, ks, st, dtype
    ([12, 1000, 2000, 4096], 4, 128, 32, 16, torch.bfloat16),     # the reference's own check (one sequence < kernel)
    ([31, 32, 33, 47, 48], 2, 64, 32, 16, torch.float16),          # window-count edges
    ([700, 129], 3, 96, 16, 16, torch.bfloat16),                   # non-overlapping windows, d=96
    ([5000], 2, 128, 64, 16, torch.bfloat16),
    ([300, 260], 1, 192, 128, 32, torch.float16),
]


def _inputs(lens, H, d, ks, dtype, device, seed=0):
    g = torch.Generator(device=device).manual_seed(seed)
    cu = cu_from_lens(lens, device)
    x = torch.randn(int(cu[-1]), H, d, generator=g, device=device).to(dtype)
    w = torch.softmax(torch.randn(H, ks, generator=g, device=device), -1).to(dtype)
    pe = (0.02 * torch.randn(H, ks, d, generator=g, device=device)).to(dtype)
    return x, w, pe, cu


@pytest.mark.parametrize("lens,H,d,ks,st,dtype", POOL_CASES)
@pytest.mark.parametrize("weighted", [True, False])
def test_pool_forward_backward(device, lens, H, d, ks, st, dtype, weighted):
    print("case", lens, H, d, ks, st, dtype, weighted, flush=True)
    x, w, pe, cu = _inputs(lens, H, d, ks, dtype, device)
    fn, ofn = (weightedpool_compress, oracle.weightedpool_compress) if weighted else (avgpool_compress, oracle.avgpool_compress)
    x1 = x.clone().requires_grad_()
    w1 = w.clone().requires_grad_() if weighted else None
    pe1 = pe.clone().requires_grad_()
    y, ycu = fn(x1, w1, cu, ks, st, pe1)
    xf, pef = x.float().requires_grad_(), pe.float().requires_grad_()
    wf = w.float().requires_grad_() if weighted else None
    want, want_cu = ofn(xf, wf, cu, ks, st, pef)
    assert ycu.dtype == torch.int32 and torch.equal(ycu.cpu(), want_cu.cpu())
    assert y.shape == want.shape and y.dtype == dtype
    assert_close(y, want, "y")
    g = torch.Generator(device=device).manual_seed(3)
    dy = torch.randn(y.shape, generator=g, device=device).to(dtype)
    y.backward(dy)
    want.backward(dy.float())
    assert_close(x1.grad, xf.grad, "dx")
    assert_close(pe1.grad, pef.grad, "dpe", rel_to=pef.grad.abs().max().item())
    if weighted:
        assert_close(w1.grad, wf.grad, "dw", rel_to=wf.grad.abs().max().item())


def test_pool_strided_input_and_short_batch(device):
    # x as a slice of a fused projection; every sequence shorter than the kernel -> empty output
    g = torch.Generator(device=device).manual_seed(1)
    cu = cu_from_lens([500, 40], device)
    kv = torch.randn(540, 6, 128, generator=g, device=device).bfloat16()
    x = kv[:, 2:4]
    w = torch.softmax(torch.randn(2, 32, generator=g, device=device), -1).bfloat16()
    y, ycu = weightedpool_compress(x, w, cu, 32, 16)
    want, _ = oracle.weightedpool_compress(x.float(), w.float(), cu, 32, 16)
    assert_close(y, want, "y")
    cu2 = cu_from_lens([10, 31], device)
    y2, ycu2 = avgpool_compress(kv[:41, :2], None, cu2, 32, 16)
    assert y2.shape == (0, 2, 128) and ycu2.tolist() == [0, 0, 0]


def test_pool_asserts(device):
    x = torch.randn(64, 2, 64, device=device).bfloat16()
    cu = cu_from_lens([64], device)
    with pytest.raises(AssertionError):
        avgpool_compress(x, torch.ones(2, 32, device=device).bfloat16(), cu, 32, 16)   # avgpool takes no weight
    with pytest.raises(AssertionError):
        weightedpool_compress(x, torch.ones(2, 32, device=device), cu, 32, 16)          # dtype mismatch
    with pytest.raises(AssertionError):
        weightedpool_compress(x, torch.ones(2, 24, device=device).bfloat16(), cu, 24, 8)  # kernel size set


LINEAR_CASES = [
    # lens, H, d, ks, st, dtype
    ([1024, 7168, 8192], 4, 128, 32, 16, torch.bfloat16),         # pipeline benchmark shape (32 rows per workgroup)
    ([12, 100, 257, 64], 2, 64, 32, 16, torch.float16),
    ([300, 75], 3, 96, 16, 16, torch.bfloat16),
    ([500], 2, 192, 32, 16, torch.float16),                        # the reference's d=192 smoke shape
    ([900, 130], 1, 32, 64, 32, torch.bfloat16),
    ([17000, 40], 4, 64, 16, 4, torch.bfloat16),                   # enough outputs for 64 rows per workgroup
    ([9000, 8200], 4, 96, 16, 4, torch.float16),                   # the same with d=96
    ([4200, 4100, 31], 8, 128, 16, 4, torch.bfloat16),             # the same with d=128
    ([4200, 4100, 31], 2, 32, 16, 4, torch.bfloat16),              # 32 rows per workgroup, d=32
]


@pytest.mark.parametrize("lens,H,d,ks,st,dtype", LINEAR_CASES)
def test_linear_compress_forward_backward(device, lens, H, d, ks, st, dtype):
    from native_sparse_attention.ops import linear_compress
    print("case", lens, H, d, ks, st, dtype, flush=True)
    g = torch.Generator(device=device).manual_seed(0)
    cu = cu_from_lens(lens, device)
    x = torch.randn(int(cu[-1]), H, d, generator=g, device=device).to(dtype)
    w = (torch.randn(H, ks * d, d, generator=g, device=device) / (ks * d) ** 0.5).to(dtype)
    pe = (0.02 * torch.randn(H, ks, d, generator=g, device=device)).to(dtype)
    x1, w1, pe1 = (t.clone().requires_grad_() for t in (x, w, pe))
    y, ycu = linear_compress(x1, w1, cu, ks, st, pe1)
    xf, wf, pef = (t.float().requires_grad_() for t in (x, w, pe))
    want, want_cu = oracle.linear_compress(xf, wf, cu, ks, st, pef)
    assert torch.equal(ycu.cpu(), want_cu.cpu()) and y.dtype == dtype
    # |y| reaches ~5 here: half an ulp of a bf16 output at that magnitude is already 1.6e-2, so the
    # bound scales with the largest reference magnitude
    assert_close(y, want, "y", rel_to=want.abs().max().item())
    dy = torch.randn(y.shape, generator=g, device=device).to(dtype)
    y.backward(dy)
    want.backward(dy.float())
    assert_close(x1.grad, xf.grad, "dx", rel_to=xf.grad.abs().max().item())
    assert_close(w1.grad, wf.grad, "dw", rel_to=wf.grad.abs().max().item())
    assert_close(pe1.grad, pef.grad, "dpe", rel_to=pef.grad.abs().max().item())
    # reproducible: no atomics anywhere in the backward
    x2, w2 = x.clone().requires_grad_(), w.clone().requires_grad_()
    y2, _ = linear_compress(x2, w2, cu, ks, st)
    y2.backward(dy)
    x3, w3 = x.clone().requires_grad_(), w.clone().requires_grad_()
    y3, _ = linear_compress(x3, w3, cu, ks, st)
    y3.backward(dy)
    assert torch.equal(x2.grad, x3.grad) and torch.equal(w2.grad, w3.grad)
