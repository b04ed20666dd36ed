"""The two schedules of the query-stationary kernels (one wave per token in launch order / persistent waves with paced
key positions) must give bit-identical results, and the paced one must match the oracle on shapes small enough to check
in full: ragged varlen batches, more than 16 heads per group, every block size, rows longer than 64 entries, sequences
shorter than one sweep."""
import pytest
import torch

import oracle
from helpers import assert_close
from native_sparse_attention.ops.topk_sparse_attention import _topk_sparse_attention_bwd, _topk_sparse_attention_fwd
from native_sparse_attention.testing import cu_from_lens, make_topk_idx

pytestmark = pytest.mark.gpu

PLAIN, PACED = 8, 16   # NSA_FWD_SCHEDULE_* / NSA_BWD_SCHEDULE_* of include/nsa_hip.h

CASES = [
    # lens, Hq, Hkv, d, block, topk, dtype
    ([3000, 5000, 1200], 64, 4, 128, 64, 16, torch.bfloat16),     # several sweeps per kv-head, sweeps that straddle sequences
    ([12, 576, 130, 1, 2100], 8, 2, 128, 32, 4, torch.bfloat16),  # sequences shorter than a block and than a sweep
    ([700, 300, 2500], 6, 2, 64, 128, 3, torch.bfloat16),         # G=3, 128-key blocks
    ([300, 900, 1500], 32, 1, 32, 256, 2, torch.float16),         # G=32: two head tiles per token, 256-key blocks
    ([1000, 2000, 4096], 64, 8, 96, 64, 5, torch.float16),        # the reference's own test shape
    ([6000], 16, 1, 64, 32, 70, torch.bfloat16),                  # rows of more than 64 entries
    ([100], 16, 2, 128, 64, 2, torch.bfloat16),                   # fewer tokens than resident waves
]


def _inputs(lens, Hq, Hkv, d, dtype, device):
    g = torch.Generator(device=device).manual_seed(3)
    cu = cu_from_lens(lens, device)
    T = int(cu[-1])
    q = torch.randn(T, Hq, d, generator=g, device=device).to(dtype)
    k = torch.randn(T, Hkv, d, generator=g, device=device).to(dtype)
    v = torch.randn(T, Hkv, d, generator=g, device=device).to(dtype)
    do = torch.randn(T, Hq, d, generator=g, device=device).to(dtype)
    return q, k, v, do, cu


@pytest.mark.parametrize("lens,Hq,Hkv,d,bs,topk,dtype", CASES)
def test_paced_equals_plain_and_oracle(device, lens, Hq, Hkv, d, bs, topk, dtype):
    print("case", lens, Hq, Hkv, d, bs, topk, dtype, flush=True)
    q, k, v, do, cu = _inputs(lens, Hq, Hkv, d, dtype, device)
    idx = make_topk_idx(cu, bs, topk, Hkv, seed=4)
    n = max(lens)
    sm = d ** -0.5
    o_plain, lse_plain = _topk_sparse_attention_fwd(q, k, v, idx, bs, cu, cu, n, n, sm, phases=3 | PLAIN)
    o_paced, lse_paced = _topk_sparse_attention_fwd(q, k, v, idx, bs, cu, cu, n, n, sm, phases=3 | PACED)
    torch.cuda.synchronize()
    assert torch.equal(o_plain, o_paced), "o differs between the schedules"
    assert torch.equal(lse_plain, lse_paced), "lse differs between the schedules"
    qf, kf, vf = (x.float().requires_grad_() for x in (q, k, v))
    want = oracle.topk_sparse_attention(qf, kf, vf, idx, bs, cu)
    assert_close(o_paced, want, "o (paced)")
    g_plain = _topk_sparse_attention_bwd(o_plain, do, lse_plain, q, k, v, idx, bs, cu, cu, n, n, sm, phases=7 | PLAIN)
    g_paced = _topk_sparse_attention_bwd(o_plain, do, lse_plain, q, k, v, idx, bs, cu, cu, n, n, sm, phases=7 | PACED)
    torch.cuda.synchronize()
    for name, a, b in zip(("dq", "dk", "dv"), g_plain, g_paced):
        assert torch.equal(a, b), name + " differs between the schedules"
    want.backward(do.float())
    assert_close(g_paced[0], qf.grad, "dq (paced)", rel_to=qf.grad.abs().max().item())


def test_paced_negative_and_zero_scale(device):
    q, k, v, do, cu = _inputs([1500, 700], 16, 2, 64, torch.bfloat16, device)
    idx = make_topk_idx(cu, 64, 6, 2, seed=5)
    for sm in (-0.2, 0.0):
        a = _topk_sparse_attention_fwd(q, k, v, idx, 64, cu, cu, 1500, 1500, sm, phases=3 | PLAIN)
        b = _topk_sparse_attention_fwd(q, k, v, idx, 64, cu, cu, 1500, 1500, sm, phases=3 | PACED)
        torch.cuda.synchronize()
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1]), sm
        want = oracle.topk_sparse_attention(q.float(), k.float(), v.float(), idx, 64, cu, softmax_scale=sm)
        assert_close(b[0], want, "o at scale %g" % sm)


def test_passes_one_call_at_a_time(device):
    """The backward's passes run as separate calls on a kept workspace: preparation alone forms delta and the per-token
    (lse, delta) pairs in a pass of its own (a different summation order from the one inside the dQ pass, so the last
    bits of delta may differ from the single call's); dK/dV before or after dQ gives identical results."""
    from native_sparse_attention import _lib
    lens, Hq, Hkv, d, bs, topk = [900, 2300, 70], 32, 2, 128, 64, 8
    q, k, v, do, cu = _inputs(lens, Hq, Hkv, d, torch.bfloat16, device)
    idx = make_topk_idx(cu, bs, topk, Hkv, seed=6)
    n, sm = max(lens), d ** -0.5
    o, lse = _topk_sparse_attention_fwd(q, k, v, idx, bs, cu, cu, n, n, sm)
    want = _topk_sparse_attention_bwd(o, do, lse, q, k, v, idx, bs, cu, cu, n, n, sm)
    lib = _lib.load()
    got = []
    for order in ((1, 4, 2), (1, 2, 4)):
        ws = _lib.workspace(lib.nsa_topk_attn_bwd_workspace_bytes(sum(lens), len(lens), Hq, Hkv, d, topk, bs), device)
        ws.fill_(0x7f)   # nothing may be read before a pass has written it
        out = tuple(torch.full_like(x, float("nan")) for x in want)
        for phase in order:
            _topk_sparse_attention_bwd(o, do, lse, q, k, v, idx, bs, cu, cu, n, n, sm, workspace=ws, phases=phase, out=out)
        torch.cuda.synchronize()
        got.append(out)
    for name, a, b, c in zip(("dq", "dk", "dv"), want, got[0], got[1]):
        assert torch.equal(b, c), name + " depends on the order of the passes"
        assert_close(b, a.float(), name + " (separate passes)", rel_to=True)
