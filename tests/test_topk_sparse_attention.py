"""GPU parity of topk_sparse_attention (through the C ABI) against the oracle."""
import pytest
import torch

import oracle
from helpers import assert_close
from native_sparse_attention.ops import topk_sparse_attention
from native_sparse_attention.testing import cu_from_lens, make_topk_idx

pytestmark = pytest.mark.gpu

CASES = [
    # lens, Hq, Hkv, d, block, topk, dtype, local_blocks
    ([512, 1024, 512], 16, 1, 64, 64, 8, torch.bfloat16, 1),          # shape of the reference's CPU-runnable test
    ([1000, 2000, 4096], 64, 8, 96, 64, 5, torch.float16, 1),         # the reference's own test shape
    ([2048], 64, 4, 128, 64, 16, torch.bfloat16, 2),                  # sweep shape, small N
    ([4096], 64, 4, 128, 64, 8, torch.bfloat16, 2),
    ([12, 576, 130, 1], 8, 2, 128, 32, 4, torch.bfloat16, 2),         # ragged, sequences shorter than a block
    ([700, 300], 6, 2, 64, 128, 3, torch.bfloat16, 1),                # G=3, big blocks
    ([300, 900], 32, 1, 32, 256, 2, torch.float16, 1),                # G=32: two head tiles per token
]


def _make(lens, Hq, Hkv, d, dtype, device, seed=0):
    g = torch.Generator(device=device).manual_seed(seed)
    cu = cu_from_lens(lens, device)
    T = int(cu[-1])
    q = torch.randn(T, Hq, d, generator=g, device=device).to(dtype)
    k = torch.randn(T, Hkv, d, generator=g, device=device).to(dtype)
    v = torch.randn(T, Hkv, d, generator=g, device=device).to(dtype)
    return q, k, v, cu


@pytest.mark.parametrize("lens,Hq,Hkv,d,bs,topk,dtype,local", CASES)
def test_forward_matches_oracle(device, lens, Hq, Hkv, d, bs, topk, dtype, local):
    print("case", lens, Hq, Hkv, d, bs, topk, dtype, flush=True)
    q, k, v, cu = _make(lens, Hq, Hkv, d, dtype, device)
    idx = make_topk_idx(cu, bs, topk, Hkv, seed=1, local_blocks=local)
    o = topk_sparse_attention(q, k, v, idx, bs, cu)
    torch.cuda.synchronize()
    want = oracle.topk_sparse_attention(q.float(), k.float(), v.float(), idx, bs, cu)
    assert o.dtype == dtype and o.shape == q.shape
    assert_close(o, want, "o")


def test_forward_strided_views_and_scale(device):
    lens, Hq, Hkv, d, bs, topk = [333, 800], 16, 2, 128, 64, 6
    cu = cu_from_lens(lens, device)
    T = int(cu[-1])
    g = torch.Generator(device=device).manual_seed(5)
    qkv = torch.randn(T, Hq + 2 * Hkv, d, generator=g, device=device).to(torch.bfloat16)
    q, k, v = qkv[:, :Hq], qkv[:, Hq:Hq + Hkv], qkv[:, Hq + Hkv:]
    idx_full = make_topk_idx(cu, bs, topk + 2, Hkv, seed=2)
    idx = idx_full.permute(1, 0, 2).contiguous().permute(1, 0, 2)      # non-standard strides
    o = topk_sparse_attention(q, k, v, idx, bs, cu, softmax_scale=0.05)
    want = oracle.topk_sparse_attention(q.float(), k.float(), v.float(), idx, bs, cu, softmax_scale=0.05)
    assert_close(o, want, "o")


def test_rejects_bad_dtypes(device):
    q = torch.randn(64, 4, 64, device=device)
    cu = cu_from_lens([64], device)
    idx = make_topk_idx(cu, 64, 1, 1)
    with pytest.raises(AssertionError):
        topk_sparse_attention(q, q[:, :1], q[:, :1], idx, 64, cu)             # fp32 not accepted
    qb = q.bfloat16()
    with pytest.raises(AssertionError):
        topk_sparse_attention(qb, qb[:, :1], qb[:, :1], idx.long(), 64, cu)   # idx must be int32
    with pytest.raises(AssertionError):
        topk_sparse_attention(qb, qb[:, :1], qb[:, :1], idx, 48, cu)          # block size set


def _grad_check(device, lens, Hq, Hkv, d, bs, topk, dtype, local, seed=0):
    q, k, v, cu = _make(lens, Hq, Hkv, d, dtype, device, seed)
    idx = make_topk_idx(cu, bs, topk, Hkv, seed=1, local_blocks=local)
    g = torch.Generator(device=device).manual_seed(9)
    do = torch.randn(q.shape, generator=g, device=device).to(dtype)
    q1, k1, v1 = (x.clone().requires_grad_() for x in (q, k, v))
    o = topk_sparse_attention(q1, k1, v1, idx, bs, cu)
    o.backward(do)
    qf, kf, vf = (x.float().requires_grad_() for x in (q, k, v))
    want = oracle.topk_sparse_attention(qf, kf, vf, idx, bs, cu)
    want.backward(do.float())
    # gradients of early keys sum over thousands of queries: bound errors relative to the
    # largest reference magnitude when that exceeds 1 (bf16 output rounding alone is 2^-9 relative)
    for name, got, ref in (("dq", q1.grad, qf.grad), ("dk", k1.grad, kf.grad), ("dv", v1.grad, vf.grad)):
        assert_close(got, ref, name, rel_to=ref.abs().max().item())


@pytest.mark.parametrize("lens,Hq,Hkv,d,bs,topk,dtype,local", CASES)
def test_backward_matches_oracle(device, lens, Hq, Hkv, d, bs, topk, dtype, local):
    print("case", lens, Hq, Hkv, d, bs, topk, dtype, flush=True)
    _grad_check(device, lens, Hq, Hkv, d, bs, topk, dtype, local)


@pytest.mark.parametrize("schedule", [8, 16])   # NSA_*_SCHEDULE_PLAIN / _PACED
def test_repeated_block_ids_count_once(device, schedule):
    """A row that lists a block twice attends to it once (the ids of a row are a set, as in the oracle's mask), in the
    forward, dQ, dK and dV alike."""
    from native_sparse_attention.ops.topk_sparse_attention import _topk_sparse_attention_bwd, _topk_sparse_attention_fwd

    lens, Hq, Hkv, d, bs, topk = [900, 1300], 16, 2, 64, 64, 6
    q, k, v, cu = _make(lens, Hq, Hkv, d, torch.bfloat16, device, seed=3)
    idx = make_topk_idx(cu, bs, topk, Hkv, seed=7)
    rep = idx.clone()
    rows = (idx[..., 3] >= 0)                       # rows with at least four valid entries
    rep[..., 2] = torch.where(rows, idx[..., 1], idx[..., 2])   # entry 2 repeats entry 1 (block idx[..., 2] is dropped)
    rep[..., 4] = torch.where(rows & (idx[..., 4] >= 0), idx[..., 0], idx[..., 4])   # a repeat that is not adjacent
    assert int((rep != idx).sum()) > 1000
    g = torch.Generator(device=device).manual_seed(11)
    do = torch.randn(q.shape, generator=g, device=device).to(q.dtype)
    n, sm = max(lens), d ** -0.5
    o, lse = _topk_sparse_attention_fwd(q, k, v, rep, bs, cu, cu, n, n, sm, phases=3 | schedule)
    dq, dk, dv = _topk_sparse_attention_bwd(o, do, lse, q, k, v, rep, bs, cu, cu, n, n, sm, phases=7 | schedule)
    qf, kf, vf = (x.float().requires_grad_() for x in (q, k, v))
    want = oracle.topk_sparse_attention(qf, kf, vf, rep, bs, cu)
    want.backward(do.float())
    assert_close(o, want, "o")
    for name, got, ref in (("dq", dq, qf.grad), ("dk", dk, kf.grad), ("dv", dv, vf.grad)):
        assert_close(got, ref, name, rel_to=ref.abs().max().item())


@pytest.mark.parametrize("schedule", [8, 16])   # NSA_*_SCHEDULE_PLAIN / _PACED
def test_rows_that_select_nothing(device, schedule):
    """Tokens whose row holds no block they may see (all -1, or only blocks after their own) get a zero output, lse = -inf
    and zero gradients, and change nothing for the other tokens.  (The reference's generator always lists block 0; its
    kernel divides 0 by 0 for such a row.)"""
    from native_sparse_attention.ops.topk_sparse_attention import _topk_sparse_attention_bwd, _topk_sparse_attention_fwd

    lens, Hq, Hkv, d, bs, topk = [1100, 700], 16, 2, 128, 64, 5
    q, k, v, cu = _make(lens, Hq, Hkv, d, torch.bfloat16, device, seed=5)
    idx = make_topk_idx(cu, bs, topk, Hkv, seed=9)
    T = q.shape[0]
    g = torch.Generator(device=device).manual_seed(12)
    do = torch.randn(q.shape, generator=g, device=device).to(q.dtype)
    empty = torch.zeros(Hkv, T, dtype=torch.bool, device=device)
    empty[0, 5::7] = True
    empty[1, 3::11] = True
    empty[:, :3] = True
    gone = idx.clone()
    gone[empty] = -1
    gone[0, 12::14] = 10_000                       # blocks far after the token's own: skipped like -1
    empty[0, 12::14] = True
    n, sm = max(lens), d ** -0.5
    o, lse = _topk_sparse_attention_fwd(q, k, v, gone, bs, cu, cu, n, n, sm, phases=3 | schedule)
    dq, dk, dv = _topk_sparse_attention_bwd(o, do, lse, q, k, v, gone, bs, cu, cu, n, n, sm, phases=7 | schedule)
    torch.cuda.synchronize()
    rows = empty.repeat_interleave(Hq // Hkv, 0)   # [Hq, T]
    assert (o.transpose(0, 1)[rows] == 0).all() and (dq.transpose(0, 1)[rows] == 0).all()
    assert (lse[rows] == float("-inf")).all()
    for x in (o, dq, dk, dv):
        assert torch.isfinite(x.float()).all()
    # the other tokens: the oracle on the original ids, with the emptied rows' dO zeroed so that they add nothing to dK / dV
    do_ref = do.float().clone()
    do_ref.transpose(0, 1)[rows] = 0
    qf, kf, vf = (x.float().requires_grad_() for x in (q, k, v))
    want = oracle.topk_sparse_attention(qf, kf, vf, idx, bs, cu)
    want.backward(do_ref)
    keep = ~rows
    assert_close(o.transpose(0, 1)[keep], want.detach().transpose(0, 1)[keep], "o of the other rows")
    assert_close(dq.transpose(0, 1)[keep], qf.grad.transpose(0, 1)[keep], "dq of the other rows", rel_to=qf.grad.abs().max().item())
    assert_close(dk, kf.grad, "dk", rel_to=kf.grad.abs().max().item())
    assert_close(dv, vf.grad, "dv", rel_to=vf.grad.abs().max().item())


def _expand_to_pieces(idx, cu, bs, piece):
    """Ids of the `piece`-key pieces of the selected bs-key blocks that start at or before each token (-1 elsewhere)."""
    sub = bs // piece
    pos = torch.cat([torch.arange(int(b - a)) for a, b in zip(cu[:-1].tolist(), cu[1:].tolist())]).to(idx.device)
    ids = idx[..., None].long() * sub + torch.arange(sub, device=idx.device)
    ok = (idx[..., None] >= 0) & (idx[..., None] <= (pos // bs)[None, :, None, None]) & (ids * piece <= pos[None, :, None, None])
    return torch.where(ok, ids, torch.full_like(ids, -1)).flatten(2).to(torch.int32)


@pytest.mark.parametrize("lens,Hkv,bs,topk", [
    ([700, 64, 1500], 2, 64, 6),
    ([300, 5, 900, 257], 2, 256, 3),        # 256-key blocks are indexed as four 64-key pieces
    ([70000, 100], 1, 32, 4),               # more blocks than the counting sort keeps in LDS at a time (two sweeps)
    ([1], 3, 128, 2),
    ([2500, 333], 1, 32, 20),               # more entries per token than the sort loads at a time
])
def test_reverse_index_bit_exact_and_deterministic(device, lens, Hkv, bs, topk):
    from native_sparse_attention.ops.topk_sparse_attention import _topk_sparse_attention_bwd, _topk_sparse_attention_fwd
    Hq, d = 4 * Hkv, 64
    q, k, v, cu = _make(lens, Hq, Hkv, d, torch.bfloat16, device)
    idx = make_topk_idx(cu, bs, topk, Hkv, seed=4)
    o, lse = _topk_sparse_attention_fwd(q, k, v, idx, bs, cu, cu, None, None, d ** -0.5)
    do = torch.randn_like(o)
    dq, dk, dv, seg_off, queries = _topk_sparse_attention_bwd(
        o, do, lse, q, k, v, idx, bs, cu, cu, None, None, d ** -0.5, return_reverse_index=True)
    ebs = 64 if bs == 256 else bs
    want_idx = _expand_to_pieces(idx, cu, bs, ebs) if ebs != bs else idx
    cu_blk, offs, qs = oracle.build_reverse_index(want_idx.cpu().numpy(), cu.cpu().numpy(), ebs)
    T, B = int(cu[-1]), len(lens)
    max_blocks = T // ebs + B
    seg_off, queries = seg_off.cpu().numpy(), queries.cpu().numpy()
    total_blocks = int(cu_blk[-1])
    for h in range(Hkv):
        for g in range(total_blocks):
            s = h * max_blocks + g
            assert seg_off[s + 1] - seg_off[s] == offs[h, g + 1] - offs[h, g], (h, g)
            assert (queries[seg_off[s]:seg_off[s + 1]] == qs[h, offs[h, g]:offs[h, g + 1]]).all(), (h, g)
        for g in range(total_blocks, max_blocks):                      # unused segments are empty
            s = h * max_blocks + g
            assert seg_off[s] == seg_off[s + 1]
    dq2, dk2, dv2 = _topk_sparse_attention_bwd(o, do, lse, q, k, v, idx, bs, cu, cu, None, None, d ** -0.5)
    assert torch.equal(dq, dq2) and torch.equal(dk, dk2) and torch.equal(dv, dv2)


@pytest.mark.parametrize("schedule", [8, 16])   # NSA_*_SCHEDULE_PLAIN / _PACED: one wave per token / persistent paced waves
def test_forward_backward_replayed_from_a_hip_graph(device, schedule):
    """Forward + backward recorded once into a HIP graph (nothing in them allocates, synchronises or clears memory with
    a memset; the paced schedule's table is reset by a kernel of the launch itself) and replayed on fresh inputs, with
    eager work and synchronisation between the replays: every replay must equal the eager result bit for bit."""
    from native_sparse_attention.ops.topk_sparse_attention import _topk_sparse_attention_bwd, _topk_sparse_attention_fwd
    lens, Hq, Hkv, d, bs, topk = [900, 130, 2000], 32, 2, 128, 64, 8
    q, k, v, cu = _make(lens, Hq, Hkv, d, torch.bfloat16, device)
    T = int(cu[-1])
    idx = make_topk_idx(cu, bs, topk, Hkv, seed=1)
    do = torch.randn_like(q)
    sm = d ** -0.5

    def step():
        o, lse = _topk_sparse_attention_fwd(q, k, v, idx, bs, cu, cu, None, None, sm, phases=3 | schedule)
        return (o,) + tuple(_topk_sparse_attention_bwd(o, do, lse, q, k, v, idx, bs, cu, cu, None, None, sm, phases=7 | schedule))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                                   # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    g = torch.Generator(device=device).manual_seed(9)
    for r in range(4):
        for x in (q, k, v, do):
            x.copy_(torch.randn(x.shape, generator=g, device=device).to(x.dtype))
        idx.copy_(make_topk_idx(cu, bs, topk, Hkv, seed=10 + r))
        graph.replay()
        torch.cuda.synchronize()
        got = [x.clone() for x in outs]
        want = step()
        torch.cuda.synchronize()
        for name, a, b in zip(("o", "dq", "dk", "dv"), got, want):
            assert torch.equal(a, b), (name, r)


@pytest.mark.parametrize("scale", [-0.2, 0.0, 3.0])
def test_any_finite_softmax_scale(device, scale):
    """The reference accepts any softmax scale (ops/triton/topk_sparse_attention.py:1133-1134 only fills in a default)."""
    lens, Hq, Hkv, d, bs, topk = [300, 77], 16, 2, 64, 64, 4
    q, k, v, cu = _make(lens, Hq, Hkv, d, torch.bfloat16, device)
    q, k = (q.float() * 0.5).bfloat16(), (k.float() * 0.5).bfloat16()
    idx = make_topk_idx(cu, bs, topk, Hkv, seed=2)
    q1, k1, v1 = (x.clone().requires_grad_() for x in (q, k, v))
    o = topk_sparse_attention(q1, k1, v1, idx, bs, cu, scale)
    qf, kf, vf = (x.float().requires_grad_() for x in (q, k, v))
    want = oracle.topk_sparse_attention(qf, kf, vf, idx, bs, cu, scale)
    assert_close(o, want, "o")
    do = torch.randn_like(o)
    o.backward(do)
    want.backward(do.float())
    # At scale 3 the softmax is nearly one-hot and dS = scale * P * (dP - delta) is a difference of nearly equal numbers
    # times 3: delta is formed from the 16-bit O (as the reference's backward_sum_o_do does, topk_sparse_attention.py:177-217),
    # whose rounding (2^-9 of |o| per element, summed over d with |dO| ~ 1) alone moves dS by ~0.1.  That case is a test of
    # "any finite scale runs and stays close", with the bounds scaled by the largest gradient; the others use row scales.
    for name, a, b in (("dq", q1.grad, qf.grad), ("dk", k1.grad, kf.grad), ("dv", v1.grad, vf.grad)):
        if scale == 3.0:
            s_ = max(1.0, b.abs().max().item())
            assert_close(a, b, name, max_abs=2e-2 * s_, mean_abs=2e-3 * s_)
        else:
            assert_close(a, b, name, rel_to=True)
