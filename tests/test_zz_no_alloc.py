"""nsa_topk_decode_static (split-K partials in the library's own device array, no workspace argument) against
nsa_topk_decode on the same inputs, through the C ABI: two calls in a row, the second on a smaller input, so that
what the first call left in the shared array must not leak into the second.  Results are bit-identical (the same
kernels run either way).  Oversized requests are refused without a launch."""
import pytest
import torch

from native_sparse_attention import _lib
from native_sparse_attention.ops.decode import _strides, topk_sparse_attention_decode
from native_sparse_attention.testing import cu_from_lens, make_topk_idx

pytestmark = pytest.mark.gpu


def _case(B, max_len, Hq, Hkv, d, bs, topk, dtype, device, seed):
    g = torch.Generator(device=device).manual_seed(seed)
    q = torch.empty(B, Hq, d, device=device).uniform_(-1, 1, generator=g).to(dtype)
    cache = torch.empty(2, B, max_len, Hkv, d, device=device).uniform_(-1, 1, generator=g).to(dtype)
    lens = torch.randint(max_len // 2, max_len + 1, (B,), generator=g, device=device).to(torch.int32)
    rows = []
    for b, L in enumerate(lens.tolist()):
        rows.append(make_topk_idx(cu_from_lens([L], device), bs, topk, Hkv, seed=seed + b)[:, L - 1])
    idx = torch.stack(rows, 1).contiguous()
    return q, cache[0], cache[1], idx, lens


def _static(q, k, v, idx, bs, lens):
    B, Hq, d = q.shape
    Hkv, L, topk = k.shape[2], k.shape[1], idx.shape[-1]
    o = torch.empty_like(q)
    rc = _lib.load().nsa_topk_decode_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), idx.data_ptr(), lens.data_ptr(), o.data_ptr(),
                                            B, Hq, Hkv, d, L, topk, bs, _strides(q, k, v, o, idx), d ** -0.5, _lib.dtype_code(q),
                                            _lib.stream_ptr(q))
    return rc, o


def test_static_scratch_decode_equals_workspace_decode(device):
    big = _case(8, 4096, 32, 2, 128, 64, 16, torch.bfloat16, device, seed=3)
    small = _case(3, 700, 16, 2, 128, 64, 4, torch.bfloat16, device, seed=4)
    for q, k, v, idx, lens in (big, small, big):
        rc, o = _static(q, k, v, idx, 64, lens)
        assert rc == 0
        want = topk_sparse_attention_decode(q, k, v, idx, 64, lens)
        torch.cuda.synchronize()
        assert torch.equal(o, want)
        assert o.float().abs().max() > 0


def test_static_scratch_decode_allocates_nothing_and_replays_from_a_graph(device):
    q, k, v, idx, lens = _case(4, 2048, 32, 2, 128, 64, 8, torch.bfloat16, device, seed=6)
    rc, want = _static(q, k, v, idx, 64, lens)          # first use on this device happens outside any capture
    assert rc == 0
    torch.cuda.synchronize()
    o = torch.empty_like(q)
    strides = _strides(q, k, v, o, idx)
    lib = _lib.load()
    call = lambda: lib.nsa_topk_decode_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), idx.data_ptr(), lens.data_ptr(), o.data_ptr(),
                                              4, 32, 2, 128, 2048, 8, 64, strides, 128 ** -0.5, _lib.dtype_code(q), _lib.stream_ptr(q))
    # neither the caching allocator nor the driver hands out memory for a call
    free0, _ = torch.cuda.mem_get_info()
    alloc0, reserved0 = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    assert call() == 0
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == alloc0 and torch.cuda.memory_reserved() == reserved0
    assert torch.cuda.mem_get_info()[0] == free0
    assert torch.equal(o, want)
    # recorded into a graph and replayed, with eager work and synchronisations between the replays
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = call()
    assert rc == 0
    for r in range(3):
        o.zero_()
        q.mul_(-1)                                       # other inputs each time: the graph reads the buffers, not a snapshot
        graph.replay()
        torch.cuda.synchronize()
        want = topk_sparse_attention_decode(q, k, v, idx, 64, lens)
        torch.cuda.synchronize()
        assert torch.equal(o, want), r


def test_static_scratch_decode_rejects_sizes_beyond_its_array(device):
    lib = _lib.load()
    B, Hq, Hkv, d, topk = 64, 64, 4, 128, 64
    assert lib.nsa_topk_decode_workspace_bytes(B, Hq, Hkv, d, topk, 64) > (4 << 20)
    q, k, v, idx, lens = _case(2, 256, 16, 1, 128, 64, 2, torch.bfloat16, device, seed=5)
    o = torch.empty_like(q)
    rc = lib.nsa_topk_decode_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), idx.data_ptr(), lens.data_ptr(), o.data_ptr(),
                                    B, Hq, Hkv, d, 256, topk, 64, _strides(q, k, v, o, idx), d ** -0.5, 0, _lib.stream_ptr(q))
    assert rc == -3
