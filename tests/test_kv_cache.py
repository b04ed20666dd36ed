"""NSACache (HIP slab kernels) against a tensor-op restatement of the reference's update rules
(native_sparse_attention/module/kv_cache.py:233-302 prepare_compress, :340-449 update_kv): lengths and
every valid slab row must be bit-identical after the prefill and after each decode step."""
from typing import Union

import pytest
import torch

from native_sparse_attention.module import NSACache
from native_sparse_attention.testing import cu_from_lens

pytestmark = pytest.mark.gpu


def _compressed_seqlens(cu_seqlens, kernel_size, kernel_stride):
    seqlens = cu_seqlens[1:] - cu_seqlens[:-1]
    y = torch.div(seqlens - kernel_size, kernel_stride, rounding_mode="floor").to(torch.int32) + 1
    y = torch.where(seqlens < kernel_size, torch.zeros_like(y), y)
    cu = torch.zeros(y.shape[0] + 1, dtype=torch.int32, device=cu_seqlens.device)
    cu[1:] = torch.cumsum(y, dim=0)
    return y, cu


def _fill_slab(slab: torch.Tensor, key: torch.Tensor, value: torch.Tensor, seq_start: torch.Tensor, seq_end: torch.Tensor):
    """slab[0 or 1, b, :seq_end[b]-seq_start[b]] = key or value[seq_start[b]:seq_end[b]] for every sequence."""
    starts, ends = seq_start.tolist(), seq_end.tolist()
    for b, (s, e) in enumerate(zip(starts, ends)):
        if e > s:
            slab[0, b, : e - s] = key[s:e]
            slab[1, b, : e - s] = value[s:e]


class TorchNSACache:
    def __init__(self, max_batch_size: int, max_length: int, num_kv_heads: int, head_dim: int, kernel_size: int,
                 kernel_stride: int, window_size: int, dtype: torch.dtype, device: Union[str, torch.device] = "cuda"):
        self.max_batch_size, self.max_length = max_batch_size, max_length
        self.num_kv_heads, self.head_dim = num_kv_heads, head_dim
        self.kernel_size, self.kernel_stride, self.window_size = kernel_size, kernel_stride, window_size
        self.dtype, self.device = dtype, device
        self.max_comp_length = (max_length - kernel_size) // kernel_stride + 1

        def slab(rows):
            return torch.zeros(2, max_batch_size, rows, num_kv_heads, head_dim, dtype=dtype, device=device)

        def lens():
            return torch.zeros(max_batch_size, dtype=torch.int32, device=device)

        self.sparse_kv_cache, self.sparse_kv_len = slab(max_length), lens()
        self.compress_kv_cache, self.compress_kv_len = slab(self.max_comp_length), lens()
        self.before_compress_kv_cache, self.before_compress_kv_len = slab(kernel_size), lens()
        self.sliding_kv_cache, self.sliding_kv_len = slab(window_size), lens()

    def reset(self):
        for t in (self.sparse_kv_cache, self.sparse_kv_len, self.compress_kv_cache, self.compress_kv_len,
                  self.before_compress_kv_cache, self.before_compress_kv_len, self.sliding_kv_cache, self.sliding_kv_len):
            t.zero_()

    # ---- before compression -------------------------------------------------------------------
    def prepare_compress(self, cu_seqlens: torch.Tensor, step: int, key: torch.Tensor, value: torch.Tensor):
        assert key.shape == value.shape and key.shape[1:] == (self.num_kv_heads, self.head_dim)
        if step == 0:
            batch = cu_seqlens.shape[0] - 1
            comp_seqlens, _ = _compressed_seqlens(cu_seqlens, self.kernel_size, self.kernel_stride)
            # tokens after the start of the next (incomplete) window wait in the staging slab
            seq_start = cu_seqlens[:-1] + comp_seqlens * self.kernel_stride
            seq_end = cu_seqlens[1:]
            _fill_slab(self.before_compress_kv_cache, key, value, seq_start, seq_end)
            self.before_compress_kv_len[:batch] = seq_end - seq_start
        else:
            batch = key.shape[0]
            assert batch == cu_seqlens.shape[0] - 1
            full = self.before_compress_kv_len[:batch] == self.kernel_size
            if bool(full.any()):
                idx = torch.nonzero(full).flatten()
                keep = self.kernel_size - self.kernel_stride
                self.before_compress_kv_cache[:, idx, :keep] = self.before_compress_kv_cache[:, idx, self.kernel_stride:].clone()
                self.before_compress_kv_len[idx] -= self.kernel_stride
            rows = torch.arange(batch, device=key.device)
            at = self.before_compress_kv_len[:batch].long()
            self.before_compress_kv_cache[0, rows, at] = key
            self.before_compress_kv_cache[1, rows, at] = value
            self.before_compress_kv_len[:batch] += 1

    # ---- after rope ---------------------------------------------------------------------------
    def update_kv(self, cu_seqlens, step, compress_key, compress_value, sparse_key, sparse_value, sliding_key, sliding_value):
        assert compress_key.shape == compress_value.shape and sparse_key.shape == sparse_value.shape
        assert sliding_key.shape == sliding_value.shape
        if step == 0:
            seqlens = cu_seqlens[1:] - cu_seqlens[:-1]
            batch = seqlens.shape[0]
            comp_seqlens, comp_cu = _compressed_seqlens(cu_seqlens, self.kernel_size, self.kernel_stride)
            _fill_slab(self.compress_kv_cache, compress_key, compress_value, comp_cu[:-1], comp_cu[1:])
            self.compress_kv_len[:batch] = comp_seqlens
            _fill_slab(self.sparse_kv_cache, sparse_key, sparse_value, cu_seqlens[:-1], cu_seqlens[1:])
            self.sparse_kv_len[:batch] = seqlens
            # the last window_size tokens, stored from row 0 (the decode kernel reads the ring as a set)
            start = torch.maximum(cu_seqlens[1:] - self.window_size, cu_seqlens[:-1])
            _fill_slab(self.sliding_kv_cache, sliding_key, sliding_value, start, cu_seqlens[1:])
            self.sliding_kv_len[:batch] = cu_seqlens[1:] - start
        else:
            batch = sparse_key.shape[0]
            full = self.before_compress_kv_len[:batch] == self.kernel_size
            if bool(full.any()):
                idx = torch.nonzero(full).flatten()
                at = self.compress_kv_len[idx].long()
                self.compress_kv_cache[0, idx, at] = compress_key[idx]
                self.compress_kv_cache[1, idx, at] = compress_value[idx]
                self.compress_kv_len[idx] += 1
            rows = torch.arange(batch, device=sparse_key.device)
            at = self.sparse_kv_len[:batch].long()
            self.sparse_kv_cache[0, rows, at] = sparse_key
            self.sparse_kv_cache[1, rows, at] = sparse_value
            self.sparse_kv_len[:batch] += 1
            ring = (self.sliding_kv_len[:batch] % self.window_size).long()
            self.sliding_kv_cache[0, rows, ring] = sliding_key
            self.sliding_kv_cache[1, rows, ring] = sliding_value
            self.sliding_kv_len[:batch] += 1


def _same(a: NSACache, b: TorchNSACache, batch, ring_as_set_at_prefill=False):
    for slab, ln in (("sparse_kv_cache", "sparse_kv_len"), ("compress_kv_cache", "compress_kv_len"),
                     ("before_compress_kv_cache", "before_compress_kv_len"), ("sliding_kv_cache", "sliding_kv_len")):
        la, lb = getattr(a, ln)[:batch], getattr(b, ln)[:batch]
        assert torch.equal(la, lb), ln
        sa, sb = getattr(a, slab), getattr(b, slab)
        rows = sa.shape[2]
        for i, n in enumerate(lb.tolist()):
            n = min(n, rows)
            assert torch.equal(sa[:, i, :n], sb[:, i, :n]), (slab, i)


@pytest.mark.parametrize("lens,steps,ks,st,window", [
    ([130, 47, 300, 31], 40, 32, 16, 64),      # staging windows fill and shift, the ring wraps
    ([12, 576], 20, 32, 32, 512),              # stride == kernel size: the staging window empties completely
    ([1000], 70, 64, 16, 128),
])
def test_prefill_and_decode_updates(device, lens, steps, ks, st, window):
    H, d, B = 2, 64, len(lens)
    g = torch.Generator(device=device).manual_seed(0)
    cu = cu_from_lens(lens, device)
    T = int(cu[-1])
    mine = NSACache(B + 1, max(lens) + steps + 4, H, d, ks, st, window, torch.bfloat16, device)
    ref = TorchNSACache(B + 1, max(lens) + steps + 4, H, d, ks, st, window, torch.bfloat16, device)

    def rnd(*shape):
        return torch.randn(*shape, generator=g, device=device).bfloat16()

    k, v = rnd(T, H, d), rnd(T, H, d)
    _, comp_cu = _compressed_seqlens(cu, ks, st)
    ck, cv = rnd(int(comp_cu[-1]), H, d), rnd(int(comp_cu[-1]), H, d)
    for c in (mine, ref):
        c.reset()
        c.prepare_compress(cu, 0, k, v)
        c.update_kv(cu, 0, ck, cv, k, v, k, v)
    _same(mine, ref, B)
    assert mine.max_seqlen(0) == max(lens)
    for step in range(1, steps + 1):
        # strided views, as the projections of a layer produce them
        kv = rnd(B, 2, H, d)
        k1, v1 = kv[:, 0], kv[:, 1]
        ck1, cv1, sk1, sv1 = rnd(B, H, d), rnd(B, H, d), rnd(B, H, d), rnd(B, H, d)
        for c in (mine, ref):
            c.prepare_compress(cu, step, k1, v1)
        _same(mine, ref, B)
        for c in (mine, ref):
            c.update_kv(cu, step, ck1, cv1, k1, v1, sk1, sv1)
        _same(mine, ref, B)


def test_plain_kv_cache_prefill_and_decode(device):
    """KVCache (dense baseline) against slice assignments: a prefill, three appended tokens, then a reset and a new prefill."""
    from native_sparse_attention.module import KVCache
    Hkv, d, maxB, maxL = 2, 64, 4, 300
    cache = KVCache(maxB, maxL, Hkv, d, torch.bfloat16, device)
    g = torch.Generator(device=device).manual_seed(3)
    for lens in ([100, 1, 257], [40, 33]):
        cu = cu_from_lens(lens, device)
        B = len(lens)
        want = torch.zeros(2, B, maxL, Hkv, d, dtype=torch.bfloat16, device=device)
        kv = torch.randn(2, sum(lens), Hkv + 1, d, generator=g, device=device).bfloat16()
        k, v = kv[0, :, :Hkv], kv[1, :, 1:]            # strided views
        cache.reset()
        cache.update_kv(cu, 0, k, v)
        s0 = 0
        for b, L in enumerate(lens):
            want[0, b, :L], want[1, b, :L] = k[s0:s0 + L], v[s0:s0 + L]
            s0 += L
        cur = list(lens)
        for step in range(1, 4):
            nk = torch.randn(B, Hkv, d, generator=g, device=device).bfloat16()
            nv = torch.randn(B, Hkv, d, generator=g, device=device).bfloat16()
            cache.update_kv(cu, step, nk, nv)
            for b in range(B):
                want[0, b, cur[b]], want[1, b, cur[b]] = nk[b], nv[b]
                cur[b] += 1
        assert cache.kv_len[:B].tolist() == cur
        for b in range(B):
            assert torch.equal(cache.kv_cache[:, b, :cur[b]], want[:, b, :cur[b]]), b
