"""KV-cache slabs for NSA inference, with the update rules the decode operators rely on.

Counterpart of the reference's NSACache (native_sparse_attention/module/kv_cache.py:125-449): four
slabs of shape [2 (k/v), max_batch, rows, num_kv_heads, head_dim] plus int32 length vectors:

  sparse_kv_cache          rows = max_length          every token, in order (top-k branch)
  compress_kv_cache        rows = max_comp_length     compressed tokens (compressed branch)
  before_compress_kv_cache rows = kernel_size         staging window that the next compressed token is made from
  sliding_kv_cache         rows = window_size         ring buffer, token t lives in row t % window_size

Decode-step rules (kv_cache.py:274-302, 401-449): a sequence whose staging window is full first
shifts it left by kernel_stride, then the new token is appended; after compression the candidate
compressed token is committed only for sequences whose staging window is full again; the new
token is appended to the sparse slab and written into the ring at sliding_kv_len % window_size.
"""
from typing import Union

import torch

from ..ops.utils import get_compressed_seqlens


def _fill_slab(slab: torch.Tensor, key: torch.Tensor, value: torch.Tensor, seq_start: torch.Tensor, seq_end: torch.Tensor):
    """slab[0 or 1, b, :seq_end[b]-seq_start[b]] = key or value[seq_start[b]:seq_end[b]] for every sequence."""
    starts, ends = seq_start.tolist(), seq_end.tolist()
    for b, (s, e) in enumerate(zip(starts, ends)):
        if e > s:
            slab[0, b, : e - s] = key[s:e]
            slab[1, b, : e - s] = value[s:e]


class NSACache:
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
            comp_seqlens, _ = get_compressed_seqlens(cu_seqlens, self.kernel_size, self.kernel_stride)
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
            comp_seqlens, comp_cu = get_compressed_seqlens(cu_seqlens, self.kernel_size, self.kernel_stride)
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
