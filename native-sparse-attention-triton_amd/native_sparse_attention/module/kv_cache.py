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

Every update is one HIP kernel that reads and writes the length vectors on the device, so a decode step
never waits for the host.  The only host-side figure is `max_seqlen` (longest prompt, taken once at
prefill, plus the decode step), which bounds slab views and fixes output shapes.
"""
import ctypes
from typing import Union

import torch

from .. import _lib
from ..ops.utils import get_compressed_seqlens, last_dim_contiguous


class KVCache:
    """Plain per-sequence KV cache for dense attention: slab [2, max_batch, max_length, num_kv_heads, head_dim] plus
    an int32 length per sequence (counterpart of kv_cache.py:21-122 of the reference).  Both updates are one kernel
    each and the lengths stay on the device."""

    def __init__(self, max_batch_size: int, max_length: int, num_kv_heads: int, head_dim: int, dtype: torch.dtype,
                 device: Union[str, torch.device] = "cuda"):
        assert dtype in (torch.bfloat16, torch.float16) and head_dim % 8 == 0
        self.max_batch_size, self.max_length = max_batch_size, max_length
        self.num_kv_heads, self.head_dim, self.dtype, self.device = num_kv_heads, head_dim, dtype, device
        self.kv_cache = torch.zeros(2, max_batch_size, max_length, num_kv_heads, head_dim, dtype=dtype, device=device)
        self.kv_len = torch.zeros(max_batch_size, dtype=torch.int32, device=device)

    def reset(self):
        self.kv_len.zero_()  # rows beyond a length are never read

    def update_kv(self, cu_seqlens: torch.Tensor, step: int, key: torch.Tensor, value: torch.Tensor):
        assert key.shape == value.shape and key.shape[1:] == (self.num_kv_heads, self.head_dim) and key.dtype == self.dtype
        batch = cu_seqlens.shape[0] - 1
        assert batch <= self.max_batch_size
        key, value = last_dim_contiguous(key), last_dim_contiguous(value)
        lib = _lib.load()
        if step == 0:
            cu_seqlens = cu_seqlens.to(torch.int32).contiguous()
            begin, end = cu_seqlens[:-1], cu_seqlens[1:]  # views into cu_seqlens, alive for the call
            rc = lib.nsa_cache_fill(key.data_ptr(), value.data_ptr(), cu_seqlens.data_ptr(), begin.data_ptr(),
                                    end.data_ptr(), self.kv_cache.data_ptr(), self.kv_len.data_ptr(), key.shape[0],
                                    batch, self.num_kv_heads, self.head_dim, key.stride(0), key.stride(1), value.stride(0),
                                    value.stride(1), self.max_batch_size, self.max_length, _lib.stream_ptr(key))
            _lib.check(rc, "nsa_cache_fill")
        else:
            assert key.shape[0] == batch
            rc = lib.nsa_cache_append_token(key.data_ptr(), value.data_ptr(), self.kv_cache.data_ptr(), self.kv_len.data_ptr(), batch,
                                            self.num_kv_heads, self.head_dim, key.stride(0), key.stride(1), value.stride(0),
                                            value.stride(1), self.max_batch_size, self.max_length, _lib.stream_ptr(key))
            _lib.check(rc, "nsa_cache_append_token")


class NSACache:
    def __init__(self, max_batch_size: int, max_length: int, num_kv_heads: int, head_dim: int, kernel_size: int,
                 kernel_stride: int, window_size: int, dtype: torch.dtype, device: Union[str, torch.device] = "cuda"):
        assert dtype in (torch.bfloat16, torch.float16) and head_dim % 8 == 0 and kernel_size % kernel_stride == 0
        self.max_batch_size, self.max_length = max_batch_size, max_length
        self.num_kv_heads, self.head_dim = num_kv_heads, head_dim
        self.kernel_size, self.kernel_stride, self.window_size = kernel_size, kernel_stride, window_size
        self.dtype, self.device = dtype, device
        self.max_comp_length = (max_length - kernel_size) // kernel_stride + 1
        self.max_prompt_len = 0  # host copy of the longest prompt of the current batch (set at prefill)
        self.prefill_serial = 0  # counts prefills
        self.decode_steps = 0    # tokens appended per sequence since the prefill, whoever ran the steps (host copy)
        self._staging_cu = None
        self._staging_out_cu = None
        self.static_shapes = False  # decode steps use the full slab extents instead of the current length bound

        def slab(rows):
            return torch.zeros(2, max_batch_size, rows, num_kv_heads, head_dim, dtype=dtype, device=device)

        def lens():
            return torch.zeros(max_batch_size, dtype=torch.int32, device=device)

        self.sparse_kv_cache, self.sparse_kv_len = slab(max_length), lens()
        self.compress_kv_cache, self.compress_kv_len = slab(self.max_comp_length), lens()
        self.before_compress_kv_cache, self.before_compress_kv_len = slab(kernel_size), lens()
        self.sliding_kv_cache, self.sliding_kv_len = slab(window_size), lens()

    def reset(self):
        # slab contents need no clearing: rows beyond the lengths are never read
        for t in (self.sparse_kv_len, self.compress_kv_len, self.before_compress_kv_len, self.sliding_kv_len):
            t.zero_()
        self.max_prompt_len = 0
        self.decode_steps = 0

    def count_decode_step(self):
        """Called once per decode step that appends a token to every sequence - by the eager path and by replays of a
        recorded step alike, so that steps of either kind on one cache are counted together.  Raises when the longest
        sequence would outgrow its slab (the kernels would then silently stop storing tokens)."""
        if self.max_prompt_len + self.decode_steps + 1 > self.max_length:
            raise RuntimeError("decode step %d of a %d-token prompt does not fit the cache (max_length %d)"
                               % (self.decode_steps + 1, self.max_prompt_len, self.max_length))
        self.decode_steps += 1

    def staging_cu_seqlens(self, batch: int) -> torch.Tensor:
        """cu_seqlens of the staging slab seen as a varlen batch: every sequence contributes kernel_size rows."""
        if self._staging_cu is None:
            self._staging_cu = torch.arange(self.max_batch_size + 1, dtype=torch.int32, device=self.device) * self.kernel_size
        return self._staging_cu[: batch + 1]

    def staging_out_cu_seqlens(self, batch: int) -> torch.Tensor:
        """cu_seqlens of the compressed staging slab: one output row per sequence."""
        if self._staging_out_cu is None:
            self._staging_out_cu = torch.arange(self.max_batch_size + 1, dtype=torch.int32, device=self.device)
        return self._staging_out_cu[: batch + 1]

    def max_seqlen(self, step: int) -> int:
        """Upper bound, known on the host, of every sequence's length at decode step `step`."""
        return self.max_prompt_len + step

    def _fill(self, slab, slab_len, key, value, cu_src, begin, end):
        key, value = last_dim_contiguous(key), last_dim_contiguous(value)
        batch = cu_src.shape[0] - 1
        rc = _lib.load().nsa_cache_fill(key.data_ptr(), value.data_ptr(), cu_src.data_ptr(), begin.data_ptr(), end.data_ptr(),
                                        slab.data_ptr(), slab_len.data_ptr(), key.shape[0], batch, self.num_kv_heads, self.head_dim,
                                        key.stride(0), key.stride(1), value.stride(0), value.stride(1), self.max_batch_size,
                                        slab.shape[2], _lib.stream_ptr(slab))
        _lib.check(rc, "nsa_cache_fill")

    # ---- before compression -------------------------------------------------------------------
    def prepare_compress(self, cu_seqlens: torch.Tensor, step: int, key: torch.Tensor, value: torch.Tensor):
        assert key.shape == value.shape and key.shape[1:] == (self.num_kv_heads, self.head_dim)
        assert key.dtype == self.dtype and value.dtype == self.dtype
        batch = cu_seqlens.shape[0] - 1
        assert batch <= self.max_batch_size
        if step == 0:
            comp_seqlens, _ = get_compressed_seqlens(cu_seqlens, self.kernel_size, self.kernel_stride)
            # tokens after the start of the next (incomplete) window wait in the staging slab
            begin = (cu_seqlens[:-1] + comp_seqlens * self.kernel_stride).contiguous()
            self._fill(self.before_compress_kv_cache, self.before_compress_kv_len, key, value, cu_seqlens, begin, cu_seqlens[1:].contiguous())
        else:
            assert key.shape[0] == batch
            key, value = last_dim_contiguous(key), last_dim_contiguous(value)
            rc = _lib.load().nsa_cache_stage_token(key.data_ptr(), value.data_ptr(), self.before_compress_kv_cache.data_ptr(),
                                                   self.before_compress_kv_len.data_ptr(), batch, self.num_kv_heads, self.head_dim,
                                                   key.stride(0), key.stride(1), value.stride(0), value.stride(1),
                                                   self.max_batch_size, self.kernel_size, self.kernel_stride, _lib.stream_ptr(key))
            _lib.check(rc, "nsa_cache_stage_token")

    # ---- a whole decode step's cache work in one launch ---------------------------------------
    @torch.no_grad()
    def decode_prepare(self, query, key, value, inv_freq, attention_scaling, weight_k=None, weight_v=None, bias_k=None):
        """prepare_compress + pooling of a completed window + rotary embedding of query, key and compressed key +
        update_kv for one new token per sequence, as a single kernel (pooling compression only: weight_k / weight_v
        [num_kv_heads, kernel_size] or None for the plain average, bias_k [num_kv_heads, head_dim] the optional
        position term of the pooled key).  Returns the rotated query.  Same cache contents as the separate calls."""
        batch = query.shape[0]
        assert batch <= self.max_batch_size and key.shape == value.shape == (batch, self.num_kv_heads, self.head_dim)
        assert query.shape[2] == self.head_dim and query.dtype == key.dtype == value.dtype == self.dtype
        assert inv_freq.dtype == torch.float32 and inv_freq.is_contiguous() and inv_freq.shape[0] == self.head_dim // 2
        query, key, value = last_dim_contiguous(query), last_dim_contiguous(key), last_dim_contiguous(value)
        for w in (weight_k, weight_v):
            assert w is None or (w.dtype == self.dtype and w.is_contiguous() and w.shape == (self.num_kv_heads, self.kernel_size))
        assert bias_k is None or (bias_k.dtype == self.dtype and bias_k.is_contiguous() and bias_k.shape == (self.num_kv_heads, self.head_dim))
        if not torch.cuda.is_current_stream_capturing():   # a capture records the launch without running it
            self.count_decode_step()
        out = torch.empty_like(query, memory_format=torch.contiguous_format)
        strides = _lib.host_i64([query.stride(0), query.stride(1), key.stride(0), key.stride(1), value.stride(0), value.stride(1),
                                 out.stride(0), out.stride(1)])
        ptr = lambda t: t.data_ptr() if t is not None else None
        rc = _lib.load().nsa_decode_prepare(
            query.data_ptr(), key.data_ptr(), value.data_ptr(), out.data_ptr(), ptr(weight_k), ptr(weight_v), ptr(bias_k),
            inv_freq.data_ptr(), float(attention_scaling), self.before_compress_kv_cache.data_ptr(), self.before_compress_kv_len.data_ptr(),
            self.compress_kv_cache.data_ptr(), self.compress_kv_len.data_ptr(), self.sparse_kv_cache.data_ptr(),
            self.sparse_kv_len.data_ptr(), self.sliding_kv_cache.data_ptr(), self.sliding_kv_len.data_ptr(), batch, query.shape[1],
            self.num_kv_heads, self.head_dim, strides, self.max_batch_size, self.kernel_size, self.kernel_stride, self.max_comp_length,
            self.max_length, self.window_size, _lib.dtype_code(query), _lib.stream_ptr(query))
        _lib.check(rc, "nsa_decode_prepare")
        return out

    # ---- after rope ---------------------------------------------------------------------------
    def update_kv(self, cu_seqlens, step, compress_key, compress_value, sparse_key, sparse_value, sliding_key, sliding_value):
        assert compress_key.shape == compress_value.shape and sparse_key.shape == sparse_value.shape
        assert sliding_key.shape == sliding_value.shape
        batch = cu_seqlens.shape[0] - 1
        if step == 0:
            seqlens = cu_seqlens[1:] - cu_seqlens[:-1]
            self.max_prompt_len = int(seqlens.max())  # the one host read of a prefill
            self.prefill_serial += 1
            self.decode_steps = 0
            assert self.max_prompt_len <= self.max_length
            _, comp_cu = get_compressed_seqlens(cu_seqlens, self.kernel_size, self.kernel_stride)
            self._fill(self.compress_kv_cache, self.compress_kv_len, compress_key, compress_value, comp_cu,
                       comp_cu[:-1].contiguous(), comp_cu[1:].contiguous())
            self._fill(self.sparse_kv_cache, self.sparse_kv_len, sparse_key, sparse_value, cu_seqlens,
                       cu_seqlens[:-1].contiguous(), cu_seqlens[1:].contiguous())
            # the last window_size tokens, stored from row 0 (the decode kernel reads the ring as a set)
            start = torch.maximum(cu_seqlens[1:] - self.window_size, cu_seqlens[:-1]).contiguous()
            self._fill(self.sliding_kv_cache, self.sliding_kv_len, sliding_key, sliding_value, cu_seqlens, start, cu_seqlens[1:].contiguous())
        else:
            assert self.static_shapes or self.max_seqlen(step) <= self.max_length, "cache slab too short for this decode step"
            if not torch.cuda.is_current_stream_capturing():
                self.count_decode_step()
            toks = [last_dim_contiguous(t) for t in (compress_key, compress_value, sparse_key, sparse_value, sliding_key, sliding_value)]
            assert all(t.shape[0] == batch and t.dtype == self.dtype for t in toks)
            ptrs = (ctypes.c_void_p * 6)(*[t.data_ptr() for t in toks])
            strides = _lib.host_i64([s for t in toks for s in (t.stride(0), t.stride(1))])
            rc = _lib.load().nsa_cache_commit_token(
                ptrs, strides, self.before_compress_kv_len.data_ptr(), self.compress_kv_cache.data_ptr(), self.compress_kv_len.data_ptr(),
                self.sparse_kv_cache.data_ptr(), self.sparse_kv_len.data_ptr(), self.sliding_kv_cache.data_ptr(),
                self.sliding_kv_len.data_ptr(), batch, self.num_kv_heads, self.head_dim, self.max_batch_size, self.kernel_size,
                self.max_comp_length, self.max_length, self.window_size, _lib.stream_ptr(toks[2]))
            _lib.check(rc, "nsa_cache_commit_token")
