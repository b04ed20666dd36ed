"""One NSA decode step captured in a HIP graph.

A decode step is about twenty small kernels (cache update, compression, rotary embedding, three attention
branches with their merges, block selection, gate) whose run time is a fraction of their launch cost.  None
of them needs a host-side value that changes from step to step: positions and lengths live in the cache's
device vectors, and with `cache.static_shapes` the slab views and the shape of the selected-block ids do not
depend on how far decoding has come.  The step can therefore be recorded once and replayed.
"""
from typing import Callable, Optional, Tuple

import torch

from .nsa_inference import nsa_infer


class NSADecodeGraph:
    """Records `nsa_infer(cu_seqlens, step > 0, ...)` for a fixed batch and replays it for every new token.

    The arguments after `num_q_heads` are those of nsa_infer.  `rope` must offer `rotate_at` (this package's
    RotaryEmbedding) and `local_blocks` must be at least 1 (a sequence's own, partly filled block is then always
    selected, which makes the block ids independent of the longest sequence in the batch).  The cache must have
    been filled by a prefill of the same batch before the first `step`; a later prefill of another batch of the same
    size into the same cache can reuse the object.  Replays run on the stream that is current when `step` is called.

    A recorded step cannot look at lengths on the host, so every replay is counted on the cache (`NSACache.count_decode_step`,
    which eager decode steps and other graphs recorded on the same cache go through as well) and raises once the longest
    sequence would outgrow the cache (`max_prompt_len + decode_steps > cache.max_length`).  The
    kernels themselves never write past a slab either: a sequence that has filled its rows is left as it is
    (no token stored, length not advanced), which keeps memory safe but would make later outputs meaningless.
    """

    def __init__(self, cu_seqlens: torch.Tensor, num_q_heads: int, rope, cache, compress_weight: Tuple[torch.Tensor, torch.Tensor],
                 compress_func: Tuple[Callable, Callable], intra_block_pe: Optional[torch.Tensor], kernel_size: int, kernel_stride: int,
                 block_size: int, topk: int, init_blocks: int, local_blocks: int, window_size: int):
        assert hasattr(rope, "rotate_at"), "positions must come from the cache's device-side lengths"
        assert local_blocks >= 1
        batch = cu_seqlens.shape[0] - 1
        dev, dt = cache.sparse_kv_cache.device, cache.dtype
        self.cache = cache
        self.query = torch.zeros(batch, num_q_heads, cache.head_dim, dtype=dt, device=dev)
        self.key = torch.zeros(batch, cache.num_kv_heads, cache.head_dim, dtype=dt, device=dev)
        self.value = torch.zeros_like(self.key)
        self.gate = torch.zeros(batch, num_q_heads, 3, dtype=dt, device=dev)
        self.cu_seqlens = cu_seqlens.to(torch.int32).clone()
        cache.static_shapes = True
        self.graph = torch.cuda.CUDAGraph()
        # capturing records the launches without running them: the cache is not touched here
        with torch.cuda.graph(self.graph):
            self.out = nsa_infer(self.cu_seqlens, 1, self.query, self.key, self.value, self.gate, rope, cache, compress_weight,
                                 compress_func, intra_block_pe, kernel_size, kernel_stride, block_size, topk, init_blocks,
                                 local_blocks, window_size)

    def _count_step(self):
        # the cache keeps one count for eager steps, this graph's replays and any other graph recorded on it
        self.cache.count_decode_step()

    @torch.no_grad()
    def step(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, gate_value: torch.Tensor) -> torch.Tensor:
        """One new token per sequence; returns a view of the graph's output buffer (valid until the next call)."""
        self._count_step()
        dst, src = [self.query, self.key, self.value, self.gate], [query, key, value, gate_value]
        if hasattr(torch, "_foreach_copy_"):
            torch._foreach_copy_(dst, src)   # one launch for the four copies
        else:
            for d, s in zip(dst, src):
                d.copy_(s)
        self.graph.replay()
        return self.out

    @torch.no_grad()
    def replay(self) -> torch.Tensor:
        """The same step for a caller that has already written the new token's states into `self.query`, `self.key`,
        `self.value` and `self.gate` (for example as the `out=` of its projections): no copies, one graph launch."""
        self._count_step()
        self.graph.replay()
        return self.out
