"""CPU restatement of the Native Sparse Attention operator path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory: it exists so that tests, the smoke check and the CPU-baseline leg of
the benchmark have an independent, slow, obviously-correct statement of what
each operator must return.  Everything here is plain PyTorch on whatever device
and dtype the inputs carry (fp64 for gradient checks, fp32 for CPU parity,
bf16 to mimic the rounding points of the device kernels).

How each function is pinned (tests/test_oracle_*.py):

* ``sparse_attn.topk_sparse_attention``   - brute-force scalar loops on tiny
  inputs; equals causal SDPA when every causal block is selected; varlen equals
  per-sequence; invariant under permutation of the selected ids.
* ``sparse_attn.build_reverse_index``     - brute-force enumeration.
* ``compress.*``                          - ``F.avg_pool1d`` / grouped
  ``F.conv1d`` / dense ``F.conv1d`` on each sequence.
* ``cmp_attn.compressed_attention``       - SDPA with an explicit boolean mask;
  block scores against a set-intersection derivation of the overlap weights;
  structural invariants of ``topk_idx``.
* ``decode.*``                            - equal to the last row of the
  corresponding prefill oracle on the same sequence.

No function is left "parity unpinned".
"""
from .sparse_attn import topk_sparse_attention, build_reverse_index  # noqa: F401
from .compress import (  # noqa: F401
    compressed_seqlens,
    avgpool_compress,
    weightedpool_compress,
    linear_compress,
)
from .cmp_attn import compressed_attention, block_scores_from_probs, select_topk  # noqa: F401
from .decode import (  # noqa: F401
    dense_attention_decode,
    topk_sparse_attention_decode,
    compressed_attention_decode,
)
