"""Import-path compatibility only: the reference's callers and scripts import the operators and their private forward /
backward helpers from ``native_sparse_attention.ops.triton.<module>`` (e.g. module/kv_cache.py:18,
infer/inference_func.py:24, test/test_topk_sparse_attention.py:19-31).  The modules here re-export this package's
implementations under those paths.  Nothing here uses Triton."""
