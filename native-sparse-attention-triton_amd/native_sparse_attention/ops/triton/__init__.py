"""Import-path compatibility only: callers of the reference import
``native_sparse_attention.ops.triton.utils.get_compressed_seqlens`` (module/kv_cache.py:18,
infer/inference_func.py:24).  Nothing here uses Triton."""
