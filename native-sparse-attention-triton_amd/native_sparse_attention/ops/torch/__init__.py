"""Import path of the reference's ops/torch package.  The reference's decode step takes compressed_attention_decode from here
(ops/__init__.py:33-35); the other modules of that package are the plain-PyTorch implementations its tests compare against
and have no counterpart in this package."""
