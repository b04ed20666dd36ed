"""The C-ABI library loads without a GPU and exports every symbol the header declares (no compute calls here)."""
import ctypes
import os
import re

from native_sparse_attention import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "nsa_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nsa_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    names = _declared()
    assert len(names) >= 20
    lib = ctypes.CDLL(_lib.lib_path())
    for n in names:
        assert hasattr(lib, n), "library does not export " + n
    assert sorted(_lib.exported_symbols()) == names, "ctypes table and header disagree"


def test_version_and_workspace_queries_run_on_host():
    lib = _lib.load()
    assert lib.nsa_version() >= 100
    # size queries are pure host arithmetic
    # fragment-major copies of K and V, plus the pacing table (8 x 512 entries  and the nine sweep bounds, int32)
    assert lib.nsa_topk_attn_fwd_workspace_bytes(32768, 1, 4, 128) == 2 * 4 * (1024 + 2) * 128 * 32 * 2 + (8 * 512 + 16) * 4
    assert lib.nsa_topk_attn_bwd_workspace_bytes(2048, 1, 64, 4, 128, 16, 64) > 0
    assert lib.nsa_pool_bwd_workspace_bytes(4095, 2, 32) >= 2 * 64 * 32 * 4
    assert lib.nsa_topk_reverse_index_segments(2048, 3, 4, 64) == 4 * (32 + 3)


def test_bad_arguments_are_rejected_without_launching():
    lib = _lib.load()
    # null pointers -> NSA_ERR_BAD_ARG before anything touches a device
    rc = lib.nsa_pool_fwd(None, None, None, None, None, 10, 0, 1, 1, 128, 32, 16, 128, 128, 128, 128, 32, 0, None)
    assert rc == -1
    rc = lib.nsa_dense_decode(None, None, None, None, None, 1, 16, 1, 128, 64, None, 1.0, 0, None, 0, None)
    assert rc == -1


def test_more_host_side_checks():
    lib = _lib.load()
    fake = 1 << 20  # non-null, 16-byte aligned; never dereferenced: the checks below fail before any launch
    # a softmax scale that is not a finite number is refused (any finite one, negative or zero included, is accepted)
    rc = lib.nsa_topk_attn_fwd(fake, fake, fake, fake, fake, fake, fake, 128, 1, 16, 1, 128, 4, 64, 2048, 128, 128, 128, 128, 128,
                               512, 4, 1, 2048, 128, float("nan"), 0, fake, 1 << 30, 3, None)
    assert rc == -1
    # the linear_compress forward sums the shares of its waves in LDS: no workspace
    assert lib.nsa_linear_compress_fwd_workspace_bytes(1021, 3, 4, 128, 32) == 0
    assert lib.nsa_linear_compress_fwd_workspace_bytes(200000, 1, 8, 128, 32) == 0
    # a cache update with more sequences than the slab holds
    assert lib.nsa_cache_stage_token(fake, fake, fake, fake, 5, 2, 128, 256, 128, 256, 128, 4, 32, 16, None) == -1
    # rope needs row strides that are multiples of 8 elements
    assert lib.nsa_rope(fake, fake, fake, fake, 10, 1, 2, 128, 260, 128, 256, 128, 0, 1, 1.0, 0, 0, None) == -2


def test_backward_refuses_strides_beyond_31_bits():
    lib = _lib.load()
    fake = 1 << 20
    # head stride of q times the group size must fit 31 bits for the dK/dV pass: [Hq, T, D] views of very long inputs do not
    strides = (ctypes.c_int64 * 19)(128, 1 << 28, 512, 128, 512, 128, 8192, 128, 8192, 128, 2048 * 16, 16, 1, 8192, 128, 512, 128, 512, 128)
    ws = lib.nsa_topk_attn_bwd_workspace_bytes(2048, 1, 64, 4, 128, 16, 64)
    rc = lib.nsa_topk_attn_bwd(fake, fake, fake, fake, fake, fake, fake, fake, fake, fake, fake, 2048, 1, 64, 4, 128, 16, 64, strides, 0.1,
                               0, fake, ws, None, None, 7, None)
    assert rc == -2


def test_decode_step_entry_points_check_their_arguments():
    lib = _lib.load()
    fake = 1 << 20
    strides8 = (ctypes.c_int64 * 8)(4096, 128, 256, 128, 256, 128, 4096, 128)
    # a null slab pointer
    rc = lib.nsa_decode_prepare(fake, fake, fake, fake, None, None, None, fake, 1.0, None, fake, fake, fake, fake, fake, fake, fake,
                                4, 32, 2, 128, strides8, 4, 32, 16, 511, 8192, 512, 0, None)
    assert rc == -1
    # more sequences than the slabs hold
    rc = lib.nsa_decode_prepare(fake, fake, fake, fake, None, None, None, fake, 1.0, fake, fake, fake, fake, fake, fake, fake, fake,
                                5, 32, 2, 128, strides8, 4, 32, 16, 511, 8192, 512, 0, None)
    assert rc == -1
    # a row stride that is not a multiple of 8 elements
    bad = (ctypes.c_int64 * 8)(4100, 128, 256, 128, 256, 128, 4096, 128)
    rc = lib.nsa_decode_prepare(fake, fake, fake, fake, None, None, None, fake, 1.0, fake, fake, fake, fake, fake, fake, fake, fake,
                                4, 32, 2, 128, bad, 4, 32, 16, 511, 8192, 512, 0, None)
    assert rc == -2
    # the two-launch branches + gate call: workspace too small
    strides28 = (ctypes.c_int64 * 28)(*([128] * 28))
    need = lib.nsa_decode_branches_gate_workspace_bytes(4, 32, 2, 128, 512, 8, 64)
    assert need > 0
    rc = lib.nsa_decode_branches_gate(fake, fake, fake, fake, fake, fake, fake, fake, fake, fake, fake, fake, fake, 4, 32, 2, 128, 8192, 512,
                                      8, 64, strides28, 0.088, 0, fake, need - 1, None)
    assert rc == -3


def test_reference_import_paths_resolve():
    """The names the reference's callers and scripts import (native_sparse_attention/ops/__init__.py:15-53,
    infer/__init__.py:15, infer/nsa_inference.py:16-22, module/__init__.py, model/__init__.py, module/kv_cache.py:18,
    test/test_topk_sparse_attention.py:16-31)
    exist under the same module paths; importing needs neither a GPU nor the shared library."""
    import importlib

    wanted = {
        "native_sparse_attention.ops": ["avgpool_compress", "weightedpool_compress", "linear_compress", "flash_attention_varlen",
                                        "compressed_attention", "topk_sparse_attention", "flash_attention_decode",
                                        "compressed_attention_decode", "topk_sparse_attention_decode"],
        "native_sparse_attention.ops.triton.utils": ["get_compressed_seqlens"],
        "native_sparse_attention.ops.triton.topk_sparse_attention": ["topk_sparse_attention", "_topk_sparse_attention_fwd",
                                                                      "_topk_sparse_attention_bwd"],
        "native_sparse_attention.ops.triton.compressed_attention": ["compressed_attention", "_compressed_attention_fwd",
                                                                     "_compressed_attention_bwd"],
        "native_sparse_attention.ops.triton.flash_attention": ["flash_attention_varlen", "_flash_attention_fwd", "_flash_attention_bwd"],
        "native_sparse_attention.ops.triton.linear_compress": ["linear_compress"],
        "native_sparse_attention.ops.triton.weighted_pool": ["weightedpool_compress", "avgpool_compress"],
        "native_sparse_attention.ops.triton.flash_attention_decode": ["flash_attention_decode"],
        "native_sparse_attention.ops.triton.topk_sparse_attention_decode": ["topk_sparse_attention_decode"],
        "native_sparse_attention.ops.torch.compressed_attention_decode": ["compressed_attention_decode"],
        "native_sparse_attention.ops.topk_sparse_attention": ["_topk_sparse_attention_fwd", "_topk_sparse_attention_bwd"],
        "native_sparse_attention.ops.compressed_attention": ["_compressed_attention_bwd"],
        "native_sparse_attention.infer": ["nsa_infer"],
        "native_sparse_attention.infer.inference_func": ["compress_infer", "compressed_attention_infer", "topk_sparse_attention_infer",
                                                         "sliding_window_attention_infer"],
        "native_sparse_attention.module": ["NativeSparseAttention", "SelfAttention", "RopeConfig", "RotaryEmbedding", "NSACache", "KVCache"],
        "native_sparse_attention.model": ["ToyNSALlama", "ToyNSALlamaConfig", "ToyLlama", "ToyLlamaConfig", "InferenceConfig"],
    }
    for module, names in wanted.items():
        mod = importlib.import_module(module)
        for name in names:
            assert hasattr(mod, name), "%s.%s" % (module, name)
