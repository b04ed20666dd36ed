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
    assert lib.nsa_topk_attn_fwd_workspace_bytes(32768, 1, 4, 128) == 2 * 4 * (1024 + 2) * 128 * 32 * 2
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
