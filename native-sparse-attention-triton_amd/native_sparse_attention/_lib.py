"""ctypes binding of libnsa_hip.so (declared in include/nsa_hip.h).

The shared library is the only compute path: if it has not been built the first call raises;
there is no PyTorch fallback.
"""
import ctypes
import os
from ctypes import c_float, c_int, c_int64, c_size_t, c_void_p

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libnsa_hip.so")
_lib = None

NSA_BF16, NSA_FP16 = 0, 1
_ERR = {-1: "bad argument", -2: "unsupported shape/dtype/alignment", -3: "workspace too small", -4: "kernel launch failed",
        -5: "first call on this device made under graph capture (call once outside a capture first)"}

P, I, F, Z = c_void_p, c_int64, c_float, c_size_t
_SIGNATURES = {
    "nsa_version": (c_int, []),
    "nsa_topk_attn_fwd_workspace_bytes": (Z, [I, I, I, I]),
    "nsa_topk_attn_fwd": (c_int, [P] * 7 + [I] * 7 + [I] * 11 + [F, c_int, P, Z, c_int, P]),
    "nsa_topk_attn_bwd_workspace_bytes": (Z, [I] * 7),
    "nsa_topk_reverse_index_segments": (I, [I] * 4),
    "nsa_topk_attn_bwd": (c_int, [P] * 11 + [I] * 7 + [P, F, c_int, P, Z, P, P, c_int, P]),
    "nsa_pool_fwd": (c_int, [P] * 5 + [I] * 12 + [c_int, P]),
    "nsa_pool_fwd_bias": (c_int, [P] * 6 + [I] * 13 + [c_int, P]),
    "nsa_pool_bwd_workspace_bytes": (Z, [I] * 3),
    "nsa_pool_bwd": (c_int, [P] * 7 + [I] * 15 + [c_int, P, Z, P]),
    "nsa_dense_decode_workspace_bytes": (Z, [I] * 5),
    "nsa_dense_decode": (c_int, [P] * 5 + [I] * 5 + [P, F, c_int, P, Z, P]),
    "nsa_topk_decode_workspace_bytes": (Z, [I] * 6),
    "nsa_topk_decode": (c_int, [P] * 6 + [I] * 7 + [P, F, c_int, P, Z, P]),
    "nsa_topk_decode_static": (c_int, [P] * 6 + [I] * 7 + [P, F, c_int, P]),
    "nsa_cmp_decode_workspace_bytes": (Z, [I] * 5),
    "nsa_cmp_decode": (c_int, [P] * 7 + [I] * 12 + [P, F, c_int, P, Z, P]),
    "nsa_cmp_attn_fwd": (c_int, [P] * 7 + [I] * 8 + [P, F, c_int, P]),
    "nsa_cmp_attn_select": (c_int, [P] * 6 + [I] * 13 + [P, F, c_int, P]),
    "nsa_cmp_attn_bwd_workspace_bytes": (Z, [I] * 6),
    "nsa_cmp_attn_bwd": (c_int, [P] * 11 + [I] * 8 + [P, F, c_int, P, Z, P]),
    "nsa_linear_compress_fwd_workspace_bytes": (Z, [I] * 5),
    "nsa_linear_compress_fwd": (c_int, [P] * 5 + [I] * 11 + [c_int, P, Z, P]),
    "nsa_linear_compress_fwd_bias": (c_int, [P] * 6 + [I] * 12 + [c_int, P]),
    "nsa_linear_compress_bwd": (c_int, [P] * 7 + [I] * 13 + [c_int, P]),
    "nsa_window_attn_fwd": (c_int, [P] * 6 + [I] * 6 + [P, F, c_int, P]),
    "nsa_cache_fill": (c_int, [P] * 7 + [I] * 10 + [P]),
    "nsa_cache_append_token": (c_int, [P] * 4 + [I] * 9 + [P]),
    "nsa_cache_stage_token": (c_int, [P] * 4 + [I] * 10 + [P]),
    "nsa_cache_commit_token": (c_int, [P] * 9 + [I] * 8 + [P]),
    "nsa_gate_combine": (c_int, [P] * 5 + [I] * 3 + [P, c_int, P]),
    "nsa_gate_combine_bwd": (c_int, [P] * 9 + [I] * 3 + [P, c_int, P]),
    "nsa_decode_branches_gate_workspace_bytes": (Z, [I] * 7),
    "nsa_decode_branches_gate": (c_int, [P] * 13 + [I] * 8 + [P, F, c_int, P, Z, P]),
    "nsa_decode_prepare": (c_int, [P] * 8 + [F] + [P] * 8 + [I] * 4 + [P] + [I] * 6 + [c_int, P]),
    "nsa_flash_attn_fwd": (c_int, [P] * 7 + [I] * 6 + [c_int, P, F, c_int, P]),
    "nsa_flash_attn_bwd_workspace_bytes": (Z, [I] * 6),
    "nsa_flash_attn_bwd": (c_int, [P] * 11 + [I] * 6 + [c_int, P, F, c_int, P, Z, P]),
    "nsa_compressed_seqlens": (c_int, [P] + [I] * 3 + [P, P, P]),
    "nsa_rope": (c_int, [P] * 4 + [I] * 10 + [F, c_int, c_int, P]),
    "nsa_window_attn_bwd_workspace_bytes": (Z, [I] * 5),
    "nsa_window_attn_bwd": (c_int, [P] * 10 + [I] * 6 + [P, F, c_int, P, Z, P]),
}


def lib_path() -> str:
    return _LIB_PATH


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                "libnsa_hip.so is not built (%s missing): run `python native-sparse-attention-triton_amd/build.py`" % _LIB_PATH
            )
        lib = ctypes.CDLL(_LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def exported_symbols():
    return sorted(_SIGNATURES)


def check(code: int, what: str):
    if code != 0:
        raise RuntimeError("%s failed: %s (code %d)" % (what, _ERR.get(code, "unknown"), code))


def dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return NSA_BF16
    if t.dtype == torch.float16:
        return NSA_FP16
    raise AssertionError("bf16 or fp16 expected, got %s" % t.dtype)


def stream_ptr(t: torch.Tensor):
    assert t.is_cuda, "the HIP kernels need device tensors"
    return torch.cuda.current_stream(t.device).cuda_stream


def host_i64(values):
    """Host int64 array for the entry points that take their strides as one array."""
    return (c_int64 * len(values))(*[int(v) for v in values])


def workspace(nbytes: int, device) -> torch.Tensor:
    return torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device=device)
