"""Host-side helpers shared by the operators."""
import torch


def get_compressed_seqlens(cu_seqlens: torch.Tensor, kernel_size: int, kernel_stride: int):
    """Per-sequence lengths after sliding-window compression and their cumulative sum.

    y_len = floor((L - kernel_size) / kernel_stride) + 1, or 0 when L < kernel_size; both results are
    int32 on the device of ``cu_seqlens`` (same contract as the reference's
    native_sparse_attention/ops/triton/utils.py:25-37).
    """
    if cu_seqlens.is_cuda and cu_seqlens.dtype == torch.int32 and cu_seqlens.is_contiguous():
        from .. import _lib  # one launch instead of a dozen tensor operations
        batch = cu_seqlens.shape[0] - 1
        y_seqlens = torch.empty(batch, dtype=torch.int32, device=cu_seqlens.device)
        y_cu_seqlens = torch.empty(batch + 1, dtype=torch.int32, device=cu_seqlens.device)
        rc = _lib.load().nsa_compressed_seqlens(cu_seqlens.data_ptr(), batch, kernel_size, kernel_stride, y_seqlens.data_ptr(),
                                                y_cu_seqlens.data_ptr(), _lib.stream_ptr(cu_seqlens))
        _lib.check(rc, "nsa_compressed_seqlens")
        return y_seqlens, y_cu_seqlens
    seqlens = cu_seqlens[1:] - cu_seqlens[:-1]
    y_seqlens = torch.div(seqlens - kernel_size, kernel_stride, rounding_mode="floor").to(torch.int32) + 1
    y_seqlens = torch.where(seqlens < kernel_size, torch.zeros_like(y_seqlens), y_seqlens)
    y_cu_seqlens = torch.zeros(y_seqlens.shape[0] + 1, dtype=torch.int32, device=cu_seqlens.device)
    y_cu_seqlens[1:] = torch.cumsum(y_seqlens, dim=0)
    return y_seqlens, y_cu_seqlens


# Compressed lengths of the cu_seqlens tensors seen last: K and V of a layer (and every layer of a model) compress with the
# same cu_seqlens object, and each fresh computation costs a launch plus, for the output shape, a device read.  An entry
# is valid while the very same tensor object is alive and has not been written to (its version counter is unchanged).
_SEQLEN_CACHE = {}


def compressed_seqlens_cached(cu_seqlens: torch.Tensor, kernel_size: int, kernel_stride: int, need_total: bool):
    """(y_cu_seqlens, total or None): as get_compressed_seqlens, remembered per cu_seqlens object; total = the sum of the
    compressed lengths as a host integer (one device read, the first time it is asked for)."""
    import weakref

    key = (id(cu_seqlens), kernel_size, kernel_stride)
    hit = _SEQLEN_CACHE.get(key)
    if hit is not None and hit[0]() is cu_seqlens and hit[1] == cu_seqlens._version:
        entry = hit
    else:
        if len(_SEQLEN_CACHE) >= 32:
            for k_ in [k_ for k_, e in _SEQLEN_CACHE.items() if e[0]() is None] or list(_SEQLEN_CACHE)[:16]:
                del _SEQLEN_CACHE[k_]
        entry = [weakref.ref(cu_seqlens), cu_seqlens._version, get_compressed_seqlens(cu_seqlens, kernel_size, kernel_stride)[1], None]
        _SEQLEN_CACHE[key] = entry
    if need_total and entry[3] is None:
        entry[3] = int(entry[2][-1])
    return entry[2], entry[3]


def last_dim_contiguous(t: torch.Tensor) -> torch.Tensor:
    return t if t.stride(-1) == 1 else t.contiguous()


# Head sizes the attention and decode kernels are compiled for.  Any other multiple of 8 up to the largest runs on the
# next built size with zero columns appended to q, k and v (they add nothing to a score, and the output columns they
# produce are zero and dropped), as the reference's kernels do inside their tiles with BLOCK_SIZE_D =
# next_power_of_2(head_dim) and masked loads (ops/triton/topk_sparse_attention.py:866).  Here the host appends the
# columns: one extra copy of the operands for such head sizes, none for the built ones.
BUILT_HEAD_DIMS = (32, 64, 96, 128)


def built_head_dim(head_dim: int) -> int:
    assert head_dim % 8 == 0 and 0 < head_dim <= BUILT_HEAD_DIMS[-1], "head_dim must be a multiple of 8, at most %d" % BUILT_HEAD_DIMS[-1]
    return next(d for d in BUILT_HEAD_DIMS if d >= head_dim)


def pad_head_dim(*tensors):
    """The tensors with their last dimension zero-padded to the built head size (unchanged when it is one)."""
    d = tensors[0].shape[-1]
    D = built_head_dim(d)
    if D == d:
        return tensors
    return tuple(torch.nn.functional.pad(t, (0, D - d)) for t in tensors)
