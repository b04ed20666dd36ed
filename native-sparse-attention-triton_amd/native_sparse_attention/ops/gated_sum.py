"""Gated sum of the three attention branches,
gate[..., 0:1] * branch0 + gate[..., 1:2] * branch1 + gate[..., 2:3] * branch2
(module/native_sparse_attention.py:228-232 and infer/nsa_inference.py:146-150 of the reference, where it is five
element-wise tensor operations), as one kernel per direction.  Products and partial sums are rounded to the
element type in the order of that expression, so the forward is bit-identical to it."""
import torch

from .. import _lib
from .utils import last_dim_contiguous


def _strides(gate_value, a, b, c, last):
    return _lib.host_i64([gate_value.stride(0), gate_value.stride(1), gate_value.stride(2), a.stride(0), a.stride(1), b.stride(0),
                          b.stride(1), c.stride(0), c.stride(1), last.stride(0), last.stride(1)])


def gate_combine(gate_value, branch0, branch1, branch2):
    """The gated sum without autograd.  gate_value [n, num_q_heads, 3]; branches [n, num_q_heads, head_dim]."""
    assert gate_value.shape == branch0.shape[:2] + (3,) and branch0.shape == branch1.shape == branch2.shape
    assert gate_value.dtype == branch0.dtype == branch1.dtype == branch2.dtype
    a, b, c = (last_dim_contiguous(t) for t in (branch0, branch1, branch2))
    out = torch.empty_like(a, memory_format=torch.contiguous_format)
    rc = _lib.load().nsa_gate_combine(gate_value.data_ptr(), a.data_ptr(), b.data_ptr(), c.data_ptr(), out.data_ptr(), a.shape[0],
                                      a.shape[1], a.shape[2], _strides(gate_value, a, b, c, out), _lib.dtype_code(a), _lib.stream_ptr(a))
    _lib.check(rc, "nsa_gate_combine")
    return out


class _GatedSum(torch.autograd.Function):
    @staticmethod
    def forward(ctx, gate_value, branch0, branch1, branch2):
        ctx.save_for_backward(gate_value, branch0, branch1, branch2)
        return gate_combine(gate_value, branch0, branch1, branch2)

    @staticmethod
    def backward(ctx, dout):
        gate_value, branch0, branch1, branch2 = ctx.saved_tensors
        a, b, c, do = (last_dim_contiguous(t) for t in (branch0, branch1, branch2, dout))
        dgate = torch.empty(gate_value.shape, dtype=gate_value.dtype, device=gate_value.device)
        da, db, dc = (torch.empty(a.shape, dtype=a.dtype, device=a.device) for _ in range(3))
        rc = _lib.load().nsa_gate_combine_bwd(gate_value.data_ptr(), a.data_ptr(), b.data_ptr(), c.data_ptr(), do.data_ptr(),
                                              dgate.data_ptr(), da.data_ptr(), db.data_ptr(), dc.data_ptr(), a.shape[0], a.shape[1],
                                              a.shape[2], _strides(gate_value, a, b, c, do), _lib.dtype_code(a), _lib.stream_ptr(a))
        _lib.check(rc, "nsa_gate_combine_bwd")
        return dgate, da, db, dc


def gated_sum(gate_value, branch0, branch1, branch2):
    """The gated sum with autograd: d branch_i = gate_i * dout, d gate_i = sum over head_dim of dout * branch_i."""
    return _GatedSum.apply(gate_value, branch0, branch1, branch2)
