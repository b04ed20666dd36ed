"""Rotary position embedding (llama3 scaling by default) for varlen rows.

Counterpart of native_sparse_attention/module/rope.py:27-209 of the reference: same `RopeConfig` fields
and the same `RotaryEmbedding(config, device)(x, cu_seqlens, step=0, stride=1)` call.  The inverse
frequencies come from the closed form the reference obtains through
transformers.modeling_rope_utils.ROPE_INIT_FUNCTIONS["llama3"] (rope.py:88-90); the rotation itself is a
HIP kernel that derives each row's position from cu_seqlens on the device (no per-sequence host loop, no
cos/sin tables in memory).
"""
import math
from dataclasses import dataclass, field

import torch
from torch import nn

from .. import _lib
from ..ops.utils import last_dim_contiguous


@dataclass
class RopeConfig:
    """Same fields and defaults as the reference's RopeConfig (rope.py:27-49): llama 3.1 settings."""

    max_position_embeddings: int = 131072
    head_dim: int = 128
    rope_theta: float = 500000
    rope_scaling: dict = field(
        default_factory=lambda: {
            "factor": 8.0,
            "high_freq_factor": 4.0,
            "low_freq_factor": 1.0,
            "original_max_position_embeddings": 8192,
            "rope_type": "llama3",
        }
    )
    hidden_size: int = 1
    num_attention_heads: int = 1

    def __post_init__(self):
        self.num_attention_heads = 1
        self.hidden_size = self.head_dim


def compute_inv_freq(config: RopeConfig, device=None):
    """(inv_freq fp32 [head_dim/2], attention_scaling) for rope types "default" and "llama3".

    default: inv_freq[i] = theta^(-2i/d).  llama3: wavelengths above original_max/low_freq_factor are
    divided by `factor`, those below original_max/high_freq_factor are kept, the band in between is
    interpolated with smooth = (original_max/wavelen - low) / (high - low)."""
    scaling = config.rope_scaling
    rope_type = "default" if not scaling else scaling.get("rope_type", scaling.get("type"))
    d = config.head_dim
    inv_freq = 1.0 / (config.rope_theta ** (torch.arange(0, d, 2, dtype=torch.int64).to(device=device, dtype=torch.float) / d))
    if rope_type == "default":
        return inv_freq, 1.0
    if rope_type != "llama3":
        raise NotImplementedError("rope_type %r (supported: default, llama3)" % (rope_type,))
    factor, low, high = scaling["factor"], scaling["low_freq_factor"], scaling["high_freq_factor"]
    old_len = scaling["original_max_position_embeddings"]
    wavelen = 2 * math.pi / inv_freq
    scaled = torch.where(wavelen > old_len / low, inv_freq / factor, inv_freq)
    smooth = (old_len / wavelen - low) / (high - low)
    smoothed = (1 - smooth) * scaled / factor + smooth * scaled
    medium = ~(wavelen < old_len / high) & ~(wavelen > old_len / low)
    return torch.where(medium, smoothed, scaled), 1.0


def rotate_half(x):
    """(-x2, x1) for x = (x1, x2) split in the middle of the last dimension (rope.py:53-58 of the reference).  Kept for
    callers that build the rotation from tensors; RotaryEmbedding.forward does not use it."""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def _rope_launch(x, inv_freq, scaling, cu_seqlens, step, stride, inverse):
    x = last_dim_contiguous(x)
    out = torch.empty_like(x, memory_format=torch.contiguous_format)
    B = max(cu_seqlens.shape[0] - 1, 1)  # ignored when cu_seqlens carries positions (step < 0)
    rc = _lib.load().nsa_rope(x.data_ptr(), out.data_ptr(), inv_freq.data_ptr(), cu_seqlens.data_ptr(), x.shape[0], B, x.shape[1],
                              x.shape[2], x.stride(0), x.stride(1), out.stride(0), out.stride(1), step, stride, scaling,
                              int(inverse), _lib.dtype_code(x), _lib.stream_ptr(x))
    _lib.check(rc, "nsa_rope")
    return out


class _Rope(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, inv_freq, scaling, cu_seqlens, step, stride):
        ctx.save_for_backward(inv_freq, cu_seqlens)
        ctx.args = (scaling, step, stride)
        return _rope_launch(x, inv_freq, scaling, cu_seqlens, step, stride, False)

    @staticmethod
    def backward(ctx, grad):
        inv_freq, cu_seqlens = ctx.saved_tensors
        scaling, step, stride = ctx.args
        return _rope_launch(grad, inv_freq, scaling, cu_seqlens, step, stride, True), None, None, None, None, None


class RotaryEmbedding(nn.Module):
    """forward(x [N, H, D], cu_seqlens, step=0, stride=1) as rope.py:199-209 of the reference.

    step == 0 (training / prefill): N == cu_seqlens[-1], token i of a sequence is rotated for position
    i * stride (stride = kernel_stride for compressed keys).  step > 0 (decode): N == batch and row b is
    rotated for position (len_b + step - 1) * stride, len_b being the prompt length held in cu_seqlens."""

    def __init__(self, config: RopeConfig, device="cuda"):
        super().__init__()
        self.config = config
        inv_freq, self.attention_scaling = compute_inv_freq(config, device)
        self.register_buffer("inv_freq", inv_freq.contiguous(), persistent=False)
        self._inv_freq_f32 = None

    def _frequencies(self):
        """fp32 view of the buffer for the kernel.  Casting the module (`.bfloat16()`, `.half()`) casts the buffer
        too, as it does in the reference, whose forward then widens the rounded values again (rope.py:127-129):
        the same rounded frequencies are used here."""
        f = self.inv_freq
        if f.dtype == torch.float32 and f.is_contiguous():
            return f
        c = self._inv_freq_f32
        if c is None or c[0] is not f:
            self._inv_freq_f32 = c = (f, f.float().contiguous())
        return c[1]

    @torch.no_grad()
    def rotate_at(self, x, position_index, stride=1):
        """Rotate row n of x [N, H, D] for position position_index[n] * stride, position_index an int32 tensor [N] on the
        device (e.g. the cache's length vector): no host knowledge of the positions is needed.  No autograd."""
        assert x.dim() == 3 and x.shape[-1] == self.config.head_dim and position_index.dtype == torch.int32
        assert position_index.shape[0] == x.shape[0] and position_index.is_contiguous()
        return _rope_launch(x, self._frequencies(), float(self.attention_scaling), position_index, -1, int(stride), False)

    @torch.no_grad()
    def generate_cos_sin(self, x, position_ids):
        """cos / sin tables [len, D] in x's dtype for position_ids [1, len] (rope.py:120-155 of the reference, without its
        class-level cache): angle = position * inv_freq in fp32, both halves of the last dimension alike, times the
        attention scaling.  Not used by forward (the kernel forms the angles itself)."""
        angles = position_ids.reshape(-1, 1).float() * self.inv_freq.float()[None, :]
        cos = (angles.cos() * self.attention_scaling).to(x.dtype)
        sin = (angles.sin() * self.attention_scaling).to(x.dtype)
        return torch.cat([cos, cos], dim=-1), torch.cat([sin, sin], dim=-1)

    @torch.no_grad()
    def generate_pos_embs(self, x, cu_seqlens, seqlens, step=0, stride=1):
        """Per-row cos / sin [N, D] as rope.py:157-197 of the reference: step == 0 gives row i of a sequence position
        i * stride, step > 0 gives sequence b the single position (len_b + step - 1) * stride."""
        if step == 0:
            total = int(cu_seqlens[-1])
            start = torch.repeat_interleave(cu_seqlens[:-1].long(), seqlens.long(), output_size=total)
            position = (torch.arange(total, device=x.device) - start) * stride
        else:
            position = (seqlens.long() + step - 1) * stride
        return self.generate_cos_sin(x, position[None, :])

    def forward(self, x, cu_seqlens, step=0, stride=1):
        assert x.dim() == 3 and x.shape[-1] == self.config.head_dim
        assert x.dtype == torch.bfloat16 or x.dtype == torch.float16
        cu_seqlens = cu_seqlens.to(torch.int32)
        assert step >= 0 and (step == 0 or x.shape[0] == cu_seqlens.shape[0] - 1)
        return _Rope.apply(x, self._frequencies(), float(self.attention_scaling), cu_seqlens, int(step), int(stride))
