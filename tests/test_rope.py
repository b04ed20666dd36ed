"""Rotary embedding: the closed-form inverse frequencies against the library routine the reference calls
(CPU), and the HIP kernel against an element-wise restatement of the reference's forward (GPU)."""
import pytest
import torch

from native_sparse_attention.module.rope import RopeConfig, RotaryEmbedding, compute_inv_freq
from native_sparse_attention.testing import cu_from_lens


def test_inv_freq_matches_transformers_llama3():
    transformers = pytest.importorskip("transformers")
    from transformers.modeling_rope_utils import ROPE_INIT_FUNCTIONS
    for d, theta in [(128, 500000.0), (64, 10000.0)]:
        cfg = RopeConfig(head_dim=d, rope_theta=theta)
        try:
            lib_cfg = transformers.LlamaConfig(hidden_size=d, num_attention_heads=1, head_dim=d, max_position_embeddings=cfg.max_position_embeddings,
                                               rope_parameters=dict(cfg.rope_scaling, rope_theta=theta))
            want, scale = ROPE_INIT_FUNCTIONS["llama3"](lib_cfg, "cpu")
        except (TypeError, AttributeError, KeyError) as e:  # another transformers generation: different config protocol
            pytest.skip("installed transformers does not take this config: %r" % (e,))
        got, got_scale = compute_inv_freq(cfg, "cpu")
        assert torch.equal(got, want) and got_scale == scale == 1.0


def test_inv_freq_default_and_bands():
    cfg = RopeConfig(head_dim=64, rope_theta=10000.0, rope_scaling=None)
    inv, _ = compute_inv_freq(cfg, "cpu")
    assert torch.allclose(inv, 10000.0 ** (-torch.arange(0, 64, 2).float() / 64))
    # llama3: short wavelengths untouched, long ones divided by the factor, monotone in between
    cfg = RopeConfig()
    base = 1.0 / (cfg.rope_theta ** (torch.arange(0, 128, 2).float() / 128))
    inv, _ = compute_inv_freq(cfg, "cpu")
    wl = 2 * torch.pi / base
    assert torch.equal(inv[wl < 8192 / 4], base[wl < 8192 / 4])
    assert torch.allclose(inv[wl > 8192], base[wl > 8192] / 8)
    assert (inv[1:] < inv[:-1]).all()


def _reference_forward(x, inv_freq, positions):
    """rope.py:120-152,199-209 restated: cos/sin in fp32, cast to x.dtype, then x*cos + rotate_half(x)*sin
    in x.dtype arithmetic."""
    freqs = positions.float()[:, None] * inv_freq.float()[None, :]
    cos = torch.cat([freqs.cos(), freqs.cos()], -1).to(x.dtype)[:, None, :]
    sin = torch.cat([freqs.sin(), freqs.sin()], -1).to(x.dtype)[:, None, :]
    half = x.shape[-1] // 2
    rot = torch.cat((-x[..., half:], x[..., :half]), dim=-1)
    return x * cos + rot * sin


@pytest.mark.gpu
@pytest.mark.parametrize("lens,H,d,stride,dtype", [
    ([100, 257, 31], 8, 128, 1, torch.bfloat16),
    ([63, 447, 511], 4, 128, 16, torch.bfloat16),     # compressed keys: positions i * kernel_stride
    ([300], 3, 64, 1, torch.float16),
    ([40000], 1, 32, 3, torch.bfloat16),              # angles beyond 1e5 rad
])
def test_prefill_rotation_and_gradient(device, lens, H, d, stride, dtype):
    g = torch.Generator(device=device).manual_seed(0)
    cu = cu_from_lens(lens, device)
    rope = RotaryEmbedding(RopeConfig(head_dim=d), device=device)
    x = torch.randn(int(cu[-1]), H, d, generator=g, device=device).to(dtype)
    pos = torch.cat([torch.arange(L, device=device) * stride for L in lens])
    x1 = x.clone().requires_grad_()
    y = rope(x1, cu, stride=stride)
    want = _reference_forward(x, rope.inv_freq, pos)
    # the same roundings on both sides; cos/sin of the two libraries may differ in the last bit, which moves a
    # result by at most one unit in the last place of the element type
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    err = (y.float() - want.float()).abs()
    assert (err <= ulp * want.float().abs().clamp(min=1.0)).all()
    assert (y == want).float().mean() > 0.98
    # gradient = the transposed rotation (checked against autograd of an fp32 statement)
    dy = torch.randn(y.shape, generator=g, device=device).to(dtype)
    y.backward(dy)
    xf = x.float().requires_grad_()
    freqs = pos.float()[:, None] * rope.inv_freq[None, :]
    cos = torch.cat([freqs.cos(), freqs.cos()], -1)[:, None, :]
    sin = torch.cat([freqs.sin(), freqs.sin()], -1)[:, None, :]
    (xf * cos + torch.cat((-xf[..., d // 2:], xf[..., :d // 2]), -1) * sin).backward(dy.float())
    assert (x1.grad.float() - xf.grad).abs().max() < 4e-2
    assert (x1.grad.float() - xf.grad).abs().mean() < 4e-3


@pytest.mark.gpu
def test_decode_positions(device):
    g = torch.Generator(device=device).manual_seed(1)
    lens, H, d = [130, 47, 300], 8, 128
    cu = cu_from_lens(lens, device)
    rope = RotaryEmbedding(RopeConfig(head_dim=d), device=device)
    x = torch.randn(len(lens), H, d, generator=g, device=device).bfloat16()
    for step, stride in [(1, 1), (7, 1), (3, 16)]:
        pos = torch.tensor([(L + step - 1) * stride for L in lens], device=device)
        y = rope(x, cu, step=step, stride=stride)
        want = _reference_forward(x, rope.inv_freq, pos)
        assert ((y.float() - want.float()).abs() <= 2.0 ** -7 * want.float().abs().clamp(min=1.0)).all()


@pytest.mark.gpu
def test_module_cast_to_bf16_rounds_the_frequencies_like_the_reference(device):
    """`.bfloat16()` on the owning module casts the inv_freq buffer (in the reference too, whose forward widens the
    rounded values again): the kernel must be handed fp32 copies of those rounded values, not the 2-byte buffer."""
    lens, H, d = [50, 20], 2, 64
    cu = cu_from_lens(lens, device)
    rope = RotaryEmbedding(RopeConfig(head_dim=d), device=device).bfloat16()
    assert rope.inv_freq.dtype == torch.bfloat16
    g = torch.Generator(device=device).manual_seed(3)
    x = torch.randn(sum(lens), H, d, generator=g, device=device).bfloat16()
    pos = torch.cat([torch.arange(L, device=device) for L in lens])
    y = rope(x, cu)
    want = _reference_forward(x, rope.inv_freq.float(), pos)
    assert torch.isfinite(y).all()
    assert ((y.float() - want.float()).abs() <= 2.0 ** -7 * want.float().abs().clamp(min=1.0)).all()


def test_tensor_level_helpers_agree_with_the_closed_form():
    """rotate_half / generate_cos_sin / generate_pos_embs (the reference's tensor-level helpers, rope.py:53-58,120-197):
    x * cos + rotate_half(x) * sin built from them is the textbook rotation of each (x1, x2) pair by position * inv_freq
    (checked in fp64 on the CPU), for prefill rows and for a decode step."""
    from native_sparse_attention.module.rope import rotate_half

    rope = RotaryEmbedding(RopeConfig(head_dim=16, rope_scaling=None, rope_theta=100.0), device="cpu")
    cu = torch.tensor([0, 3, 8], dtype=torch.int32)
    seqlens = cu[1:] - cu[:-1]
    g = torch.Generator().manual_seed(0)
    x = torch.randn(8, 2, 16, generator=g, dtype=torch.float64)
    assert torch.equal(rotate_half(x), torch.cat((-x[..., 8:], x[..., :8]), -1))
    for step, stride, rows, positions in ((0, 4, x, [0, 4, 8, 0, 4, 8, 12, 16]), (2, 1, x[:2], [4, 6])):
        cos, sin = rope.generate_pos_embs(rows, cu, seqlens, step=step, stride=stride)
        assert cos.shape == (rows.shape[0], 16) and cos.dtype == rows.dtype
        got = rows * cos[:, None, :] + rotate_half(rows) * sin[:, None, :]
        ang = torch.tensor(positions, dtype=torch.float64)[:, None] * rope.inv_freq.double()[None, :]
        x1, x2 = rows[..., :8], rows[..., 8:]
        want = torch.cat((x1 * ang.cos()[:, None] - x2 * ang.sin()[:, None], x2 * ang.cos()[:, None] + x1 * ang.sin()[:, None]), -1)
        assert torch.allclose(got, want, atol=1e-6)
