import torch

MAX_ABS, MEAN_ABS = 2e-2, 2e-3   # bf16/fp16 inputs, fp32 accumulation


def assert_close(got: torch.Tensor, want: torch.Tensor, what: str, max_abs: float = MAX_ABS, mean_abs: float = MEAN_ABS, rel_to=None):
    """max-abs / mean-abs bound; for gradients whose magnitude is far from 1 pass rel_to to scale the bound."""
    g, w = got.float(), want.float()
    assert g.shape == w.shape, (what, g.shape, w.shape)
    assert torch.isfinite(g).all(), what + ": non-finite values"
    scale = 1.0 if rel_to is None else max(1.0, float(rel_to))
    err = (g - w).abs()
    assert err.max().item() <= max_abs * scale, "%s: max abs err %.4g > %.4g" % (what, err.max().item(), max_abs * scale)
    assert err.mean().item() <= mean_abs * scale, "%s: mean abs err %.4g > %.4g" % (what, err.mean().item(), mean_abs * scale)
