import torch

MAX_ABS, MEAN_ABS = 2e-2, 2e-3   # bf16/fp16 inputs, fp32 accumulation


def assert_close(got: torch.Tensor, want: torch.Tensor, what: str, max_abs: float = MAX_ABS, mean_abs: float = MEAN_ABS, rel_to=None):
    """max-abs / mean-abs bound against the oracle.  Plain (rel_to None): absolute bounds, for outputs of magnitude ~1.
    With rel_to (any value): every row (last dimension: the head_dim values of one token and head, the taps of one
    pooling weight ...) is held to the bounds scaled by max(1, largest reference magnitude of THAT row) - gradients of
    early keys sum over thousands of queries and reach the hundreds, where half a bf16 ulp alone is 0.1, while late keys
    and most query rows stay below 1 and are held to the absolute bound."""
    g, w = got.float(), want.float()
    assert g.shape == w.shape, (what, g.shape, w.shape)
    assert torch.isfinite(g).all(), what + ": non-finite values"
    err = (g - w).abs()
    if rel_to is not None and w.dim() >= 1 and w.numel() > 0:
        err = err / w.abs().amax(dim=-1, keepdim=True).clamp(min=1.0)
    assert err.max().item() <= max_abs, "%s: max abs err %.4g (relative to its row's scale) > %.4g" % (what, err.max().item(), max_abs)
    assert err.mean().item() <= mean_abs, "%s: mean abs err %.4g (relative to row scales) > %.4g" % (what, err.mean().item(), mean_abs)


def clear_margin_rows(block_score: torch.Tensor, want_idx: torch.Tensor, q_block: torch.Tensor, margin: float = 1e-3) -> torch.Tensor:
    """Rows [Hkv, R] on which the oracle's selection is decided by more than `margin`: the smallest selected block score
    exceeds the largest rejected one (among causal blocks with a finite score, i.e. not forced) by more than that.
    block_score [Hkv, R, n_blocks] fp32 (forced blocks +inf), want_idx [Hkv, R, k] (ids, -1 padded), q_block [R]."""
    nb = block_score.shape[-1]
    causal = torch.arange(nb, device=block_score.device)[None, None] <= q_block[None, :, None]
    sc = torch.where(causal & torch.isfinite(block_score), block_score, torch.full_like(block_score, float("nan")))
    sel = torch.zeros_like(block_score, dtype=torch.bool)
    sel.scatter_(2, want_idx.clamp(min=0).long(), True)
    sel &= causal
    worst_in = torch.where(sel, sc, torch.full_like(sc, float("inf"))).nan_to_num(float("inf")).amin(-1)
    best_out = torch.where(~sel & causal, sc, torch.full_like(sc, float("-inf"))).nan_to_num(float("-inf")).amax(-1)
    # more forced (+inf) blocks than slots: which of them the selection keeps is a tie among equal scores
    n_forced = (causal & torch.isinf(block_score)).sum(-1)
    return ((worst_in - best_out) > margin) & (n_forced <= want_idx.shape[-1])


def assert_ids_match(idx: torch.Tensor, want_idx: torch.Tensor, block_score: torch.Tensor, q_block: torch.Tensor, what: str,
                     min_overlap: float = 0.97):
    """The contract for selected block ids: bit-exact on every row whose oracle margin is clear (> 1e-3); on the other
    rows (two block scores within rounding of each other) the overlap of the id sets is reported and bounded."""
    assert idx.shape == want_idx.shape and idx.dtype == torch.int32, (what, idx.shape, want_idx.shape, idx.dtype)
    clear = clear_margin_rows(block_score, want_idx, q_block)
    exact = (idx == want_idx).all(-1)
    bad = int((~exact[clear]).sum())
    assert bad == 0, "%s: %d rows with a clear margin differ" % (what, bad)
    overlap = (idx[..., :, None] == want_idx[..., None, :]).any(-1).float().mean().item()
    print("%s: rows with clear margin %.1f%%, exact rows overall %.2f%%, id overlap %.4f"
          % (what, 100 * clear.float().mean().item(), 100 * exact.float().mean().item(), overlap), flush=True)
    assert overlap >= min_overlap, (what, overlap)
    return clear, exact
