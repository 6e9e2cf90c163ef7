"""Shared helpers of the GPU parity tests (HIP path vs the CPU oracle)."""
import torch

OUT_MAX_ABS = 2e-2   # bf16 attention output, max-abs tolerance of the parity contract
OUT_MEAN_ABS = 5e-3  # ... and mean-abs
TAU_BAND = 1e-5      # masks may differ only on blocks whose cumulative mass is this close to tau


def lists_from_mask(mask):
    """bool [H, Nq, Nk] -> (col_idx int32 [H, Nq, Nk], col_cnt int32 [H, Nq]), ascending columns."""
    H, nq, nk = mask.shape
    order = torch.argsort((~mask).to(torch.int8), dim=-1, stable=True).to(torch.int32)
    cnt = mask.sum(-1).to(torch.int32)
    return order.contiguous(), cnt.contiguous()


def mask_mismatch_report(sums, got, want, tau, causal, diag_offset):
    """Compares two block masks given the block sums both were selected from.

    Returns (n_mismatch, n_outside_band): a mismatching block is inside the band
    when the mass gathered before it (forced blocks + larger blocks), or before
    its successor, is within TAU_BAND * total of tau * total.
    """
    sums = sums.double().cpu()
    got, want = got.cpu().bool(), want.cpu().bool()
    H = sums.shape[0]
    taus = tau if isinstance(tau, torch.Tensor) else torch.full((H,), float(tau), dtype=torch.float64)
    taus = taus.double().cpu().reshape(-1)
    if taus.numel() == 1:
        taus = taus.expand(H)
    bad = (got != want).nonzero().tolist()
    outside = 0
    for h, i, j in bad:
        row = sums[h, i]
        total = row.sum().item()
        diag = i + diag_offset
        forced = {0, diag} if causal else set()
        if causal and j > diag:
            outside += 1
            continue
        base = sum(row[c].item() for c in forced if c < row.numel())
        others = [(row[c].item(), c) for c in range(row.numel()) if c not in forced]
        bigger = sum(v for v, c in others if v > row[j].item())
        ties = sum(v for v, c in others if v == row[j].item())
        lo, hi = base + bigger, base + bigger + ties
        need = taus[h].item() * total
        if not (lo - TAU_BAND * total <= need <= hi + TAU_BAND * total):
            outside += 1
    return len(bad), outside
