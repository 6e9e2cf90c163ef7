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


def mask_mismatch_report(sums, got, want, tau, causal, diag_offset, blocks_per_chunk=None):
    """Compares two block masks given the block sums both were selected from.

    Returns (n_mismatch, n_outside_band).  A mismatching block is inside the band
    when the mass the selection rule compares against tau * total for it (or for
    a block of equal sum) is within TAU_BAND * total of tau * total - the only
    place where summation order or tie order can flip a decision.
    """
    sums = sums.double().cpu()
    got, want = got.cpu().bool(), want.cpu().bool()
    H, nq, nk = sums.shape
    bpc = blocks_per_chunk or nq
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
        one_forced = causal and diag_offset + (i // bpc) * bpc == 0
        forced = ({diag} if one_forced else {0, diag}) if causal else set()
        if causal and j > diag or j in forced:
            outside += 1
            continue
        base = sum(row[c].item() for c in forced if c < nk)
        limit = diag + 1 if causal else nk
        others = sorted(((row[c].item(), c) for c in range(limit) if c not in forced), key=lambda t: (-t[0], t[1]))
        need = taus[h].item() * total
        vj = row[j].item()
        ok = False
        run = base
        prev = 0.0
        for rank, (v, c) in enumerate(others):
            mass = (0.0 if rank == 0 else run - prev) if one_forced else run
            if v == vj and abs(mass - need) <= TAU_BAND * max(total, 1e-30):
                ok = True
            run += v
            prev = v
        if j == 0 and not ok:
            # column 0 is also set whenever any rank is left out: it flips with the last kept/left-out block
            ok = any(abs(((0.0 if r == 0 else base + sum(v for v, _ in others[:r]) - others[r - 1][0]) if one_forced
                          else base + sum(v for v, _ in others[:r])) - need) <= TAU_BAND * max(total, 1e-30)
                     for r in range(len(others)))
        if not ok:
            outside += 1
    return len(bad), outside
