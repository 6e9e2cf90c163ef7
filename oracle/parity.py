"""Checker-side comparison of block masks: which mismatches the parity contract allows.

TEST INFRASTRUCTURE ONLY, like the rest of this package: imported by ``tests/``,
the smoke test and the benchmark's parity/CPU-baseline legs, never by the
product path.
"""
import torch

from . import xattn_oracle as O

TAU_BAND = 1e-5      # masks may differ only on blocks whose cumulative mass is this close to tau


def mask_mismatch_report(sums, got, want, tau, causal, diag_offset, blocks_per_chunk=None):
    """Compares two block masks given the block sums both were selected from.

    Returns (n_mismatch, n_outside_band).  A mismatching block is inside the band
    when the mass the selection rule compares against tau * total for it (or for
    a block of equal sum) is within TAU_BAND * total of tau * total - the only
    place where summation order or tie order can flip a decision.  Column 0 is
    also set whenever any rank is left out, so it may flip with whichever block
    sits at the crossing.  Forced blocks and blocks beyond the diagonal are
    never inside the band.
    """
    import numpy as np

    sums = sums.double().cpu().numpy()
    got, want = got.cpu().bool(), want.cpu().bool()
    H, nq, nk = sums.shape
    bpc = blocks_per_chunk or nq
    taus = tau if isinstance(tau, torch.Tensor) else torch.full((H,), float(tau), dtype=torch.float64)
    taus = taus.double().cpu().reshape(-1)
    if taus.numel() == 1:
        taus = taus.expand(H)
    bad = (got != want).nonzero().tolist()
    outside = 0
    rows = {}
    for h, i, j in bad:
        diag = i + diag_offset
        one_forced = causal and diag_offset + (i // bpc) * bpc == 0
        forced = ({diag} if one_forced else {0, diag}) if causal else set()
        if (causal and j > diag) or j in forced:
            outside += 1
            continue
        if (h, i) not in rows:
            row = sums[h, i]
            total = float(row.sum())
            limit = min(diag + 1, nk) if causal else nk
            cols = np.array([c for c in range(limit) if c not in forced], dtype=np.int64)
            vals = row[cols]
            order = np.lexsort((cols, -vals))          # descending sum, ascending column among equals
            vals = vals[order]
            base = float(sum(row[c] for c in forced if c < nk))
            before = base + np.concatenate(([0.0], np.cumsum(vals)[:-1])) if len(vals) else np.zeros(0)
            if one_forced and len(vals):
                before = before - np.concatenate(([0.0], vals[:-1]))
                before[0] = 0.0
            near = np.abs(before - taus[h].item() * total) <= TAU_BAND * max(total, 1e-30)
            rows[(h, i)] = (row, vals, near)
        row, vals, near = rows[(h, i)]
        ok = bool((near & (vals == row[j])).any()) or (j == 0 and bool(near.any()))
        if not ok:
            outside += 1
    return len(bad), outside


def head_mask_parity(q, k, head, got_mask, stride, threshold, chunk_size, causal, pad0_quirk, sums_got=None):
    """Runs the oracle's estimate for ONE query head on the host, in fp32, on the
    values ``q``/``k`` hold (any dtype/device; K may carry fewer heads), and
    compares its block mask with ``got_mask`` (that head's ``[Nq_p, Nk_p]`` mask
    from the path under test).

    Returns a dict: blocks, mismatches, in_band (mismatches the contract
    allows), outside_band, density of the oracle's mask over the padded grid
    and, when ``sums_got`` is given, the largest absolute difference of the
    block sums.
    """
    H, Hkv = q.shape[1], k.shape[1]
    kv = head // (H // Hkv)
    qh = q[:, head : head + 1].detach().float().cpu()
    kh = k[:, kv : kv + 1].detach().float().cpu()
    tau = threshold
    if isinstance(tau, torch.Tensor):
        tau = tau.detach().cpu().reshape(-1)
        tau = tau[head : head + 1] if tau.numel() > 1 else tau
    want_sums, want_mask = O.xattn_estimate(qh, kh, 128, stride, threshold=tau, chunk_size=chunk_size,
                                            causal=causal, pad0_quirk=pad0_quirk)
    nq_p, nk_p = want_mask.shape[2], want_mask.shape[3]
    got = got_mask.reshape(1, nq_p, nk_p)
    nbad, outside = mask_mismatch_report(want_sums[0], got, want_mask[0], tau, causal, nk_p - nq_p, chunk_size // 128)
    rep = {"head": int(head), "blocks": int(want_mask.numel()), "mismatches": int(nbad), "in_band": int(nbad - outside),
           "outside_band": int(outside), "oracle_density": round(float(want_mask.float().mean()), 5)}
    if sums_got is not None:
        rep["sums_max_abs_diff"] = float((sums_got.detach().float().cpu().reshape(nq_p, nk_p) - want_sums[0, 0]).abs().max())
    return rep
