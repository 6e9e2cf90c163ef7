"""Checker-side comparison of block masks: which mismatches the parity contract allows.

TEST INFRASTRUCTURE ONLY, like the rest of this package: imported by ``tests/``,
the smoke test and the benchmark's parity/CPU-baseline legs, never by the
product path.
"""
import torch

from . import xattn_oracle as O

TAU_BAND = 1e-5      # masks may differ only on blocks whose cumulative mass is this close to tau


def mask_mismatch_detail(sums, got, want, tau, causal, diag_offset, blocks_per_chunk=None, keep_recent=False):
    """Compares two block masks given the block sums both were selected from.

    Returns a dict: ``mismatches``; ``in_band`` - mismatching blocks for which the
    mass the selection rule compares against tau * total (for it or for a block of
    equal sum) is within TAU_BAND * total of tau * total, the only place where
    summation order can flip a decision (column 0 is also set whenever any rank is
    left out, so it may flip with whichever block sits at the crossing);
    ``ties`` - mismatching blocks that belong to a run of equal sums (equal to
    within TAU_BAND * total, the same tolerance) which the threshold crossing cuts
    through, with both masks keeping as many of them as the rule allows: which members of
    such a run are kept is the order an unstable sort happens to give (the
    reference uses torch.sort, xattn/src/utils.py:110,126,150) or, for sums that
    differ in the last bits, the order rounding gives; when causal, the zero sums of
    the blocks after the diagonal are members of a run of zeros too (the reference
    sorts whole rows and clears those blocks afterwards), so a pick may vanish there;
    ``outside`` - everything else, i.e. real disagreements.  Forced blocks and
    blocks beyond the diagonal are never excused.  ``keep_recent`` says that the
    masks were post-processed with the block diagonal forced
    (xattn/src/Xattention.py:288-297): without causality that column is an ordinary
    candidate of the selection that ends up set whether chosen or not, like column 0.
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
    outside = ties = 0
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
            # every column is a candidate of the reference's sort, blocks after the diagonal included: their
            # sums are zero, so they only ever matter as members of a run of zeros (they are cleared afterwards)
            cols = np.array([c for c in range(nk) if c not in forced], dtype=np.int64)
            vals = row[cols]
            order = np.lexsort((cols, -vals))          # descending sum, ascending column among equals
            vals, cols = vals[order], cols[order]
            base = float(sum(row[c] for c in forced if c < nk))
            csum = np.concatenate(([0.0], np.cumsum(vals)))             # csum[t] = the t largest ordinary sums
            if causal:
                # xattn/src/utils.py:107-141: the row is ranked by the sum for ordinary blocks and by
                # 100000 * (1 + sum) for forced ones; rank r is judged against M(r), M(0) = M(1) = 0,
                # M(r) = forced sum + the r - 2 largest ordinary sums.  The i-th ordinary block sits at rank
                # i + (forced keys not below its own): i + 2 as a rule, i + 1 where only the diagonal is forced
                fkeys = [100000.0 * (1.0 + row[c]) for c in forced if c < nk]
                rank = np.arange(len(vals)) + np.array([sum(1 for f in fkeys if not v > f) for v in vals], dtype=np.int64)
                before = np.where(rank < 2, 0.0, base + csum[np.maximum(rank - 2, 0)])
            else:
                before = csum[:-1]
            need = taus[h].item() * total
            near = np.abs(before - need) <= TAU_BAND * max(total, 1e-30)
            rows[(h, i)] = (row, vals, cols, near, before < need)
        row, vals, cols, near, keep = rows[(h, i)]
        same = np.abs(vals - row[j]) <= TAU_BAND * max(float(row.sum()), 1e-30)
        if bool((near & same).any()) or (j == 0 and bool(near.any())):
            continue
        run = cols[same]
        kept = int(keep[same].sum())
        cut = 0 < kept < len(run)
        if cut:
            # any `kept` members of the run may be the chosen ones; column 0, when it is a member, is set
            # anyway (unselected ranks scatter to it), and so is the diagonal under keep_recent: a mask may
            # show one chosen member fewer beside each such member
            free = [c for c in ([0, diag] if keep_recent and not causal else [0]) if c in run]
            visible = run[run <= diag] if causal else run
            rest = visible[~np.isin(visible, free)]
            # picks that land on members after the diagonal are cleared again and show nowhere
            counts = set(range(max(0, kept - len(free) - (len(run) - len(visible))), kept + 1))
            ok = all(int(m[h, i][rest].sum()) in counts and all(bool(m[h, i][c]) for c in free) for m in (got, want))
            if ok:
                ties += 1
                continue
        outside += 1
    return {"mismatches": len(bad), "in_band": len(bad) - outside - ties, "ties": ties, "outside": outside}


def mask_mismatch_report(sums, got, want, tau, causal, diag_offset, blocks_per_chunk=None, keep_recent=False):
    """(number of mismatching blocks, number of them that the parity contract does
    not excuse) - see :func:`mask_mismatch_detail`."""
    d = mask_mismatch_detail(sums, got, want, tau, causal, diag_offset, blocks_per_chunk, keep_recent)
    return d["mismatches"], d["outside"]


def head_mask_parity(q, k, head, got_mask, stride, threshold, chunk_size, causal, pad0_quirk, sums_got=None,
                     return_mask=False):
    """Runs the oracle's estimate for ONE query head on the host, in fp32, on the
    values ``q``/``k`` hold (any dtype/device; K may carry fewer heads), and
    compares its block mask with ``got_mask`` (that head's ``[Nq_p, Nk_p]`` mask
    from the path under test).

    Returns a dict: blocks, mismatches, in_band and ties (mismatches the contract
    allows), outside_band, density of the oracle's mask over the padded grid
    and, when ``sums_got`` is given, the largest absolute difference of the
    block sums; with ``return_mask`` also the oracle's mask for the head
    (``oracle_mask``, bool ``[Nq_p, Nk_p]``).
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
    d = mask_mismatch_detail(want_sums[0], got, want_mask[0], tau, causal, nk_p - nq_p, chunk_size // 128)
    rep = {"head": int(head), "blocks": int(want_mask.numel()), "mismatches": d["mismatches"], "in_band": d["in_band"],
           "ties": d["ties"], "outside_band": d["outside"], "oracle_density": round(float(want_mask.float().mean()), 5)}
    if sums_got is not None:
        rep["sums_max_abs_diff"] = float((sums_got.detach().float().cpu().reshape(nq_p, nk_p) - want_sums[0, 0]).abs().max())
    if return_mask:
        rep["oracle_mask"] = want_mask[0, 0].clone()
    return rep
