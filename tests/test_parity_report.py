"""CPU: the band report the mask-parity tests rely on must flag flips away from
the threshold crossing and tolerate flips at it."""
import torch

from oracle import xattn_oracle as O
from oracle.parity import TAU_BAND, head_mask_parity, mask_mismatch_detail, mask_mismatch_report


def _row_case(causal):
    # one head, 4 q-block rows over 8 columns (k_len > q_len by 4 blocks when causal)
    g = torch.Generator().manual_seed(3)
    x = torch.rand(1, 4, 8, generator=g, dtype=torch.float64) + 0.05
    off = 4
    if causal:
        x = x * (torch.arange(8)[None, :] <= torch.arange(4)[:, None] + off)
    want = O.find_blocks_chunked(x[None].float(), off, 0.6, None, decoding=False, mode="prefill", causal=causal)[0]
    if causal:
        want &= torch.arange(8)[None, :] <= torch.arange(4)[:, None] + off
    return x.float(), want, off


def test_flip_far_from_the_crossing_is_outside_the_band():
    for causal in (True, False):
        x, want, off = _row_case(causal)
        assert mask_mismatch_report(x, want, want, 0.6, causal, off) == (0, 0)
        # the largest non-forced block of row 2 is kept long before the crossing: dropping it is a real error
        row = x[0, 2].clone()
        if causal:
            row[0] = row[2 + off] = -1
        j = int(row.argmax())
        got = want.clone()
        assert got[0, 2, j]
        got[0, 2, j] = False
        assert mask_mismatch_report(x, got, want, 0.6, causal, off) == (1, 1)
        if causal:   # forced blocks and blocks beyond the diagonal are never excused
            got = want.clone()
            got[0, 1, 1 + off] = False
            got[0, 0, 7] = True
            assert mask_mismatch_report(x, got, want, 0.6, causal, off) == (2, 2)


def test_flip_at_the_crossing_is_inside_the_band():
    # non-causal row [4, 3, 2, 1] (total 10): mass before the third block is 7 -> with tau = 0.7 the decision
    # "7 < 7" sits exactly on the threshold; a path that sees 6.9999999 keeps the block
    x = torch.tensor([[[4.0, 3.0, 2.0, 1.0]]])
    want = O.find_blocks_chunked(x[None], 0, 0.7, None, decoding=False, mode="prefill", causal=False)[0]
    assert want[0, 0].tolist() == [True, True, False, False]
    got = want.clone()
    got[0, 0, 2] = True
    assert mask_mismatch_report(x, got, want, 0.7, False, 0) == (1, 0)
    got[0, 0, 3] = True                      # the last block is a full unit of mass past the crossing
    assert mask_mismatch_report(x, got, want, 0.7, False, 0) == (2, 1)
    # shifting the threshold by more than the band makes the same flip an error
    tau = 0.7 - 3 * TAU_BAND
    want2 = O.find_blocks_chunked(x[None], 0, tau, None, decoding=False, mode="prefill", causal=False)[0]
    got2 = want2.clone()
    got2[0, 0, 2] = True
    assert mask_mismatch_report(x, got2, want2, tau, False, 0) == (1, 1)


def test_head_mask_parity_runs_one_head_of_a_grouped_layout():
    g = torch.Generator().manual_seed(0)
    q = torch.randn(1, 4, 512, 128, generator=g).bfloat16()
    k = torch.randn(1, 2, 512, 128, generator=g).bfloat16()
    sums, mask = O.xattn_estimate(q.float(), k.repeat_interleave(2, 1).float(), 128, 8, threshold=0.9, chunk_size=256,
                                  pad0_quirk=False)
    for h in range(4):
        rep = head_mask_parity(q, k, h, mask[0, h], 8, 0.9, 256, True, False, sums_got=sums[0, h])
        assert rep["mismatches"] == 0 and rep["blocks"] == 16 and rep["sums_max_abs_diff"] < 1e-5
    wrong = mask[0, 3].clone()
    wrong[3, 3] = False                       # a forced diagonal block
    assert head_mask_parity(q, k, 3, wrong, 8, 0.9, 256, True, False)["outside_band"] == 1
    taus = torch.tensor([0.5, 0.9, 0.7, 0.99])
    _, m2 = O.xattn_estimate(q.float(), k.repeat_interleave(2, 1).float(), 128, 8, threshold=taus, chunk_size=256,
                             pad0_quirk=False)
    assert head_mask_parity(q, k, 2, m2[0, 2], 8, taus, 256, True, False)["mismatches"] == 0


def test_ties_cut_by_the_crossing_are_excused_only_when_the_counts_agree():
    # row [5, 1, 1, 1, 1, 1] (total 10), tau 0.65: need 6.5 -> the 5 and two of the five equal blocks are kept;
    # WHICH two is the sort's business
    x = torch.tensor([[[5.0, 1.0, 1.0, 1.0, 1.0, 1.0]]])
    want = O.find_blocks_chunked(x[None], 0, 0.65, None, decoding=False, mode="prefill", causal=False)[0]
    assert int(want.sum()) == 3 and want[0, 0, 0]
    got = torch.tensor([[[True, False, False, True, False, True]]])
    if not torch.equal(got, want):
        d = mask_mismatch_detail(x, got, want, 0.65, False, 0)
        assert d["outside"] == 0 and d["ties"] == d["mismatches"] > 0
    three = torch.tensor([[[True, True, True, True, False, False]]])       # one too many of the run
    assert mask_mismatch_detail(x, three, want, 0.65, False, 0)["outside"] > 0
    dropped = want.clone()
    dropped[0, 0, 0] = False                                                  # the big block is not part of any run
    assert mask_mismatch_detail(x, dropped, want, 0.65, False, 0)["outside"] == 1


def _first_chunk_row(vals, want, got, tau):
    """One causal q-block row of the first query chunk (the diagonal is the last listed value)."""
    diag = len(vals) - 1
    x = torch.zeros(1, diag + 1, 32)
    x[0, diag, : len(vals)] = torch.tensor(vals)
    w = torch.zeros(1, diag + 1, 32, dtype=torch.bool)
    g = w.clone()
    w[0, diag, : len(want)] = torch.tensor(want).bool()
    g[0, diag, : len(got)] = torch.tensor(got).bool()
    return mask_mismatch_detail(x, g, w, tau, True, 0, 32)


def test_column_zero_comes_free_with_a_cut_run():
    """Rows of exactly equal sums (uniform attention of zero-padded queries): in the first query chunk
    column 0 is set whenever a rank is left out, so a selection that spent one of its picks on column 0
    shows one block fewer than one that did not; both are outcomes of the reference's unstable sort."""
    v = [2.12759852] * 7 + [1.10680962]
    d = _first_chunk_row(v, [1, 1, 1, 1, 1, 1, 0, 1], [1, 1, 1, 1, 1, 0, 0, 1], 0.5)
    assert d == {"mismatches": 1, "in_band": 0, "ties": 1, "outside": 0}
    d = _first_chunk_row(v, [1, 1, 1, 1, 1, 1, 0, 1], [1, 1, 1, 1, 0, 0, 0, 1], 0.5)     # two fewer: an error
    assert d["outside"] == 2
    d = _first_chunk_row([0.43079475] * 16 + [0.10728443], [1] * 8 + [0] + [1] * 8, [1] * 14 + [0, 0, 1], 0.8)
    assert d["outside"] == 0 and d["ties"] == 3
    # the oracle itself lands on one of the allowed outcomes
    x = torch.zeros(1, 1, 8, 32)
    x[0, 0, 7, :8] = torch.tensor(v)
    for r in range(7):
        x[0, 0, r, : r + 1] = 1.0
    want = O.find_blocks_chunked(x, 0, 0.5, None, decoding=False, mode="prefill", causal=True)[0]
    lowest = torch.zeros(32, dtype=torch.bool)
    lowest[[0, 1, 2, 3, 4, 7]] = True
    got = want.clone()
    got[0, 7] = lowest
    assert mask_mismatch_detail(x[0], got, want, 0.5, True, 0, 32)["outside"] == 0


def test_forced_diagonal_of_keep_recent_comes_free_without_causality():
    """Non-causal row of six equal sums, tau 0.45: three are chosen (which three is the sort's business), then
    keep_recent sets the diagonal (here column 4) and column 0 is set because ranks were left out.  A mask
    whose picks include those columns shows fewer blocks than one whose picks avoid them."""
    x = torch.ones(1, 1, 6)
    picks_low = torch.tensor([[[True, True, True, False, True, False]]])      # picks 0,1,2; diagonal 4 forced
    picks_mid = torch.tensor([[[True, True, True, True, True, False]]])       # picks 1,2,3; columns 0 and 4 come free
    picks_hit = torch.tensor([[[True, True, False, False, True, False]]])     # picks 0,1,4: both free columns used up
    for a in (picks_low, picks_mid, picks_hit):
        for b in (picks_low, picks_mid, picks_hit):
            d = mask_mismatch_detail(x, a, b, 0.45, False, 4, keep_recent=True)
            assert d["outside"] == 0 and d["ties"] == d["mismatches"]
    # without the flag the diagonal is an ordinary member of the run and the counts no longer agree
    assert mask_mismatch_detail(x, picks_hit, picks_mid, 0.45, False, 4)["outside"] > 0
    too_few = torch.tensor([[[True, False, False, False, True, False]]])      # only the free columns
    assert mask_mismatch_detail(x, too_few, picks_mid, 0.45, False, 4, keep_recent=True)["outside"] > 0
    # the oracle's own post-processed mask is one of the allowed outcomes
    want = O.find_blocks_chunked(x[None], 0, 0.45, None, decoding=False, mode="prefill", causal=False)[0]
    want[0, 0, 4] = True
    assert mask_mismatch_detail(x, picks_low, want, 0.45, False, 4, keep_recent=True)["outside"] == 0


def test_a_pick_among_zero_sums_may_land_after_the_diagonal():
    """First query chunk, row 2 of a 6-column grid, sums [a, 0, 0 | 0, 0, 0]: the rule keeps the diagonal, column 0
    and ONE of the zero-sum blocks; the reference sorts all six columns, so that pick is column 1 or one of the
    three blocks after the diagonal, which are cleared afterwards.  Both outcomes are the reference's."""
    x = torch.zeros(1, 3, 6)
    x[0, 0, 0] = 1.0
    x[0, 1, :2] = torch.tensor([0.5, 0.5])
    x[0, 2, 0] = 0.0645
    a = torch.zeros(1, 3, 6, dtype=torch.bool)
    a[0, 0, 0] = a[0, 1, 0] = a[0, 1, 1] = True
    b = a.clone()
    a[0, 2, :3] = torch.tensor([True, True, True])       # the pick landed on column 1
    b[0, 2, :3] = torch.tensor([True, False, True])      # ... or after the diagonal
    d = mask_mismatch_detail(x, a, b, 0.5, True, 0, 3)
    assert d == {"mismatches": 1, "in_band": 0, "ties": 1, "outside": 0}
    # the oracle's own answer is one of the two
    want = O.find_blocks_chunked(x[None], 0, 0.5, None, decoding=False, mode="prefill", causal=True)[0]
    want &= torch.arange(6)[None, :] <= torch.arange(3)[:, None]
    assert mask_mismatch_detail(x, a, want, 0.5, True, 0, 3)["outside"] == 0
    assert mask_mismatch_detail(x, b, want, 0.5, True, 0, 3)["outside"] == 0
    # keeping BOTH zero-sum candidates of a longer row is one pick too many
    x2 = torch.zeros(1, 4, 6)
    x2[0, 3, 0] = 0.0645
    w2 = torch.zeros(1, 4, 6, dtype=torch.bool)
    w2[0, 3, [0, 1, 3]] = True
    g2 = w2.clone()
    g2[0, 3, 2] = True
    assert mask_mismatch_detail(x2, g2, w2, 0.5, True, 0, 4)["outside"] == 1
