"""Pins oracle.find_blocks_chunked: golden vectors from the reference's own
xattn/src/utils.py (tests/golden/find_blocks_golden.pt), an independent
brute-force enumeration, and selection properties."""
import os

import pytest
import torch

from oracle import xattn_oracle as O

GOLD = os.path.join(os.path.dirname(__file__), "golden", "find_blocks_golden.pt")


def load_cases():
    return torch.load(GOLD, weights_only=True)


def test_golden_vectors_from_reference():
    cases = load_cases()
    assert len(cases) >= 20
    for c in cases:
        tau = c["threshold"] if c["threshold_is_tensor"] else float(c["threshold"])
        got = O.find_blocks_chunked(
            c["x"].clone(), c["current_index"], tau, None, decoding=False, mode="prefill", causal=c["causal"]
        )
        assert got.dtype == torch.bool
        assert torch.equal(got, c["mask"]), c["name"]


def brute_select_row(vals, tau, causal, diag, limit, first_diag=1):
    """Sorted-prefix enumeration for one row, written from the rule rather than
    the tensor program: forced = {0, diag} (only {diag} in a chunk whose first
    diagonal is column 0, where eye() overwrites the sink, utils.py:100-106);
    visit the rest by descending value and keep a block while the mass gathered
    before it is below tau*total; unselected ranks land on column 0."""
    n = len(vals)
    total = sum(vals)
    need = total * tau
    keep = [False] * n
    if causal:
        forced = sorted({0, diag}) if first_diag != 0 else [diag]
        mass = 0.0
        for f in forced:
            keep[f] = True
            mass += vals[f]
        rest = sorted((i for i in range(n) if i not in forced), key=lambda i: -vals[i])
        extra = 1 if len(forced) == 1 else 0  # one-slot-longer prefix, utils.py:115-124
        gathered = []
        for rank, i in enumerate(rest):
            before = 0.0 if rank < extra else mass + sum(gathered[: rank - extra])
            if before < need:
                keep[i] = True
            else:
                keep[0] = True  # scatter of unselected ranks, utils.py:142
            gathered.append(vals[i])
        for i in range(limit, n):
            keep[i] = False
    else:
        order = sorted(range(n), key=lambda i: -vals[i])
        mass = 0.0
        dropped = False
        for i in order:
            if mass < need:
                keep[i] = True
            else:
                dropped = True
            mass += vals[i]
        if dropped:
            keep[0] = True  # unselected ranks are scattered to column 0, utils.py:164
    return keep


@pytest.mark.parametrize("causal,cur", [(True, 8), (True, 0), (False, 0)])
@pytest.mark.parametrize("tau", [0.0, 0.5, 0.9, 1.0])
def test_bruteforce_enumeration(causal, cur, tau):
    g = torch.Generator().manual_seed(int(tau * 100) + causal + cur)
    rows, cols = 6, 14
    x = torch.rand(1, 2, rows, cols, generator=g, dtype=torch.float64) + 0.01
    if causal:
        for r in range(rows):
            x[:, :, r, cur + r + 1 :] = 0
    got = O.find_blocks_chunked(x, cur, tau, None, decoding=False, mode="prefill", causal=causal)
    for h in range(2):
        for r in range(rows):
            vals = x[0, h, r].tolist()
            want = brute_select_row(vals, tau, causal, cur + r, cur + rows, first_diag=cur)
            if causal and (tau == 1.0 or cur == 0):
                # zero-valued future blocks tie; compare only the causal part
                want, have = want[: cur + r + 1], got[0, h, r, : cur + r + 1].tolist()
            else:
                have = got[0, h, r].tolist()
            assert have == want, (h, r)


def test_selection_properties():
    g = torch.Generator().manual_seed(7)
    rows, cols, cur = 8, 16, 8
    x = torch.rand(1, 4, rows, cols, generator=g, dtype=torch.float64) ** 2 + 1e-3
    for r in range(rows):
        x[:, :, r, cur + r + 1 :] = 0
    prev = None
    for tau in (0.0, 0.2, 0.5, 0.8, 0.95):
        m = O.find_blocks_chunked(x, cur, tau, None, decoding=False, mode="prefill", causal=True)
        # forced sink + diagonal
        assert m[..., 0].all()
        assert all(m[0, :, r, cur + r].all() for r in range(rows))
        # reaches the required mass
        got = torch.where(m, x, 0.0).sum(-1)
        assert (got >= tau * x.sum(-1) - 1e-12).all()
        # minimality: dropping the smallest selected non-forced block falls below
        for h in range(4):
            for r in range(rows):
                sel = [c for c in range(cols) if m[0, h, r, c] and c not in (0, cur + r)]
                if sel:
                    smallest = min(sel, key=lambda c: x[0, h, r, c].item())
                    assert got[0, h, r] - x[0, h, r, smallest] < tau * x[0, h, r].sum()
        # monotone in tau
        if prev is not None:
            assert (m | ~prev).all()
        prev = m
    m0 = O.find_blocks_chunked(x, cur, 0.0, None, decoding=False, mode="prefill", causal=True)
    assert m0.sum().item() == 4 * rows * 2  # tau=0 -> forced blocks only


def test_per_head_threshold_broadcast():
    g = torch.Generator().manual_seed(9)
    x = torch.rand(1, 3, 4, 12, generator=g, dtype=torch.float64)
    taus = torch.tensor([0.2, 0.7, 0.95], dtype=torch.float32)
    m = O.find_blocks_chunked(x, 0, taus, None, decoding=False, mode="prefill", causal=False)
    for h in range(3):
        mh = O.find_blocks_chunked(
            x[:, h : h + 1], 0, float(taus[h].double()), None, decoding=False, mode="prefill", causal=False
        )
        assert torch.equal(m[:, h : h + 1], mh)


def test_create_causal_mask_against_a_loop_and_the_product_helper():
    """xattn/src/utils.py:3-42: row r of block d sees every earlier block and columns <= r of its own."""
    from xattn.src.utils import create_causal_mask

    for bs, nb, d in [(4, 3, 0), (4, 3, 1), (4, 3, 2), (8, 1, 0), (2, 5, 3)]:
        m = O.create_causal_mask(2, 3, bs, nb, d)
        assert m.shape == (2, 3, bs, bs * nb)
        for r in range(bs):
            for c in range(bs * nb):
                want = 0.0 if c <= d * bs + r else float("-inf")
                assert m[1, 2, r, c].item() == want, (bs, nb, d, r, c)
        assert torch.equal(create_causal_mask(2, 3, bs, nb, d, device="cpu"), m)
    for bad in (-1, 3):
        with pytest.raises(ValueError):
            O.create_causal_mask(1, 1, 4, 3, bad)
        with pytest.raises(ValueError):
            create_causal_mask(1, 1, 4, 3, bad, device="cpu")


def test_decode_mode_of_find_blocks_chunked():
    """xattn/src/utils.py:71-86: no selection; the causal form is a join of row slices along the
    column axis, which has a shape only when the slices have equally many rows."""
    from xattn.src.utils import find_blocks_chunked

    x = torch.rand(1, 2, 4, 6)
    for f in (O.find_blocks_chunked, find_blocks_chunked):
        assert f(x, 1, 0.9, None, decoding=False, mode="decode", causal=False).all()
        m = f(x, 1, 0.9, None, decoding=False, mode="decode", causal=True)       # rows 0..1 | rows 2..3
        assert m.shape == (1, 2, 2, 12) and m[..., :6].all() and not m[..., 6:].any()
        with pytest.raises(RuntimeError):
            f(x, 0, 0.9, None, decoding=False, mode="decode", causal=True)         # 1 row against 3
        assert f(x, 0, 0.9, None, decoding=True, mode="prefill").all()


def test_sums_beyond_a_forced_key_move_up_in_rank():
    """Hand-worked: the reference ranks forced blocks by 100000 * (1 + sum) and the rest by their sum
    (xattn/src/utils.py:126-130); rank r is kept while M(r) < tau * total with M = cumsum([0, 0, forced_sum,
    others...]) (:115-141).  Un-normalised sums (softmax=False) can exceed a forced key.  Row with sink 10,
    diagonal 50 (keys 1.1e6 and 5.1e6) and others 5e6, 3e6, 2: order [diag, 5e6, 3e6, sink, 2], masses
    [0, 0, 60, 60 + 5e6, ...] against 0.5 * 8000062: both big blocks are kept - with the forced blocks ranked
    first the second one (mass 60 + 5e6) would not be."""
    x = torch.zeros(1, 1, 1, 8, dtype=torch.float32)
    x[0, 0, 0, :5] = torch.tensor([10.0, 5e6, 3e6, 2.0, 50.0])
    want = O.find_blocks_chunked(x, 4, 0.5, None, decoding=False, mode="prefill", causal=True)[0, 0, 0]
    assert want.tolist() == [True, True, True, False, True, False, False, False]
    # below 100000 nothing changes rank: sink 10, diagonal 50, others 90, 30, 2 (total 182, need 91): the first
    # other is judged against 60, the second against 150
    y = torch.zeros(1, 1, 1, 8, dtype=torch.float32)
    y[0, 0, 0, :5] = torch.tensor([10.0, 90.0, 30.0, 2.0, 50.0])
    got = O.find_blocks_chunked(y, 4, 0.5, None, decoding=False, mode="prefill", causal=True)[0, 0, 0]
    assert got.tolist() == [True, True, False, False, True, False, False, False]
    # a sum beyond BOTH keys takes rank 0: sink 1, diagonal 2 (keys 2e5, 3e5), others 4e5, 3.5e5, 1e5, 9e4
    # order [4e5, 3.5e5, diag, sink, 1e5, 9e4]; masses [0, 0, 3, 3 + 4e5, 3 + 7.5e5, ...]; need 0.85 * 940003
    z = torch.zeros(1, 1, 1, 8, dtype=torch.float32)
    z[0, 0, 0, :6] = torch.tensor([1.0, 4e5, 3.5e5, 1e5, 9e4, 2.0])
    got = O.find_blocks_chunked(z, 5, 0.85, None, decoding=False, mode="prefill", causal=True)[0, 0, 0]
    assert got.tolist() == [True, True, True, True, False, True, False, False]
