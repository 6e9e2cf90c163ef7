"""Pins oracle.xattn_estimate / estimate_chunk_block_sums against a brute-force
fp64 softmax over brute-force antidiagonal scores, and against the invariants
the construction fixes (row mass, causal zeros, padded rows, chunk-size
independence without the torch-branch slice quirk)."""
import math

import pytest
import torch

from oracle import xattn_oracle as O


def brute_block_sums(q, k, S, bs, causal, real_q_rows=None, k_lo_of_row=None):
    """fp64: softmax over reshaped keys of the scaled antidiagonal scores,
    causal on reshaped positions (inclusive), summed into (bs/S)^2 tiles."""
    d = q.shape[-1]
    B, H, Lq, _ = q.shape
    Lk = k.shape[2]
    nq, nk, rbs = Lq // S, Lk // S, bs // S
    full = torch.einsum("bhqd,bhkd->bhqk", q.double(), k.double())
    s = torch.zeros(B, H, nq, nk, dtype=torch.float64)
    for i in range(S):
        s += full[:, :, (S - 1 - i) :: S, i::S]
    s = s / math.sqrt(d) / S
    off = nk - nq
    if causal:
        qi = torch.arange(nq)[:, None] + off
        ki = torch.arange(nk)[None, :]
        vis = ki <= qi
        if k_lo_of_row is not None:
            vis = vis & (ki >= k_lo_of_row[:, None])
        s = s.masked_fill(~vis, float("-inf"))
    p = torch.softmax(s, dim=-1)
    if real_q_rows is not None:
        p[:, :, real_q_rows:, :] = 0
    return p.view(B, H, nq // rbs, rbs, nk // rbs, rbs).sum(-1).sum(-2)


def make(L, H=2, d=16, seed=0, Lk=None):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(1, H, L, d, generator=g, dtype=torch.float64)
    k = torch.randn(1, H, Lk or L, d, generator=g, dtype=torch.float64)
    return q, k


@pytest.mark.parametrize("S", [4, 8, 16])
@pytest.mark.parametrize("causal", [True, False])
def test_single_chunk_matches_bruteforce(S, causal):
    bs, L = 32, 256
    q, k = make(L, seed=S)
    sums, mask = O.xattn_estimate(q, k, bs, S, threshold=0.9, chunk_size=L, causal=causal, pad0_quirk=False)
    want = brute_block_sums(q, k, S, bs, causal)
    assert sums.shape == (1, 2, L // bs, L // bs)
    assert torch.allclose(sums.double(), want, atol=1e-5)


def test_multi_chunk_no_quirk_equals_single_chunk_and_bruteforce():
    S, bs, L = 8, 32, 512
    q, k = make(L, seed=3)
    want = brute_block_sums(q, k, S, bs, True)
    for C in (128, 256, 512):
        sums, _ = O.xattn_estimate(q, k, bs, S, chunk_size=C, causal=True, pad0_quirk=False)
        assert torch.allclose(sums.double(), want, atol=1e-5), C


def test_pad0_quirk_restricts_later_chunks_to_their_own_keys():
    S, bs, L, C = 8, 32, 512, 128
    q, k = make(L, seed=4)
    sums, mask = O.xattn_estimate(q, k, bs, S, chunk_size=C, causal=True, pad0_quirk=True)
    rows = torch.arange(L // S)
    k_lo = (rows // (C // S)) * (C // S)
    want = brute_block_sums(q, k, S, bs, True, k_lo_of_row=k_lo)
    assert torch.allclose(sums.double(), want, atol=1e-5)
    bpc = C // bs
    for c in range(1, L // C):
        assert (sums[:, :, c * bpc : (c + 1) * bpc, : c * bpc] == 0).all()
        # only the forced sink survives selection in the invisible part
        assert not mask[:, :, c * bpc : (c + 1) * bpc, 1 : c * bpc].any()
        assert mask[:, :, c * bpc : (c + 1) * bpc, 0].all()


def test_quirk_vanishes_when_keys_are_padded():
    S, bs, C = 8, 32, 128
    q, k = make(200, seed=5)
    a, ma = O.xattn_estimate(q, k, bs, S, chunk_size=C, causal=True, pad0_quirk=True)
    b, mb = O.xattn_estimate(q, k, bs, S, chunk_size=C, causal=True, pad0_quirk=False)
    assert torch.equal(a, b) and torch.equal(ma, mb)


@pytest.mark.parametrize("causal", [True, False])
def test_padding_rows_keys_and_row_mass(causal):
    S, bs, C, L = 8, 32, 128, 200  # pad = 56 tokens = 7 reshaped rows
    q, k = make(L, seed=6)
    sums, mask = O.xattn_estimate(q, k, bs, S, chunk_size=C, causal=causal, pad0_quirk=False)
    Lp = 256
    qp = torch.nn.functional.pad(q, (0, 0, 0, Lp - L))
    kp = torch.nn.functional.pad(k, (0, 0, 0, Lp - L))
    real_rows = Lp // S - (Lp - L) // S
    want = brute_block_sums(qp, kp, S, bs, causal, real_q_rows=real_rows)
    assert torch.allclose(sums.double(), want, atol=1e-5)
    rbs = bs // S
    mass = sums.double().sum(-1)  # per q-block row
    full_rows = real_rows // rbs
    assert torch.allclose(mass[..., :full_rows], torch.full_like(mass[..., :full_rows], rbs), atol=1e-5)
    assert torch.allclose(mass[..., full_rows], torch.full_like(mass[..., full_rows], real_rows - full_rows * rbs), atol=1e-5)
    if causal:
        nb = Lp // bs
        upper = torch.triu(torch.ones(nb, nb, dtype=torch.bool), diagonal=1)
        assert (sums[:, :, upper] == 0).all()
    else:
        # zero-padded keys take part in the softmax with logit 0
        assert (sums[:, :, :full_rows, -1] > 0).all()


def test_kv_longer_than_q_offsets():
    S, bs, C = 8, 32, 128
    q, k = make(128, seed=8, Lk=384)
    sums, mask = O.xattn_estimate(q, k, bs, S, chunk_size=C, causal=True, pad0_quirk=False)
    want = brute_block_sums(q, k, S, bs, True)
    assert sums.shape == (1, 2, 4, 12)
    assert torch.allclose(sums.double(), want, atol=1e-5)
    # forced sink and bottom-right diagonal
    assert mask[..., 0].all()
    assert all(mask[0, :, r, 8 + r].all() for r in range(4))
    assert not any(mask[0, :, r, 8 + r + 1 :].any() for r in range(4))


def test_glue_tril_keep_sink_keep_recent():
    S, bs, L = 8, 32, 256
    q, k = make(L, seed=9)
    _, m = O.xattn_estimate(q, k, bs, S, threshold=0.9, chunk_size=128, causal=True)
    nb = L // bs
    upper = torch.triu(torch.ones(nb, nb, dtype=torch.bool), diagonal=1)
    assert not m[:, :, upper].any()
    assert m[..., 0].all() and torch.diagonal(m, dim1=-2, dim2=-1).all()
    _, ms = O.xattn_estimate(q, k, bs, S, threshold=0.0, chunk_size=128, causal=True, keep_sink=True)
    assert ms[:, :, 0, :].all()  # keep_sink sets q-block ROW 0 (Xattention.py:286-287)
    assert torch.equal(ms[:, :, 1:], O.xattn_estimate(q, k, bs, S, threshold=0.0, chunk_size=128, causal=True)[1][:, :, 1:])
    _, mr = O.xattn_estimate(q, k, bs, S, threshold=0.3, chunk_size=128, causal=False, keep_recent=True)
    assert torch.diagonal(mr, dim1=-2, dim2=-1).all()


def test_default_chunk_rule():
    table = {1024: 2048, 2048: 2048, 4096: 4096, 16384: 16384, 32768: 8192, 65536: 4096, 131072: 2048, 119056: 2048, 1 << 20: 2048}
    for L, want in table.items():
        assert O.default_chunk_size(L) == want, L
