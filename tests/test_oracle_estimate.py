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


def loop_block_sums(q, k, S, bs, C, causal, *, kdb=1, norm=1.0, triton=False):
    """Row-by-row restatement (python loops, fp64) of what the reference computes
    per query chunk, written from the definitions rather than from tensor masks:

    query row j of the padded, reshaped sequence stands for reshaped row ``j*kdb``
    (tokens ``j*kdb*S + S-1-i``); when causal it sees reshaped keys up to position
    ``j*kdb + kdb-1 + off`` (xattn/src/Xattention.py:204-222), zero-padded keys
    included; the torch branch zeroes the last
    ``q_pad_r // kdb`` rows of the last chunk (:237-238), the Triton branch the
    rows whose key-axis position is at or beyond the real reshaped key length
    (xattn/src/kernels.py:70, Xattention.py:169); a q-block sums ``rbs // kdb`` rows."""
    d = q.shape[-1]
    B, H, Lq, _ = q.shape
    Lk = k.shape[2]
    q_pad, k_pad = -Lq % C, -Lk % C
    qp = torch.nn.functional.pad(q.double(), (0, 0, 0, q_pad))
    kp = torch.nn.functional.pad(k.double(), (0, 0, 0, k_pad))
    n_rq, n_rk = (Lq + q_pad) // S, (Lk + k_pad) // S
    rbs, rcs = bs // S, C // S
    off = n_rk - n_rq
    rows = n_rq // kdb
    rq_blk = rbs // kdb
    out = torch.zeros(B, H, n_rq // rbs, n_rk // rbs, dtype=torch.float64)
    q_pad_r, k_pad_r = q_pad // S, k_pad // S
    last_chunk_first_row = (n_rq - rcs) // kdb
    for h in range(H):
        for j in range(rows):
            m = j * kdb
            s = torch.zeros(n_rk, dtype=torch.float64)
            for i in range(S):
                s += kp[0, h, i::S] @ qp[0, h, m * S + S - 1 - i]
            s = s / math.sqrt(d) / S / norm
            if causal:
                vis = torch.arange(n_rk) <= m + kdb - 1 + off
                # zero-padded keys are NOT hidden: the -inf the torch branch writes over them (:201) is
                # overwritten by the triangle of the row's own chunk (:203-214), the only chunk whose rows
                # reach them; they enter the softmax with logit 0 for every row at or beyond their position
                if not triton and not k_pad_r:
                    # the slice [..., -0:] of Xattention.py:201 hides every key before the row's own chunk
                    vis &= torch.arange(n_rk) >= (m // rcs) * rcs + off
                s = s.masked_fill(~vis, float("-inf"))
            if triton:
                zero = m + off >= n_rk - k_pad_r
            else:
                nz = q_pad_r // kdb
                zero = q_pad_r != 0 and (j >= rows - nz if nz else j >= last_chunk_first_row)
            if zero:
                continue
            p = torch.softmax(s, dim=0)
            out[0, h, j // rq_blk] += p.view(n_rk // rbs, rbs).sum(-1)
    return out


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("kdb,S,L", [(2, 8, 512), (4, 8, 512), (2, 4, 200), (4, 16, 1024), (2, 8, 456), (4, 8, 508)])
def test_kdb_matches_row_loops(kdb, S, L, causal):
    """Query-row subsampling of the torch branch (Xattention.py:76-83,174-181,217-222,245)."""
    bs, C = 128, 256
    q, k = make(L, H=1, seed=20 + kdb + S)
    sums, mask = O.xattn_estimate(q, k, bs, S, threshold=0.9, chunk_size=C, causal=causal, kdb=kdb, pad0_quirk=True)
    want = loop_block_sums(q, k, S, bs, C, causal, kdb=kdb)
    assert sums.shape == want.shape
    assert torch.allclose(sums.double(), want, atol=1e-5), (sums.double() - want).abs().max()
    rbs = bs // S
    full_rows = L // bs
    if L % C == 0:
        assert torch.allclose(sums.double().sum(-1)[..., :full_rows], torch.full((1, 1, full_rows), rbs / kdb, dtype=torch.float64), atol=1e-5)


def test_kdb_is_refused_with_the_triton_branch():
    q, k = make(256, H=1, seed=1)
    with pytest.raises(ValueError):
        O.xattn_estimate(q, k, 128, 8, chunk_size=256, kdb=2, pad0_quirk=False)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("Lq,Lk,C", [(200, 456, 256), (300, 300, 256), (128, 600, 128), (250, 700, 256)])
def test_triton_branch_zeroes_rows_by_key_position(Lq, Lk, C, causal):
    """With k_len > q_len and different paddings the two branches zero different rows:
    the Triton rule (kernels.py:70) against the row loops, the torch rule likewise."""
    S, bs = 8, 32
    q, k = make(Lq, H=1, seed=Lq + Lk, Lk=Lk)
    for triton in (True, False):
        sums, _ = O.xattn_estimate(q, k, bs, S, chunk_size=C, causal=causal, pad0_quirk=not triton)
        want = loop_block_sums(q, k, S, bs, C, causal, triton=triton)
        assert torch.allclose(sums.double(), want, atol=1e-5), (triton, (sums.double() - want).abs().max())
    a, _ = O.xattn_estimate(q, k, bs, S, chunk_size=C, causal=causal, pad0_quirk=False)
    b, _ = O.xattn_estimate(q, k, bs, S, chunk_size=C, causal=causal, pad0_quirk=True)
    if (-Lq % C) != (-Lk % C):
        assert not torch.allclose(a, b)           # the rules really differ on these shapes


@pytest.mark.parametrize("norm", [2, 0.5])
def test_norm_divides_the_logits(norm):
    S, bs, L = 8, 32, 256
    q, k = make(L, H=1, seed=31)
    sums, _ = O.xattn_estimate(q, k, bs, S, chunk_size=128, causal=True, norm=norm, pad0_quirk=False)
    want = loop_block_sums(q, k, S, bs, 128, True, norm=norm, triton=True)
    assert torch.allclose(sums.double(), want, atol=1e-5)
    # equivalent to scaling the queries
    other, _ = O.xattn_estimate(q / norm, k, bs, S, chunk_size=128, causal=True, pad0_quirk=False)
    assert torch.allclose(sums, other, atol=1e-6)
    plain, _ = O.xattn_estimate(q, k, bs, S, chunk_size=128, causal=True, pad0_quirk=False)
    assert not torch.allclose(sums, plain, atol=1e-3)
