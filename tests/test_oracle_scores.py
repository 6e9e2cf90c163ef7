"""Pins oracle.antidiagonal_scores to the mathematics: brute force over the
full Q.K^T (sum of the S x S antidiagonal cells) and the pointer form of the
reference's Triton kernel (xattn/src/kernels.py:219-230)."""
import pytest
import torch

from oracle import xattn_oracle as O


def brute_antidiagonal(q, k, S):
    full = torch.einsum("bhqd,bhkd->bhqk", q.double(), k.double())
    B, H, Lq, Lk = full.shape
    out = torch.zeros(B, H, Lq // S, Lk // S, dtype=torch.float64)
    for m in range(Lq // S):
        for n in range(Lk // S):
            acc = 0
            for i in range(S):
                acc = acc + full[:, :, m * S + S - 1 - i, n * S + i]
            out[:, :, m, n] = acc
    return out


@pytest.mark.parametrize("S", [4, 8, 16])
def test_scores_match_bruteforce(S):
    g = torch.Generator().manual_seed(S)
    q = torch.randn(1, 2, 6 * S, 16, generator=g)
    k = torch.randn(1, 2, 5 * S, 16, generator=g)
    got = O.antidiagonal_scores(q.double(), k.double(), S)
    assert torch.allclose(got, brute_antidiagonal(q, k, S), atol=1e-10)


def test_pointer_form_equals_concat_form():
    S, d = 8, 32
    g = torch.Generator().manual_seed(1)
    q = torch.randn(1, 3, 16 * S, d, generator=g, dtype=torch.float64)
    k = torch.randn(1, 3, 16 * S, d, generator=g, dtype=torch.float64)
    acc = torch.zeros(1, 3, 16, 16, dtype=torch.float64)
    rows = torch.arange(16) * S
    for it in range(S):
        acc += q[:, :, rows + (S - 1) - it, :] @ k[:, :, rows + it, :].transpose(2, 3)
    assert torch.allclose(acc, O.antidiagonal_scores(q, k, S), atol=1e-10)


def test_a_transposed_or_unreversed_operand_would_fail():
    S = 4
    g = torch.Generator().manual_seed(2)
    q = torch.randn(1, 1, 4 * S, 8, generator=g, dtype=torch.float64)
    k = torch.randn(1, 1, 4 * S, 8, generator=g, dtype=torch.float64)
    good = brute_antidiagonal(q, k, S)
    unreversed = torch.cat([q[:, :, i::S] for i in range(S)], -1) @ torch.cat(
        [k[:, :, i::S] for i in range(S)], -1
    ).transpose(2, 3)
    assert not torch.allclose(unreversed, good, atol=1e-6)
    assert torch.allclose(O.antidiagonal_scores(q, k, S), good, atol=1e-10)


@pytest.mark.parametrize("mode", ["slash", "random", "double", "triple"])
@pytest.mark.parametrize("S", [4, 8])
def test_select_modes_are_sums_over_offset_pairs(mode, S):
    """Every select_mode of the torch branch (xattn/src/Xattention.py:72-135) is a
    sum of Q[m*S + a] . K[n*S + b] over a fixed list of (a, b): the lists below
    are written out by hand, independently of the product's table."""
    g = torch.Generator().manual_seed(S)
    q = torch.randn(1, 2, 5 * S, 8, generator=g, dtype=torch.float64)
    k = torch.randn(1, 2, 7 * S, 8, generator=g, dtype=torch.float64)
    perm = torch.randperm(S, generator=g)
    rq, rk = O.reshape_operands(q, k, S, mode, perm)
    got = rq @ rk.transpose(2, 3)
    full = torch.einsum("bhqd,bhkd->bhqk", q, k)
    pairs = {
        "slash": [(i, i, 1) for i in range(S)],
        "random": [(int(perm[i]), i, 1) for i in range(S)],
        "double": [(S - 1 - i, i, 1) for i in range(S)] + [(S - 1 - i, (i + 1) % S, 1) for i in range(S)],
        "triple": [(S - 1 - i, i, 2) for i in range(S)] + [(S - 1 - i, (i + 1) % S, 1) for i in range(S)]
        + [(S - 1 - i, (i - 1) % S, 1) for i in range(S)],
    }[mode]
    want = sum(w * full[:, :, a::S, b::S] for a, b, w in pairs)
    assert torch.allclose(got, want, atol=1e-10)
    # and the product's table encodes the same list
    from xattn.src.Xattention import slab_pairs_for
    import collections

    table = collections.Counter(slab_pairs_for(mode, S, perm))
    assert table == collections.Counter({(a, b): w for a, b, w in pairs})
    assert slab_pairs_for("inverse", S) is None
