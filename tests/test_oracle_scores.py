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
