"""Pins the oracle's threshold-profiler functions to their definitions (the
reference module imports flash_attn and needs a GPU, so it cannot be run here)."""
import math

import torch

from oracle import xattn_oracle as O


def test_block_mass_matches_full_softmax_and_row_sums():
    g = torch.Generator().manual_seed(0)
    H, Hkv, L, d, bs = 4, 2, 45, 8, 16
    q = torch.randn(1, H, L, d, generator=g)
    k = torch.randn(1, Hkv, L, d, generator=g)
    got = O.chunk_prefill_to_attn_sum(q, k, block_size=bs)
    nb = (L + bs - 1) // bs
    want = torch.zeros(1, H, nb, nb)
    for h in range(H):
        for r in range(L):
            logits = torch.tensor([float(q[0, h, r] @ k[0, h // 2, c]) / math.sqrt(d) for c in range(r + 1)])
            p = torch.softmax(logits, 0)
            for c in range(r + 1):
                want[0, h, r // bs, c // bs] += p[c]
    assert torch.allclose(got, want, atol=1e-5)
    rows = torch.tensor([min(bs, L - i * bs) for i in range(nb)], dtype=torch.float32)
    assert torch.allclose(got.sum(-1), rows.expand(1, H, nb), atol=1e-4)
    assert (got.triu(1) == 0).all()


def test_threshold_hand_example():
    # one head, two rows.  Row 0: masses .5 .3 .15 .05 -> cumsum .5 .8 .95 1.0, three blocks reach 0.9;
    # their estimates are 4, 1, 2 -> cut 1 -> every estimate >= 1 counts: 4 + 1 + 2 + 3 = 10 of 10.
    # Row 1: mass .95 .05 0 0 -> one block, estimate 5 -> cut 5 -> only 5 counts, of 5 + 1 + 1 + 3 = 10.
    attn = torch.tensor([[[[0.5, 0.3, 0.15, 0.05], [0.95, 0.05, 0.0, 0.0]]]])
    x = torch.tensor([[[[4.0, 1.0, 2.0, 3.0], [5.0, 1.0, 1.0, 3.0]]]])
    got = O.profile_threshold_head(attn, x)
    assert torch.allclose(got, torch.tensor([[15.0 / 20.0]]), atol=1e-6)


def test_threshold_matches_python_definition():
    g = torch.Generator().manual_seed(1)
    H, n = 3, 9
    attn = torch.rand(1, H, n, n, generator=g).tril() ** 3
    x = (attn + 0.2 * torch.rand(1, H, n, n, generator=g)).tril()
    got = O.profile_threshold_head(attn, x, coverage=0.8)
    for h in range(H):
        num = den = 0.0
        for i in range(n):
            a, xs = attn[0, h, i].tolist(), x[0, h, i].tolist()
            order = sorted(range(n), key=lambda j: (-a[j], j))
            tot, cum, taken = sum(a), 0.0, []
            for j in order:
                taken.append(j)
                cum += a[j]
                if not cum < 0.8 * tot:
                    break
            cut = min(xs[j] for j in taken)
            num += sum(v for v in xs if v >= cut)
            den += sum(xs)
        assert abs(got[0, h].item() - num / (den + 1e-8)) < 1e-5
