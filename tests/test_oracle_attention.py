"""Pins oracle.block_sparse_attention to the mathematics (the upstream kernel,
block_sparse_attn==0.0.1, is absent from the reference tree: parity with it is
unpinned).  All-True mask == torch SDPA; tiny cases == a per-row python loop."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import xattn_oracle as O


@pytest.mark.parametrize("causal", [True, False])
def test_full_mask_is_sdpa(causal):
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(1, 4, 300, 32, generator=g) for _ in range(3))
    nb = 3
    m = torch.ones(1, 4, nb, nb, dtype=torch.bool)
    got = O.block_sparse_attention(q, k, v, m, causal=causal, row_tile=128)
    want = F.scaled_dot_product_attention(q, k, v, is_causal=causal)
    assert torch.allclose(got, want, atol=2e-5)


@pytest.mark.parametrize("causal", [True, False])
def test_random_mask_matches_row_loop(causal):
    g = torch.Generator().manual_seed(1)
    bs, Lq, Lk, d, H, Hkv = 16, 40, 72, 8, 4, 2
    q = torch.randn(1, H, Lq, d, generator=g)
    k = torch.randn(1, Hkv, Lk, d, generator=g)
    v = torch.randn(1, Hkv, Lk, d, generator=g)
    m = torch.rand(1, H, 3, 5, generator=g) < 0.5
    m[..., 0] = True
    got = O.block_sparse_attention(q, k, v, m, causal=causal, block_size=bs)
    for h in range(H):
        for r in range(Lq):
            cols = [
                c
                for c in range(Lk)
                if m[0, h, r // bs, c // bs] and (not causal or c <= r + (Lk - Lq))
            ]
            logits = torch.tensor([float(q[0, h, r] @ k[0, h // 2, c]) / math.sqrt(d) for c in cols])
            p = torch.softmax(logits, 0)
            want = sum(p[i] * v[0, h // 2, c] for i, c in enumerate(cols))
            assert torch.allclose(got[0, h, r], want, atol=1e-5)


def test_gqa_equals_repeated_kv():
    g = torch.Generator().manual_seed(2)
    q = torch.randn(1, 8, 256, 16, generator=g)
    k = torch.randn(1, 2, 256, 16, generator=g)
    v = torch.randn(1, 2, 256, 16, generator=g)
    m = torch.tril(torch.rand(1, 8, 2, 2, generator=g) < 0.7) | torch.eye(2, dtype=torch.bool)
    a = O.block_sparse_attention(q, k, v, m, causal=True)
    b = O.block_sparse_attention(q, k.repeat_interleave(4, 1), v.repeat_interleave(4, 1), m, causal=True)
    assert torch.equal(a, b)


def test_prefill_glue_slices_mask_and_runs():
    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(1, 2, 300, 16, generator=g) for _ in range(3))
    out, mask = O.Xattention_prefill(q, k, v, 8, threshold=0.9, chunk_size=256, return_mask=True)
    assert out.shape == q.shape and mask.shape == (1, 2, 3, 3)
    full = O.block_sparse_attention(q, k, v, torch.ones_like(mask), causal=True)
    dense = O.Xattention_prefill(q, k, v, 8, threshold=1.0, chunk_size=256, pad0_quirk=False)
    assert torch.allclose(dense, full, atol=1e-6)
