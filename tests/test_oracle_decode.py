"""Pins oracle.single_decode_with_kv_cache to the mathematics (the upstream
kernel, flashinfer==0.1.6, is absent from the reference tree and from this
image: parity with it is unpinned)."""
import pytest
import torch
import torch.nn.functional as F

from oracle import xattn_oracle as O


@pytest.mark.parametrize("layout", ["HND", "NHD"])
def test_decode_is_sdpa_with_repeated_kv(layout):
    g = torch.Generator().manual_seed(0)
    H, Hkv, L, d = 8, 2, 333, 32
    q = torch.randn(H, d, generator=g)
    k = torch.randn(Hkv, L, d, generator=g)
    v = torch.randn(Hkv, L, d, generator=g)
    kk, vv = (k, v) if layout == "HND" else (k.transpose(0, 1).contiguous(), v.transpose(0, 1).contiguous())
    got = O.single_decode_with_kv_cache(q, kk, vv, kv_layout=layout)
    want = F.scaled_dot_product_attention(
        q[None, :, None, :], k.repeat_interleave(H // Hkv, 0)[None], v.repeat_interleave(H // Hkv, 0)[None]
    )[0, :, 0]
    assert torch.allclose(got, want, atol=2e-6)


def test_decode_is_last_row_of_causal_prefill():
    g = torch.Generator().manual_seed(1)
    H, Hkv, L, d = 4, 2, 200, 16
    q = torch.randn(1, H, L, d, generator=g)
    k = torch.randn(1, Hkv, L, d, generator=g)
    v = torch.randn(1, Hkv, L, d, generator=g)
    full = O.block_sparse_attention(q, k, v, torch.ones(1, H, 2, 2, dtype=torch.bool), causal=True)
    got = O.single_decode_with_kv_cache(q[0, :, -1], k[0], v[0], kv_layout="HND")
    assert torch.allclose(got, full[0, :, -1], atol=2e-6)


def test_decode_scale_and_single_key():
    g = torch.Generator().manual_seed(2)
    q = torch.randn(2, 8, generator=g)
    k = torch.randn(2, 1, 8, generator=g)
    v = torch.randn(2, 1, 8, generator=g)
    assert torch.allclose(O.single_decode_with_kv_cache(q, k, v, "HND"), v[:, 0])
    k3 = torch.randn(1, 3, 8, generator=g)
    v3 = torch.randn(1, 3, 8, generator=g)
    got = O.single_decode_with_kv_cache(q, k3, v3, "HND", sm_scale=0.0)   # uniform weights
    assert torch.allclose(got, v3[0].mean(0).expand(2, 8), atol=1e-6)
