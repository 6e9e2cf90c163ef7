"""GPU parity: xattn_decode_fwd (through the C ABI) vs the CPU oracle."""
import pytest
import torch

from helpers import OUT_MAX_ABS, OUT_MEAN_ABS
from oracle import xattn_oracle as O

pytestmark = pytest.mark.gpu


def _mk(H, Hkv, L, seed, spread=1.0):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(H, 128, generator=g) * spread).bfloat16()
    k = torch.randn(Hkv, L, 128, generator=g).bfloat16()
    v = torch.randn(Hkv, L, 128, generator=g).bfloat16()
    return q, k, v


def _check(out, want):
    err = (out.float().cpu() - want.float()).abs()
    assert torch.isfinite(out.float()).all()
    assert err.max().item() <= OUT_MAX_ABS, err.max().item()
    assert err.mean().item() <= OUT_MEAN_ABS, err.mean().item()


@pytest.mark.parametrize(
    "shape",
    [(32, 8, 4096), (32, 8, 1), (32, 8, 31), (32, 8, 33), (8, 8, 1000), (28, 4, 5555), (32, 1, 700),
     (4, 2, 40000), (32, 8, 131072 + 17)],
)
def test_decode_matches_oracle(shape):
    from xattn.src.decode import single_decode_with_kv_cache

    H, Hkv, L = shape
    q, k, v = _mk(H, Hkv, L, 5, spread=3.0)
    out = single_decode_with_kv_cache(q.cuda(), k.cuda(), v.cuda(), kv_layout="HND")
    assert out.shape == (H, 128) and out.dtype == torch.bfloat16
    _check(out, O.single_decode_with_kv_cache(q, k, v, kv_layout="HND"))


def test_decode_layouts_views_and_scale():
    from xattn.src.decode import single_decode_with_kv_cache

    H, Hkv, L = 32, 8, 3000
    q, k, v = _mk(H, Hkv, L, 6)
    want = O.single_decode_with_kv_cache(q, k, v, kv_layout="HND", sm_scale=0.05)
    kc, vc = k.cuda(), v.cuda()
    # token-major cache
    out = single_decode_with_kv_cache(
        q.cuda(), kc.transpose(0, 1).contiguous(), vc.transpose(0, 1).contiguous(), kv_layout="NHD", sm_scale=0.05
    )
    _check(out, want)
    # a static cache longer than what is filled: sliced views, as the reference's forward passes them
    big_k = torch.zeros(Hkv, 4096, 128, dtype=torch.bfloat16, device="cuda")
    big_v = torch.full((Hkv, 4096, 128), float("nan"), dtype=torch.bfloat16, device="cuda")
    big_k[:, :L], big_v[:, :L] = kc, vc
    out = single_decode_with_kv_cache(q.cuda(), big_k[:, :L], big_v[:, :L], kv_layout="HND", sm_scale=0.05)
    _check(out, want)
    # caller-provided output and workspace
    from xattn.src import hip_backend as hb

    ws = torch.empty(hb.lib().xattn_decode_workspace_bytes(H, Hkv, L), dtype=torch.uint8, device="cuda")
    dst = torch.empty(H, 128, dtype=torch.bfloat16, device="cuda")
    got = single_decode_with_kv_cache(q.cuda(), kc, vc, kv_layout="HND", sm_scale=0.05, out=dst, workspace=ws)
    assert got is dst
    _check(dst, want)


def test_decode_is_last_row_of_prefill_kernel():
    from xattn.src.decode import single_decode_with_kv_cache
    from xattn.src.Xattention import block_sparse_attention

    g = torch.Generator().manual_seed(7)
    H, Hkv, L = 32, 8, 2048
    q = torch.randn(1, H, L, 128, generator=g).bfloat16().cuda()
    k = torch.randn(1, Hkv, L, 128, generator=g).bfloat16().cuda()
    v = torch.randn(1, Hkv, L, 128, generator=g).bfloat16().cuda()
    full = block_sparse_attention(q, k, v, causal=True)
    out = single_decode_with_kv_cache(q[0, :, -1], k[0], v[0], kv_layout="HND")
    assert (out.float() - full[0, :, -1].float()).abs().max().item() <= 1e-2


def test_decode_rejects_bad_arguments():
    from xattn.src import hip_backend as hb
    from xattn.src.decode import single_decode_with_kv_cache

    q, k, v = (t.cuda() for t in _mk(32, 8, 64, 8))
    with pytest.raises(ValueError):
        single_decode_with_kv_cache(q[:30], k, v, kv_layout="HND")          # 30 heads over 8
    with pytest.raises(KeyError):
        single_decode_with_kv_cache(q, k, v, kv_layout="DNH")
    with pytest.raises(hb.XattnHipError):
        single_decode_with_kv_cache(q.cpu(), k.cpu(), v.cpu(), kv_layout="HND")
    lib = hb.lib()
    assert lib.xattn_decode_workspace_bytes(32, 5, 64) == 0
    ws = torch.empty(16, dtype=torch.uint8, device="cuda")
    out = torch.empty(32, 128, dtype=torch.bfloat16, device="cuda")
    code = lib.xattn_decode_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), ws.data_ptr(), 16,
                                32, 8, 64, 128, 128, 64 * 128, 128, 64 * 128, 128, 128, 0.1, None)
    assert code == -7   # XATTN_ERR_WORKSPACE
