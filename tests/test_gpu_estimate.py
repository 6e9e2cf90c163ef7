"""GPU parity: fused antidiagonal estimator (C ABI) vs the CPU oracle in fp32 on
the same bf16-valued inputs."""
import math

import pytest
import torch

from helpers import mask_mismatch_report
from oracle import xattn_oracle as O

pytestmark = pytest.mark.gpu


def _mk(H, Hkv, Lq, Lk, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    q = (scale * torch.randn(1, H, Lq, 128, generator=g)).bfloat16()
    k = (scale * torch.randn(1, Hkv, Lk, 128, generator=g)).bfloat16()
    return q, k


def _oracle_sums(q, k, S, C, causal, quirk, group):
    kk = k.repeat_interleave(group, 1).float()
    sums, _ = O.xattn_estimate(q.float(), kk, 128, S, threshold=0.9, chunk_size=C, causal=causal, pad0_quirk=quirk)
    return sums[0]


@pytest.mark.parametrize("S", [4, 8, 16])
def test_raw_scores_match_antidiagonal_sums(S):
    from xattn.src.Xattention import estimate_and_select

    q, k = _mk(2, 1, 1024, 1024, S)
    r = estimate_and_select(q.cuda(), k.cuda(), S, 0.9, 512, causal=False, dump_scores=True)
    want = O.antidiagonal_scores(q.float(), k.repeat_interleave(2, 1).float(), S)[0]
    got = r["scores"].cpu()
    assert got.shape == want.shape
    assert torch.allclose(got, want, rtol=1e-4, atol=2e-3), (got - want).abs().max()


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("S,C,L", [(8, 512, 2048), (16, 2048, 4096), (4, 256, 1024), (16, 1024, 3000), (8, 512, 1300)])
def test_block_sums_match_oracle(S, C, L, causal):
    from xattn.src.Xattention import estimate_and_select

    q, k = _mk(4, 2, L, L, 10 + S, scale=1.5)
    for use_triton in (True, False):
        r = estimate_and_select(q.cuda(), k.cuda(), S, 0.9, C, causal=causal, use_triton=use_triton, want_lists=False)
        want = _oracle_sums(q, k, S, C, causal, quirk=not use_triton, group=2)
        got = r["sums"].cpu()
        assert got.shape == want.shape
        assert torch.isfinite(got).all()
        assert torch.allclose(got, want, rtol=2e-4, atol=2e-5), (use_triton, (got - want).abs().max())


def test_kv_longer_than_q_and_strided_views():
    from xattn.src.Xattention import estimate_and_select

    S, C = 8, 512
    g = torch.Generator().manual_seed(4)
    q = torch.randn(1, 512, 4, 128, generator=g).bfloat16().transpose(1, 2)
    k = torch.randn(1, 1536, 4, 128, generator=g).bfloat16().transpose(1, 2)
    r = estimate_and_select(q.cuda(), k.cuda(), S, 0.9, C, causal=True, want_lists=False)
    want = _oracle_sums(q, k, S, C, True, quirk=False, group=1)
    assert torch.allclose(r["sums"].cpu(), want, rtol=2e-4, atol=2e-5)


def test_row_mass_invariant_large_logits():
    """Each real q-block row of the block sums adds up to block_size/stride even
    when logits are large (exercises the tile-local maxima)."""
    from xattn.src.Xattention import estimate_and_select

    S, C, L = 16, 2048, 8192
    q, k = _mk(2, 2, L, L, 6, scale=4.0)
    r = estimate_and_select(q.cuda(), k.cuda(), S, 0.9, C, causal=True, want_lists=False)
    mass = r["sums"].double().sum(-1).cpu()
    assert torch.allclose(mass, torch.full_like(mass, 128 / S), atol=1e-3)
    nb = L // 128
    upper = torch.triu(torch.ones(nb, nb, dtype=torch.bool), diagonal=1)
    assert (r["sums"].cpu()[:, upper] == 0).all()


@pytest.mark.parametrize("is_causal", [True, False])
def test_seam_flat_group_gemm_fuse_reshape(is_causal):
    """The reference-named seam (xattn/src/kernels.py:325) on a middle query chunk."""
    from xattn.src.kernels import flat_group_gemm_fuse_reshape, softmax_fuse_block_sum

    S = 8
    q, k = _mk(2, 2, 3 * S * 128, 3 * S * 128, 21)
    qc = q[:, :, S * 128 : 2 * S * 128]            # second chunk of three
    out = flat_group_gemm_fuse_reshape(qc.cuda(), k.cuda(), S, 128, 256, is_causal=is_causal)
    want = O.antidiagonal_scores(qc.float(), k.float(), S)
    assert out.shape == (1, 2, 128, 384) and out.dtype == torch.bfloat16
    cols = 256 if is_causal else 384            # tiles past the chunk's diagonal are not computed
    assert torch.allclose(out[..., :cols].float().cpu(), want[..., :cols], rtol=1e-2, atol=0.2)
    # ... and the second seam on those very scores, the reference's own two-step sequence
    # (xattn/src/Xattention.py:141-172), against a plain torch softmax of them
    scale = 1.4426950408889634 / math.sqrt(128) / S
    sums = softmax_fuse_block_sum(out, 16, 16, 128, 256, 300, scale, is_causal=is_causal)
    assert sums.shape == (1, 2, 8, 24) and sums.dtype == torch.bfloat16
    x = out.float().cpu() * (scale / 1.4426950408889634)
    if is_causal:
        pos = torch.arange(128)[:, None] + 128
        x = x.masked_fill(torch.arange(384)[None, :] > pos, float("-inf"))
    p = torch.softmax(x, -1)
    p[:, :, 300 - 128:, :] = 0                      # rows at positions >= real_q_len
    want_sums = p.view(1, 2, 8, 16, 24, 16).sum(-1).sum(-2)
    assert torch.allclose(sums.float().cpu(), want_sums, rtol=1e-2, atol=1e-3)


@pytest.mark.parametrize("rbs,n_rq,n_rk,start", [(8, 64, 1024, 960), (32, 96, 2048, 512), (16, 16, 528, 0)])
def test_seam_softmax_fuse_block_sum_fp32_check(rbs, n_rq, n_rk, start):
    """Closer check of the stand-alone kernel through the C ABI (fp32 output)."""
    from xattn.src import hip_backend as hb

    g = torch.Generator().manual_seed(rbs)
    x = (3.0 * torch.randn(3, n_rq, n_rk, generator=g)).bfloat16()
    xd = x.cuda()
    for causal in (1, 0):
        out = torch.empty(3, n_rq // rbs, n_rk // rbs, dtype=torch.float32, device="cuda")
        hb.check(hb.lib().xattn_softmax_block_sums(xd.data_ptr(), out.data_ptr(), 3, n_rq, n_rk, xd.stride(0),
                                                   xd.stride(1), rbs, start, start + n_rq - 5, 0.7, causal, None), "sbs")
        s = x.double() * 0.7 * math.log(2.0)
        if causal:
            s = s.masked_fill(torch.arange(n_rk)[None, :] > torch.arange(n_rq)[:, None] + start, float("-inf"))
        p = torch.softmax(s, -1)
        p[:, n_rq - 5:] = 0
        want = p.view(3, n_rq // rbs, rbs, n_rk // rbs, rbs).sum(-1).sum(-2)
        assert torch.allclose(out.double().cpu(), want, rtol=1e-4, atol=1e-6), (causal, (out.double().cpu() - want).abs().max())


def test_workspace_limit_splits_the_launch_without_changing_results(monkeypatch):
    import xattn.src.Xattention as X

    q, k = _mk(4, 2, 4096, 4096, 33)
    a = X.estimate_and_select(q.cuda(), k.cuda(), 8, 0.9, 512, causal=True, want_lists=False)["sums"].clone()
    monkeypatch.setattr(X, "WORKSPACE_LIMIT", 1 << 20)     # forces several chunk groups
    b = X.estimate_and_select(q.cuda(), k.cuda(), 8, 0.9, 512, causal=True, want_lists=False)["sums"]
    assert torch.equal(a, b)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("mode", ["slash", "random", "double", "triple"])
@pytest.mark.parametrize("S,C,L", [(8, 512, 1300), (16, 1024, 2048), (4, 256, 1024)])
def test_select_modes_match_oracle(S, C, L, mode, causal):
    """The other reshapes of the reference's torch branch (xattn/src/Xattention.py:72-135)
    through the public operator: block sums against the oracle (fp32 inputs, so
    its rolled key sums are exact like the kernel's fp32 accumulation)."""
    from xattn.src.Xattention import xattn_estimate

    q, k = _mk(4, 2, L, L, 20 + S)
    torch.manual_seed(123)                 # "random" draws torch.randperm(stride) from the global generator
    perm = torch.randperm(S)
    torch.manual_seed(123)
    got, mask = xattn_estimate(q.cuda(), k.cuda(), 128, S, threshold=0.9, chunk_size=C, select_mode=mode,
                               causal=causal)
    want, want_mask = O.xattn_estimate(q.float(), k.repeat_interleave(2, 1).float(), 128, S, threshold=0.9,
                                       chunk_size=C, select_mode=mode, causal=causal, pad0_quirk=False, perm=perm)
    assert got.shape == want.shape and got.dtype == torch.bfloat16
    assert torch.allclose(got.float().cpu(), want, rtol=1e-2, atol=1e-3)     # bf16 result of the public operator
    nbad, outside = mask_mismatch_report(want[0], mask[0], want_mask[0], 0.9, causal, 0, C // 128)
    assert outside == 0, (nbad, outside)


@pytest.mark.parametrize("causal", [True, False])
def test_softmax_false_matches_oracle(causal):
    """softmax=False (xattn/src/Xattention.py:231-234): block sums of exp(scaled score)."""
    from xattn.src.Xattention import estimate_and_select

    S, C, L = 8, 512, 1300
    q, k = _mk(4, 2, L, L, 31, scale=1.5)
    r = estimate_and_select(q.cuda(), k.cuda(), S, 0.9, C, causal=causal, want_lists=False, softmax=False)
    want, _ = O.xattn_estimate(q.float(), k.repeat_interleave(2, 1).float(), 128, S, threshold=0.9, chunk_size=C,
                               causal=causal, pad0_quirk=False, softmax=False)
    assert torch.allclose(r["sums"].cpu(), want[0], rtol=2e-4, atol=2e-5)


def test_bad_slab_pairs_are_refused():
    from xattn.src import hip_backend as hb
    from xattn.src.Xattention import estimate_and_select

    q, k = _mk(2, 2, 512, 512, 1)
    with pytest.raises(hb.XattnHipError):
        estimate_and_select(q.cuda(), k.cuda(), 8, 0.9, 512, slab_pairs=[(8, 0)])      # offset outside the stride
    with pytest.raises(hb.XattnHipError):
        estimate_and_select(q.cuda(), k.cuda(), 8, 0.9, 512, slab_pairs=[(0, 0)] * 65)  # more than 64 pairs


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("kdb,S,C,L", [(2, 8, 512, 2048), (4, 8, 512, 1300), (2, 16, 1024, 3000), (4, 16, 2048, 4096),
                                       (2, 4, 256, 1024), (4, 4, 256, 900), (2, 8, 256, 1016)])
def test_kdb_matches_oracle(kdb, S, C, L, causal):
    """Query-row subsampling of the reference's torch branch (xattn/src/Xattention.py:88-93,
    174-181, 217-222, 245): block sums and mask against the oracle; (2, 8, 256, 1016) has
    one padded reshaped row, fewer than kdb, which zeroes the whole last chunk (the slice [-0:])."""
    from xattn.src.Xattention import estimate_and_select, xattn_estimate

    q, k = _mk(4, 2, L, L, 40 + S + kdb, scale=1.5)
    r = estimate_and_select(q.cuda(), k.cuda(), S, 0.9, C, causal=causal, use_triton=False, kdb=kdb)
    want, want_mask = O.xattn_estimate(q.float(), k.repeat_interleave(2, 1).float(), 128, S, threshold=0.9,
                                       chunk_size=C, causal=causal, kdb=kdb, pad0_quirk=True)
    got = r["sums"].cpu()
    assert got.shape == want[0].shape and torch.isfinite(got).all()
    assert torch.allclose(got, want[0], rtol=2e-4, atol=2e-5), (got - want[0]).abs().max()
    nbad, outside = mask_mismatch_report(want[0], r["mask"], want_mask[0], 0.9, causal, 0, C // 128)
    assert outside == 0, (nbad, outside)
    with pytest.raises(ValueError):
        xattn_estimate(q.cuda(), k.cuda(), 128, S, chunk_size=C, kdb=kdb)          # use_triton=True, like the reference
    _, m2 = xattn_estimate(q.cuda(), k.cuda(), 128, S, threshold=0.9, chunk_size=C, kdb=kdb, use_triton=False,
                           causal=causal)
    assert torch.equal(m2[0].cpu(), r["mask"].bool().cpu())


@pytest.mark.parametrize("norm", [2, 0.5])
@pytest.mark.parametrize("causal", [True, False])
def test_norm_matches_oracle(norm, causal):
    from xattn.src.Xattention import estimate_and_select

    S, C, L = 8, 512, 1800
    q, k = _mk(4, 2, L, L, 50, scale=1.5)
    r = estimate_and_select(q.cuda(), k.cuda(), S, 0.9, C, causal=causal, norm=norm)
    want, want_mask = O.xattn_estimate(q.float(), k.repeat_interleave(2, 1).float(), 128, S, threshold=0.9,
                                       chunk_size=C, causal=causal, norm=norm, pad0_quirk=False)
    assert torch.allclose(r["sums"].cpu(), want[0], rtol=2e-4, atol=2e-5)
    nbad, outside = mask_mismatch_report(want[0], r["mask"], want_mask[0], 0.9, causal, 0, C // 128)
    assert outside == 0, (nbad, outside)
    plain = estimate_and_select(q.cuda(), k.cuda(), S, 0.9, C, causal=causal)["sums"]
    assert not torch.allclose(plain, r["sums"], atol=1e-3)


@pytest.mark.parametrize("use_triton", [True, False])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("Lq,Lk,C", [(4000, 5000, 2048), (1000, 3000, 1024), (2100, 2300, 512)])
def test_ragged_kv_longer_than_q_follows_each_branch_row_rule(Lq, Lk, C, causal, use_triton):
    """Different query and key padding: the Triton branch zeroes rows by key-axis position against
    the real key length (xattn/src/kernels.py:70), the torch branch the padded query tail."""
    from xattn.src.Xattention import estimate_and_select

    S = 8
    q, k = _mk(4, 2, Lq, Lk, 60, scale=1.5)
    r = estimate_and_select(q.cuda(), k.cuda(), S, 0.9, C, causal=causal, use_triton=use_triton)
    want, want_mask = O.xattn_estimate(q.float(), k.repeat_interleave(2, 1).float(), 128, S, threshold=0.9,
                                       chunk_size=C, causal=causal, pad0_quirk=not use_triton)
    assert torch.allclose(r["sums"].cpu(), want[0], rtol=2e-4, atol=2e-5), (r["sums"].cpu() - want[0]).abs().max()
    nq_p, nk_p = want_mask.shape[2], want_mask.shape[3]
    nbad, outside = mask_mismatch_report(want[0], r["mask"], want_mask[0], 0.9, causal, nk_p - nq_p, C // 128)
    assert outside == 0, (nbad, outside)


@pytest.mark.parametrize("use_triton", [True, False])
@pytest.mark.parametrize("S,L,C", [(16, 2426, 128), (8, 4096 - 5, 2048), (16, 2048 - 15, 512), (4, 1024 - 3, 256)])
def test_padding_shorter_than_the_stride(S, L, C, use_triton):
    """0 < padding < stride: the reshaped padding count is 0, so the torch branch's slice over "the last 0
    reshaped keys" covers every key and each query chunk again sees only its own chunk
    (xattn/src/Xattention.py:67,201); the Triton branch zeroes no row (kernels.py:70)."""
    from xattn.src.Xattention import estimate_and_select

    q, k = _mk(4, 2, L, L, 61, scale=1.5)
    r = estimate_and_select(q.cuda(), k.cuda(), S, 0.9, C, causal=True, use_triton=use_triton)
    want, want_mask = O.xattn_estimate(q.float(), k.repeat_interleave(2, 1).float(), 128, S, threshold=0.9,
                                       chunk_size=C, causal=True, pad0_quirk=not use_triton)
    assert torch.allclose(r["sums"].cpu(), want[0], rtol=2e-4, atol=2e-5), (r["sums"].cpu() - want[0]).abs().max()
    nbad, outside = mask_mismatch_report(want[0], r["mask"], want_mask[0], 0.9, True, 0, C // 128)
    assert outside == 0, (nbad, outside)


@pytest.mark.parametrize("causal,use_triton", [(True, True), (True, False), (False, True)])
def test_more_tiles_than_compute_units(causal, use_triton):
    """S=4 at 12k tokens and 8 heads is 600-1200 tiles of 256x256: every workgroup of the estimator then works
    through several tiles (the next tile's first slabs are requested before the current tile's epilogue), with
    a ragged last tile and a cached prefix."""
    from xattn.src.Xattention import estimate_and_select

    S, C, Lq, Lk = 4, 2048, 12288 - 37, 12288 + 1024 - 37
    if not causal:
        Lk = Lq
    q, k = _mk(8, 2, Lq, Lk, 77, scale=1.5)
    r = estimate_and_select(q.cuda(), k.cuda(), S, 0.9, C, causal=causal, use_triton=use_triton)
    want, want_mask = O.xattn_estimate(q.float(), k.repeat_interleave(4, 1).float(), 128, S, threshold=0.9,
                                       chunk_size=C, causal=causal, pad0_quirk=not use_triton)
    assert torch.allclose(r["sums"].cpu(), want[0], rtol=2e-4, atol=2e-5), (r["sums"].cpu() - want[0]).abs().max()
    nq_p, nk_p = want_mask.shape[2], want_mask.shape[3]
    nbad, outside = mask_mismatch_report(want[0], r["mask"], want_mask[0], 0.9, causal, nk_p - nq_p, C // 128)
    assert outside == 0, (nbad, outside)
