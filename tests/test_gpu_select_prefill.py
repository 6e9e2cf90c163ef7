"""GPU parity: block selection kernel and the whole operator vs the CPU oracle."""
import os

import pytest
import torch

from helpers import OUT_MAX_ABS, OUT_MEAN_ABS, mask_mismatch_report
from oracle import xattn_oracle as O

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden", "find_blocks_golden.pt")


def _select(sums, tau, causal, diag_offset, keep_sink=False, keep_recent=False):
    """Runs xattn_select_blocks on fp32 block sums [H, nq, nk]; returns bool mask, lists."""
    from xattn.src import hip_backend as hb

    lib = hb.lib()
    H, nq, nk = sums.shape
    s = sums.float().contiguous().cuda()
    if isinstance(tau, torch.Tensor):
        t = tau.double().reshape(-1)
        t = (t.expand(H) if t.numel() == 1 else t).contiguous().cuda()
    else:
        t = torch.full((H,), float(tau), dtype=torch.float64).cuda()
    mask = torch.empty((H, nq, nk), dtype=torch.uint8, device="cuda")
    idx = torch.empty((H, nq, nk), dtype=torch.int32, device="cuda")
    cnt = torch.empty((H, nq), dtype=torch.int32, device="cuda")
    hb.check(
        lib.xattn_select_blocks(
            s.data_ptr(), t.data_ptr(), mask.data_ptr(), idx.data_ptr(), cnt.data_ptr(), nk,
            H, nq, nk, 0, nq, diag_offset, int(causal), int(keep_sink), int(keep_recent),
            nk, nq * 128, diag_offset * 128, nq, 0, 0, torch.cuda.current_stream().cuda_stream,
        ),
        "xattn_select_blocks",
    )
    torch.cuda.synchronize()
    return mask.bool().cpu(), idx.cpu(), cnt.cpu()


def test_golden_vectors_of_the_reference():
    """Reference masks (xattn/src/utils.py on CPU) after the block-tril that
    xattn_estimate applies (Xattention.py:275-285), which the kernel fuses."""
    cases = torch.load(GOLD, weights_only=True)
    n = 0
    for c in cases:
        if c["name"] == "causal_dense_future":
            continue  # the kernel takes sums beyond the diagonal as zero (the estimator writes zeros there)
        x = c["x"][0].float()
        tau = c["threshold"] if c["threshold_is_tensor"] else float(c["threshold"])
        want = c["mask"][0].clone()
        rows, cols = want.shape[1:]
        if c["causal"]:
            vis = torch.arange(cols)[None, :] <= torch.arange(rows)[:, None] + c["current_index"]
            want &= vis
        got, idx, cnt = _select(x, tau, c["causal"], c["current_index"])
        nbad, outside = mask_mismatch_report(x, got, want, tau, c["causal"], c["current_index"])
        assert outside == 0, (c["name"], nbad)
        # compacted list == mask
        for h in range(x.shape[0]):
            for r in range(rows):
                assert idx[h, r, : cnt[h, r]].tolist() == got[h, r].nonzero().flatten().tolist()
        n += 1
    assert n >= 20


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("nk", [33, 256, 1000])
def test_selection_matches_oracle_on_random_sums(causal, nk):
    g = torch.Generator().manual_seed(nk)
    H, nq = 3, min(nk, 64)
    off = nk - nq
    x = torch.rand(H, nq, nk, generator=g) ** 4
    if causal:
        vis = torch.arange(nk)[None, :] <= torch.arange(nq)[:, None] + off
        x = x * vis
    taus = torch.tensor([0.5, 0.9, 0.97], dtype=torch.float32)
    got, _, _ = _select(x, taus, causal, off)
    want = O.find_blocks_chunked(x[None], off, taus, None, decoding=False, mode="prefill", causal=causal)[0]
    if causal:
        want &= vis
    nbad, outside = mask_mismatch_report(x, got, want, taus, causal, off)
    assert outside == 0 and nbad <= 2, (nbad, outside)


def test_keep_sink_and_keep_recent():
    g = torch.Generator().manual_seed(1)
    x = torch.rand(2, 8, 8, generator=g) * torch.tril(torch.ones(8, 8))
    got, idx, cnt = _select(x, 0.0, True, 0, keep_sink=True)
    assert got[:, 0, :].all()                       # row 0 entirely, future blocks included
    assert cnt[:, 0].tolist() == [1, 1]             # ... but the list holds visible blocks only
    assert got[:, 1:].sum().item() == 2 * 7 * 2  # tau=0: sink + diagonal only
    xn = torch.rand(2, 8, 8, generator=g)
    got, _, _ = _select(xn, 0.2, False, 0, keep_recent=True)
    assert torch.diagonal(got, dim1=-2, dim2=-1).all()


@pytest.mark.parametrize(
    "name,L,H,Hkv,S,C,tau,causal",
    [
        ("text_S8", 4096, 8, 2, 8, 2048, 0.9, True),
        ("text_S16", 8192, 4, 4, 16, 2048, 0.9, True),
        ("text_ragged", 3000, 4, 2, 8, 1024, 0.9, True),
        ("noncausal", 2304, 4, 4, 8, 1024, 0.95, False),
    ],
)
@pytest.mark.parametrize("use_triton", [True, False])
def test_operator_mask_and_output_parity(name, L, H, Hkv, S, C, tau, causal, use_triton):
    from xattn.src.Xattention import Xattention_prefill, block_sparse_attention, xattn_estimate
    from xattn.synthetic import WORKLOADS, make_inputs

    w = WORKLOADS[1]
    q, k, v = make_inputs(w, device="cpu", seed=3, L=L, heads=H, kv_heads=Hkv)
    group = H // Hkv
    qf, kf = q.float(), k.repeat_interleave(group, 1).float()
    want_sums, want_mask = O.xattn_estimate(
        qf, kf, 128, S, threshold=tau, chunk_size=C, causal=causal, pad0_quirk=not use_triton
    )
    sums, mask = xattn_estimate(
        q.cuda(), k.cuda(), 128, S, threshold=tau, chunk_size=C, causal=causal, use_triton=use_triton
    )
    assert mask.dtype == torch.bool and mask.shape == want_mask.shape and sums.dtype == q.dtype
    off = 0
    nbad, outside = mask_mismatch_report(want_sums[0], mask[0], want_mask[0], tau, causal, off, C // 128)
    print(f"{name}: {nbad} mask mismatches, {outside} outside the tau band, density {want_mask.float().mean():.3f}")
    assert outside == 0
    assert nbad <= max(2, int(1e-3 * mask.numel()))

    # attention output given the ORACLE's mask
    nb = (L + 127) // 128
    m = want_mask[0, :, :nb, :nb]
    from helpers import lists_from_mask

    idx, cnt = lists_from_mask(m)
    out = block_sparse_attention(q.cuda(), k.cuda(), v.cuda(), idx.cuda(), cnt.cuda(), causal=causal)
    want = O.block_sparse_attention(q, k, v, m[None], causal=causal)
    err = (out.float().cpu() - want.float()).abs()
    assert err.max().item() <= OUT_MAX_ABS and err.mean().item() <= OUT_MEAN_ABS

    # and the operator end to end (its own mask)
    full = Xattention_prefill(q.cuda(), k.cuda(), v.cuda(), S, threshold=tau, chunk_size=C, causal=causal, use_triton=use_triton)
    assert full.shape == (1, H, L, 128) and torch.isfinite(full.float()).all()
    # chunk-by-chunk orchestration on side streams computes the same thing
    piped = Xattention_prefill(q.cuda(), k.cuda(), v.cuda(), S, threshold=tau, chunk_size=C, causal=causal,
                               use_triton=use_triton, pipeline_chunks=True)
    torch.cuda.synchronize()
    assert torch.equal(piped, full)
    if nbad == 0:
        assert (full.float().cpu() - want.float()).abs().max().item() <= OUT_MAX_ABS


def test_seam_find_blocks_chunked_matches_reference_goldens():
    """The reference-named seam (xattn/src/utils.py:44) against the golden masks,
    cropped to each row's diagonal as the seam documents."""
    from xattn.src.utils import find_blocks_chunked

    for c in torch.load(GOLD, weights_only=True):
        if c["name"] == "causal_dense_future":
            continue
        tau = c["threshold"] if c["threshold_is_tensor"] else float(c["threshold"])
        got = find_blocks_chunked(c["x"].cuda(), c["current_index"], tau, None, decoding=False, mode="prefill", causal=c["causal"])
        want = c["mask"].clone()
        rows, cols = want.shape[2:]
        if c["causal"]:
            want &= torch.arange(cols)[None, :] <= torch.arange(rows)[:, None] + c["current_index"]
        nbad, outside = mask_mismatch_report(c["x"][0].float(), got[0], want[0], tau, c["causal"], c["current_index"])
        assert got.dtype == torch.bool and outside == 0, c["name"]
    ones = find_blocks_chunked(torch.rand(1, 2, 4, 4).cuda(), 0, 0.9, None, decoding=True, mode="prefill")
    assert ones.all()


def test_operator_with_kv_longer_than_q():
    """Chunked prefill against a KV cache (k_len > q_len): the block diagonal and the
    token-causal mask are bottom-right aligned (xattn/src/Xattention.py:39-40, 153-157, 257)."""
    from xattn.src.Xattention import Xattention_prefill, xattn_estimate
    from xattn.synthetic import WORKLOADS, make_inputs

    S, C, Lq, Lk, H, Hkv = 8, 2048, 2048, 6144, 8, 2
    q_all, k, v = make_inputs(WORKLOADS[1], device="cpu", seed=11, L=Lk, heads=H, kv_heads=Hkv)
    q = q_all[:, :, -Lq:].contiguous()
    kf, vf = k.repeat_interleave(H // Hkv, 1).float(), v.repeat_interleave(H // Hkv, 1).float()
    want_sums, want_mask = O.xattn_estimate(q.float(), kf, 128, S, threshold=0.9, chunk_size=C, pad0_quirk=False)
    sums, mask = xattn_estimate(q.cuda(), k.cuda(), 128, S, threshold=0.9, chunk_size=C)
    assert mask.shape == (1, H, Lq // 128, Lk // 128)
    nbad, outside = mask_mismatch_report(want_sums[0], mask[0], want_mask[0], 0.9, True, (Lk - Lq) // 128, C // 128)
    assert outside == 0 and nbad <= 2
    want = O.block_sparse_attention(q, k, v, want_mask, causal=True)
    out = Xattention_prefill(q.cuda(), k.cuda(), v.cuda(), S, threshold=0.9, chunk_size=C)
    if nbad == 0:
        err = (out.float().cpu() - want.float()).abs()
        assert err.max().item() <= OUT_MAX_ABS and err.mean().item() <= OUT_MEAN_ABS


def test_sums_beyond_a_forced_key_move_up_in_rank():
    """Un-normalised block sums (softmax=False) above 100000 * (1 + forced sum) rank before that forced block
    in the reference (xattn/src/utils.py:126-130) and are judged against less mass; hand-worked rows (see the
    oracle's test of the same name) and random rows whose sums straddle the forced keys."""
    rows = [([10.0, 5e6, 3e6, 2.0, 50.0], 4, 0.5, [1, 1, 1, 0, 1, 0, 0, 0]),
            ([10.0, 90.0, 30.0, 2.0, 50.0], 4, 0.5, [1, 1, 0, 0, 1, 0, 0, 0]),
            ([1.0, 4e5, 3.5e5, 1e5, 9e4, 2.0], 5, 0.85, [1, 1, 1, 1, 0, 1, 0, 0])]
    for vals, diag, tau, want in rows:
        x = torch.zeros(1, 1, 8)
        x[0, 0, : len(vals)] = torch.tensor(vals)
        got, _, _ = _select(x, tau, True, diag)
        assert got[0, 0].int().tolist() == want, (vals, got[0, 0].int().tolist())
    g = torch.Generator().manual_seed(11)
    for nk, off in [(40, 8), (300, 268), (1500, 1468), (32, 0)]:           # extraction path, sort path, first chunk
        nq = 32
        x = torch.exp(torch.rand(4, nq, nk, generator=g) * 18.0)             # sums from 1 to 6e7
        vis = torch.arange(nk)[None, :] <= torch.arange(nq)[:, None] + off
        x = x * vis
        taus = torch.tensor([0.3, 0.6, 0.9, 0.99])
        got, _, _ = _select(x, taus, True, off)
        want = O.find_blocks_chunked(x[None], off, taus, None, decoding=False, mode="prefill", causal=True)[0] & vis
        nbad, outside = mask_mismatch_report(x, got, want, taus, True, off)
        assert outside == 0, (nk, off, nbad, outside)
