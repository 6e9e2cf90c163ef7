"""GPU checks at the benchmark's full sizes, through properties that do not
need a full-size oracle run: row mass of the block sums, structure of the
mask, list/mask consistency, dense == sparse-with-every-block, linearity in
V, and oracle parity on sampled q-blocks (the oracle is run on just those
rows).  Plus operator edge cases at small sizes."""
import math

import pytest
import torch

from helpers import OUT_MAX_ABS, OUT_MEAN_ABS, lists_from_mask, mask_mismatch_report
from oracle import xattn_oracle as O

pytestmark = pytest.mark.gpu


def _sampled_block_parity(q, k, v, mask, out, causal, samples):
    """Oracle attention for single q-blocks (all keys) vs the kernel's output."""
    H, Hkv = q.shape[1], k.shape[1]
    L = q.shape[2]
    for h, qb in samples:
        r0, r1 = qb * 128, min(L, qb * 128 + 128)
        kend = r1 if causal else L
        kv = h // (H // Hkv)
        qq = q[:, h : h + 1, r0:r1].float().cpu()
        kk = k[:, kv : kv + 1, :kend].float().cpu()
        vv = v[:, kv : kv + 1, :kend].float().cpu()
        nkb = (kend + 127) // 128
        m = mask[h : h + 1, qb : qb + 1, :nkb].bool().cpu()[None]
        want = O.block_sparse_attention(qq, kk, vv, m, causal=causal)
        got = out[:, h : h + 1, r0:r1].float().cpu()
        err = (got - want).abs()
        assert err.max().item() <= OUT_MAX_ABS, (h, qb, err.max().item())
        assert err.mean().item() <= OUT_MEAN_ABS, (h, qb, err.mean().item())


@pytest.mark.parametrize("idx", [1, 2, 3, 4])
def test_full_size_workload_properties(idx):
    from xattn.src.Xattention import block_sparse_attention, default_chunk_size, estimate_and_select
    from xattn.synthetic import WORKLOADS, make_inputs

    w = WORKLOADS[idx]
    L, H, S = w.L, w.heads, w.stride
    q, k, v = make_inputs(w, device="cuda", seed=0)
    chunk = w.chunk_size or default_chunk_size(L)
    r = estimate_and_select(q, k, S, w.threshold, chunk, causal=w.causal)
    sums, mask, idx_t, cnt = r["sums"], r["mask"], r["col_idx"], r["col_cnt"]
    nb = (L + 127) // 128
    nbp = sums.shape[-1]
    rbs = 128 // S
    assert torch.isfinite(sums).all()
    # each fully real q-block row of the block sums carries mass block_size / stride
    full_rows = L // 128
    mass = sums[:, :full_rows].double().sum(-1)
    assert (mass - rbs).abs().max().item() < 5e-3
    if L % 128:
        part = sums[:, full_rows].double().sum(-1)
        assert (part - (L % 128) // S).abs().max().item() < 5e-3     # L % 128 is a multiple of S here
    assert (sums[:, nb:] == 0).all()                                   # padded q-block rows
    ar = torch.arange(nbp, device="cuda")
    if w.causal:
        upper = ar[None, :] > ar[:, None]
        assert (sums[:, upper] == 0).all()
        assert not mask[:, upper].any()
        assert mask[:, :nb, 0].all() and mask[:, ar[:nb], ar[:nb]].all()
    else:
        assert (sums[:, :nb, nb:] > 0).all() if nbp > nb else True    # zero-padded keys take mass
    # compacted lists == mask rows (cropped to real blocks)
    assert torch.equal(cnt[:, :nb].long(), mask[:, :nb, :nb].long().sum(-1))
    sel = torch.zeros((H, nb, nb), dtype=torch.bool, device="cuda")
    cols = torch.arange(idx_t.shape[-1], device="cuda")[None, None, :]
    valid = cols < cnt[:, :nb, None]
    hh, rr, _ = valid.nonzero(as_tuple=True)
    sel[hh, rr, idx_t[:, :nb][valid].long()] = True
    assert torch.equal(sel, mask[:, :nb, :nb].bool())

    out = block_sparse_attention(q, k, v, idx_t, cnt, causal=w.causal)
    assert torch.isfinite(out.float()).all()
    # deterministic samples: the (head, q-block) with the longest list, the median one, the first and the last
    # (ragged for workload 4) q-block, and one q-block of every KV group
    lens = cnt[:, :nb].long().reshape(-1).cpu()
    order = torch.argsort(lens)
    samples = [divmod(int(order[-1]), nb), divmod(int(order[len(order) // 2]), nb), (0, 0), (H - 1, nb - 1)]
    group = H // w.kv_heads
    g = torch.Generator().manual_seed(idx)
    for kvh in range(w.kv_heads):
        samples.append((kvh * group + int(torch.randint(group, (1,), generator=g)), int(torch.randint(nb, (1,), generator=g))))
    _sampled_block_parity(q, k, v, mask, out, w.causal, sorted(set(samples)))
    density = cnt[:, :nb].sum().item() / (H * (nb * (nb + 1) // 2 if w.causal else nb * nb))
    print(f"{w.name}: density {density:.4f}")


def test_dense_equals_full_list_and_linearity_in_v():
    from xattn.src.Xattention import block_sparse_attention
    from xattn.synthetic import WORKLOADS, make_inputs

    w = WORKLOADS[1]
    L, H = 8192, 8
    q, k, v = make_inputs(w, device="cuda", seed=1, L=L, heads=H, kv_heads=2)
    nb = L // 128
    full = torch.tril(torch.ones(nb, nb, dtype=torch.bool)).expand(H, nb, nb).contiguous()
    idx, cnt = lists_from_mask(full)
    a = block_sparse_attention(q, k, v, idx.cuda(), cnt.cuda(), causal=True)
    b = block_sparse_attention(q, k, v, causal=True)
    assert torch.equal(a, b)
    v2 = torch.randn_like(v)
    lin = block_sparse_attention(q, k, (v.float() + v2.float()).bfloat16(), causal=True).float()
    parts = b.float() + block_sparse_attention(q, k, v2, causal=True).float()
    assert (lin - parts).abs().max().item() < 6e-2


@pytest.mark.parametrize("L", [100, 129, 1000])
def test_tiny_and_ragged_lengths(L):
    from xattn.src.Xattention import Xattention_prefill, xattn_estimate

    g = torch.Generator().manual_seed(L)
    q, k, v = (torch.randn(1, 4, L, 128, generator=g).bfloat16() for _ in range(3))
    out = Xattention_prefill(q.cuda(), k.cuda(), v.cuda(), 8, threshold=0.9)
    want, wmask = O.Xattention_prefill(q.float(), k.float(), v.float(), 8, threshold=0.9, pad0_quirk=False, return_mask=True)
    _, mask = xattn_estimate(q.cuda(), k.cuda(), 128, 8, threshold=0.9, chunk_size=2048)
    nb = (L + 127) // 128
    assert torch.equal(mask[:, :, :nb, :nb].cpu(), wmask)
    err = (out.float().cpu() - want).abs()
    assert err.max().item() <= OUT_MAX_ABS and err.mean().item() <= OUT_MEAN_ABS


def test_threshold_forms_and_keep_flags():
    from xattn.src.Xattention import Xattention_prefill, block_sparse_attention, xattn_estimate
    from xattn.synthetic import WORKLOADS, make_inputs

    L, H, S, C = 4096, 8, 16, 2048
    q, k, v = make_inputs(WORKLOADS[1], device="cpu", seed=5, L=L, heads=H, kv_heads=2)
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    kf = k.repeat_interleave(4, 1).float()
    # tau = 1 keeps every causal block -> dense attention
    dense = block_sparse_attention(qc, kc, vc, causal=True)
    full = Xattention_prefill(qc, kc, vc, S, threshold=1.0, chunk_size=C)
    assert (full.float() - dense.float()).abs().max().item() <= OUT_MAX_ABS
    # per-head tensor thresholds (0 and 1 included), on another device than the inputs
    taus = torch.tensor([0.0, 0.9, 0.5, 1.0, 0.95, 0.0, 0.7, 0.9], dtype=torch.float32)
    _, m = xattn_estimate(qc, kc, 128, S, threshold=taus, chunk_size=C)
    wsums, wm = O.xattn_estimate(q.float(), kf, 128, S, threshold=taus, chunk_size=C, pad0_quirk=False)
    nbad, outside = mask_mismatch_report(wsums[0], m[0], wm[0], taus, True, 0, C // 128)
    assert outside == 0 and nbad <= 8, (nbad, outside)   # tau = 1.0 sits exactly on the band
    # tau = 0: forced blocks only (sink + diagonal, plus the first chunk's unconditional extra block)
    nb = L // 128
    assert m[0, 0].sum().item() <= 3 * nb
    # 0-d tensor threshold == float threshold
    _, m0 = xattn_estimate(qc, kc, 128, S, threshold=torch.tensor(0.9), chunk_size=C)
    _, m1 = xattn_estimate(qc, kc, 128, S, threshold=0.9, chunk_size=C)
    assert (m0 != m1).sum().item() <= 2
    for flags in (dict(keep_sink=True), dict(keep_recent=True), dict(keep_sink=True, keep_recent=True)):
        _, mk = xattn_estimate(qc, kc, 128, S, threshold=0.5, chunk_size=C, **flags)
        _, wk = O.xattn_estimate(q.float(), kf, 128, S, threshold=0.5, chunk_size=C, pad0_quirk=False, **flags)
        assert (mk.cpu() != wk).sum().item() <= 2, flags
        out = Xattention_prefill(qc, kc, vc, S, threshold=0.5, chunk_size=C, **flags)
        assert torch.isfinite(out.float()).all()
